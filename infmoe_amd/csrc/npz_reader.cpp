#include "npz_reader.h"

#include <sys/stat.h>
#include <zlib.h>

#include <algorithm>
#include <cstring>

namespace infmoe {
namespace {

uint16_t rd16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }
uint32_t rd32(const uint8_t* p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
uint64_t rd64(const uint8_t* p) { return (uint64_t)rd32(p) | ((uint64_t)rd32(p + 4) << 32); }

constexpr uint32_t kSigLocal = 0x04034b50, kSigCentral = 0x02014b50, kSigEocd = 0x06054b50;
constexpr uint32_t kSigEocd64 = 0x06064b50, kSigEocd64Loc = 0x07064b50;

struct NpyHeader {
    bool fortran = false;
    std::string descr;
    std::vector<uint64_t> shape;
    size_t data_offset = 0;  // from the start of the member
};

// header: magic "\x93NUMPY", major, minor, header length (u16 for v1, u32 for v2/3), python dict
Status parse_npy_header(const uint8_t* buf, size_t n, NpyHeader* h) {
    if (n < 10 || memcmp(buf, "\x93NUMPY", 6) != 0) return fail(INFMOE_ERR_IO, "npz member is not an npy array");
    const int major = buf[6];
    size_t hlen, hoff;
    if (major == 1) {
        hlen = rd16(buf + 8), hoff = 10;
    } else {
        if (n < 12) return fail(INFMOE_ERR_IO, "truncated npy header");
        hlen = rd32(buf + 8), hoff = 12;
    }
    if (hoff + hlen > n) return fail(INFMOE_ERR_IO, "npy header longer than expected");
    const std::string dict(reinterpret_cast<const char*>(buf + hoff), hlen);
    h->data_offset = hoff + hlen;
    // value of `key`: position of the first character after "'key' :" and blanks, or npos
    auto value_of = [&](const char* key) -> size_t {
        size_t p = dict.find(key);
        if (p == std::string::npos) return p;
        p = dict.find(':', p);
        if (p == std::string::npos) return p;
        return dict.find_first_not_of(" ", p + 1);
    };
    size_t p = value_of("'descr'");
    if (p == std::string::npos || dict[p] != '\'') return fail(INFMOE_ERR_IO, "npy header without a descr string");
    const size_t q = dict.find('\'', p + 1);
    if (q == std::string::npos) return fail(INFMOE_ERR_IO, "bad npy descr");
    h->descr = dict.substr(p + 1, q - p - 1);
    p = value_of("'fortran_order'");
    if (p == std::string::npos) return fail(INFMOE_ERR_IO, "npy header without fortran_order");
    if (dict.compare(p, 4, "True") == 0) h->fortran = true;
    else if (dict.compare(p, 5, "False") == 0) h->fortran = false;
    else return fail(INFMOE_ERR_IO, "bad npy fortran_order");
    p = value_of("'shape'");
    if (p == std::string::npos || dict[p] != '(') return fail(INFMOE_ERR_IO, "npy header without a shape tuple");
    const size_t e = dict.find(')', p);
    if (e == std::string::npos) return fail(INFMOE_ERR_IO, "bad npy shape");
    uint64_t v = 0;
    bool in_num = false;
    for (size_t i = p + 1; i <= e; ++i) {
        const char c = dict[i];
        if (c >= '0' && c <= '9') {
            v = v * 10 + (uint64_t)(c - '0');
            in_num = true;
        } else if (in_num) {
            h->shape.push_back(v);
            v = 0;
            in_num = false;
        }
    }
    return INFMOE_OK;
}

}  // namespace

NpzReader::~NpzReader() {
    if (mFile) fclose(mFile);
}

Status NpzReader::read_at(uint64_t off, void* dst, size_t n) {
    if (fseeko(mFile, (off_t)off, SEEK_SET) != 0 || fread(dst, 1, n, mFile) != n)
        return fail(INFMOE_ERR_IO, "%s: short read at offset %llu", mPath.c_str(), (unsigned long long)off);
    return INFMOE_OK;
}

Status NpzReader::open(const char* path) {
    mPath = path ? path : "";
    struct stat st {};
    if (path == nullptr || stat(path, &st) != 0) return fail(INFMOE_ERR_IO, "cannot stat weight file: %s", mPath.c_str());
    if (!S_ISREG(st.st_mode)) return fail(INFMOE_ERR_IO, "weight file must be a regular file: %s", mPath.c_str());
    mFile = fopen(path, "rb");
    if (!mFile) return fail(INFMOE_ERR_IO, "cannot open weight file: %s", mPath.c_str());
    const uint64_t fsize = (uint64_t)st.st_size;
    // end-of-central-directory record: search the last 64 KiB + 22 bytes
    const size_t tail = (size_t)std::min<uint64_t>(fsize, 65557);
    std::vector<uint8_t> buf(tail);
    INFMOE_TRY(read_at(fsize - tail, buf.data(), tail));
    ssize_t eocd = -1;
    for (ssize_t i = (ssize_t)tail - 22; i >= 0; --i)
        if (rd32(&buf[i]) == kSigEocd) {
            eocd = i;
            break;
        }
    if (eocd < 0) return fail(INFMOE_ERR_IO, "%s: not a zip archive (no end record)", mPath.c_str());
    uint64_t n_entries = rd16(&buf[eocd + 10]), cd_size = rd32(&buf[eocd + 12]), cd_off = rd32(&buf[eocd + 16]);
    if (eocd >= 20 && rd32(&buf[eocd - 20]) == kSigEocd64Loc) {
        const uint64_t e64 = rd64(&buf[eocd - 20 + 8]);
        uint8_t r[56];
        INFMOE_TRY(read_at(e64, r, sizeof(r)));
        if (rd32(r) != kSigEocd64) return fail(INFMOE_ERR_IO, "%s: bad zip64 end record", mPath.c_str());
        n_entries = rd64(r + 32), cd_size = rd64(r + 40), cd_off = rd64(r + 48);
    }
    if (cd_off > fsize || cd_size > fsize - cd_off)
        return fail(INFMOE_ERR_IO, "%s: central directory lies outside the file", mPath.c_str());
    mFileSize = fsize;
    std::vector<uint8_t> cd((size_t)cd_size);
    INFMOE_TRY(read_at(cd_off, cd.data(), cd.size()));
    size_t p = 0;
    for (uint64_t k = 0; k < n_entries; ++k) {
        if (p + 46 > cd.size() || rd32(&cd[p]) != kSigCentral) return fail(INFMOE_ERR_IO, "%s: bad central directory", mPath.c_str());
        Entry en;
        en.method = rd16(&cd[p + 10]);
        en.comp_size = rd32(&cd[p + 20]);
        en.uncomp_size = rd32(&cd[p + 24]);
        const size_t nlen = rd16(&cd[p + 28]), xlen = rd16(&cd[p + 30]), clen = rd16(&cd[p + 32]);
        en.local_offset = rd32(&cd[p + 42]);
        if (p + 46 + nlen + xlen + clen > cd.size()) return fail(INFMOE_ERR_IO, "%s: truncated central directory", mPath.c_str());
        std::string name(reinterpret_cast<const char*>(&cd[p + 46]), nlen);
        // zip64 extended information: present values replace the 0xFFFFFFFF fields, in this order
        size_t x = p + 46 + nlen;
        const size_t xend = x + xlen;
        while (x + 4 <= xend) {
            const uint16_t id = rd16(&cd[x]), sz = rd16(&cd[x + 2]);
            if (id == 0x0001) {
                size_t y = x + 4;
                if (en.uncomp_size == 0xFFFFFFFFu && y + 8 <= xend) en.uncomp_size = rd64(&cd[y]), y += 8;
                if (en.comp_size == 0xFFFFFFFFu && y + 8 <= xend) en.comp_size = rd64(&cd[y]), y += 8;
                if (en.local_offset == 0xFFFFFFFFu && y + 8 <= xend) en.local_offset = rd64(&cd[y]), y += 8;
            }
            x += 4 + sz;
        }
        if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
        mEntries[name] = en;
        p += 46 + nlen + xlen + clen;
    }
    return INFMOE_OK;
}

bool NpzReader::has(const char* name) const { return mEntries.count(name) != 0; }

std::vector<std::string> NpzReader::names() const {
    std::vector<std::string> v;
    for (auto& kv : mEntries) v.push_back(kv.first);
    return v;
}

Status NpzReader::read_f32(const char* name_in, float* dst, size_t rows, size_t cols) {
    const size_t count = rows * (cols ? cols : 1);
    std::string name(name_in);
    if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
    auto it = mEntries.find(name);
    if (it == mEntries.end()) return fail(INFMOE_ERR_MISSING_FIELD, "%s: no array named %s", mPath.c_str(), name.c_str());
    const Entry& en = it->second;
    uint8_t lh[30];
    INFMOE_TRY(read_at(en.local_offset, lh, sizeof(lh)));
    if (rd32(lh) != kSigLocal) return fail(INFMOE_ERR_IO, "%s: bad local header for %s", mPath.c_str(), name.c_str());
    const uint64_t data_off = en.local_offset + 30 + rd16(lh + 26) + rd16(lh + 28);
    if (data_off > mFileSize || en.comp_size > mFileSize - data_off)
        return fail(INFMOE_ERR_IO, "%s: member %s lies outside the file", mPath.c_str(), name.c_str());
    if (en.uncomp_size > ((uint64_t)1 << 40)) return fail(INFMOE_ERR_IO, "%s: member %s is implausibly large", mPath.c_str(), name.c_str());

    std::vector<uint8_t> raw;  // the uncompressed member (header + data) when deflated
    NpyHeader h;
    const uint8_t* payload = nullptr;
    std::vector<uint8_t> head;
    if (en.method == 0) {
        head.resize((size_t)std::min<uint64_t>(en.uncomp_size, 4096));
        INFMOE_TRY(read_at(data_off, head.data(), head.size()));
        INFMOE_TRY(parse_npy_header(head.data(), head.size(), &h));
    } else if (en.method == 8) {
        std::vector<uint8_t> comp((size_t)en.comp_size);
        INFMOE_TRY(read_at(data_off, comp.data(), comp.size()));
        raw.resize((size_t)en.uncomp_size);
        z_stream zs{};
        if (inflateInit2(&zs, -MAX_WBITS) != Z_OK) return fail(INFMOE_ERR_IO, "zlib init failed");
        size_t in_done = 0, out_done = 0;
        int rc = Z_OK;
        while (rc != Z_STREAM_END) {  // zlib counts in 32 bits: feed it in slices
            zs.next_in = comp.data() + in_done;
            zs.avail_in = (uInt)std::min<size_t>(comp.size() - in_done, 1u << 30);
            zs.next_out = raw.data() + out_done;
            zs.avail_out = (uInt)std::min<size_t>(raw.size() - out_done, 1u << 30);
            const uInt in0 = zs.avail_in, out0 = zs.avail_out;
            rc = inflate(&zs, Z_NO_FLUSH);
            in_done += in0 - zs.avail_in;
            out_done += out0 - zs.avail_out;
            if (rc != Z_OK && rc != Z_STREAM_END) break;
            if (in0 == zs.avail_in && out0 == zs.avail_out) break;  // no progress
        }
        inflateEnd(&zs);
        if (rc != Z_STREAM_END || out_done != raw.size())
            return fail(INFMOE_ERR_IO, "%s: inflate failed for %s", mPath.c_str(), name.c_str());
        INFMOE_TRY(parse_npy_header(raw.data(), raw.size(), &h));
        payload = raw.data() + h.data_offset;
    } else {
        return fail(INFMOE_ERR_IO, "%s: unsupported zip compression method %u for %s", mPath.c_str(), en.method, name.c_str());
    }

    if (h.descr != "<f4" && h.descr != "=f4" && h.descr != "|f4" && h.descr != "f4")
        return fail(INFMOE_ERR_IO, "%s: %s has dtype %s, expected little-endian float32", mPath.c_str(), name.c_str(), h.descr.c_str());
    uint64_t elems = 1;
    std::string shape_text = "(";
    for (uint64_t s : h.shape) {
        if (s != 0 && elems > UINT64_MAX / s) return fail(INFMOE_ERR_IO, "%s: %s has an overflowing shape", mPath.c_str(), name.c_str());
        elems *= s;
        shape_text += std::to_string(s) + ",";
    }
    shape_text += ")";
    // The reference asserts on the byte count only (plugin/sublayers/T5FFLayer.cc:62,69,76,83), so a
    // matrix saved transposed ([d][h] where [h][d] is meant: same count) passes there; here the shape
    // has to be the expected one.
    const bool shape_ok = cols == 0 ? (h.shape.size() == 1 && h.shape[0] == rows)
                                    : (h.shape.size() == 2 && h.shape[0] == rows && h.shape[1] == cols);
    if (!shape_ok || elems != count)
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "%s: %s has shape %s, expected (%zu,%s)", mPath.c_str(), name.c_str(),
                    shape_text.c_str(), rows, cols ? std::to_string(cols).c_str() : "");
    if (h.data_offset > en.uncomp_size || elems * 4 > en.uncomp_size - h.data_offset)
        return fail(INFMOE_ERR_IO, "%s: %s is shorter than its header says", mPath.c_str(), name.c_str());

    const bool transpose = h.fortran && h.shape.size() == 2 && h.shape[0] > 1 && h.shape[1] > 1;
    if (h.fortran && h.shape.size() > 2) return fail(INFMOE_ERR_UNSUPPORTED, "%s: Fortran-ordered arrays above 2-D are not supported", name.c_str());
    std::vector<float> tmp;
    float* target = dst;
    if (transpose) {
        tmp.resize(count);
        target = tmp.data();
    }
    if (payload) {
        memcpy(target, payload, count * sizeof(float));
    } else {
        INFMOE_TRY(read_at(data_off + h.data_offset, target, count * sizeof(float)));
    }
    if (transpose) {  // element (i,j) of the logical [r][c] array sits at j*r + i in the file
        const size_t r = (size_t)h.shape[0], c = (size_t)h.shape[1];
        for (size_t i = 0; i < r; ++i)
            for (size_t j = 0; j < c; ++j) dst[i * c + j] = tmp[j * r + i];
    }
    return INFMOE_OK;
}

}  // namespace infmoe
