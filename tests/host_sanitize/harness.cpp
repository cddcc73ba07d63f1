// Host code of the library under AddressSanitizer + UndefinedBehaviorSanitizer (no GPU needed): built by
// tests/test_host_sanitize.py from the library's own .cpp files with g++ and the sanitizers, linked with the
// device objects the normal build left behind (they are only referenced, never run here).
//   harness BLOB_FILE...      or      harness --create SEED COUNT
// Every file is handed to infmoe_deserialize, which parses bytes somebody else wrote (the reference reads the
// same kind of blob back from a TensorRT engine file, plugin/MoELayerPlugin.cc:104-143).  A layer that comes
// back is configured, asked for its workspace size, serialised again, cloned and destroyed.  Whatever the bytes
// are, every call has to return a status: no crash, no sanitizer report.  One line per file:
//   <status of deserialize> <bytes of the re-serialised layer or 0>
// --create: COUNT field collections drawn from SEED go to infmoe_create - fields missing, doubled, unknown,
// with lengths of 0, with null data, with sizes that do not fit each other, strings that are not terminated - and a
// layer that comes back goes through the same host-side calls.  Prints how many were accepted.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "infmoe.h"

static std::vector<unsigned char> slurp(const char* path) {
    std::vector<unsigned char> v;
    if (FILE* f = fopen(path, "rb")) {
        unsigned char buf[4096];
        size_t n;
        while ((n = fread(buf, 1, sizeof(buf), f)) > 0) v.insert(v.end(), buf, buf + n);
        fclose(f);
    }
    return v;
}

static void exercise(infmoe_plugin* p, int d) {
    const int32_t dims[3] = {2, 8, d};
    size_t ws = 0, n = 0;
    if (infmoe_configure(p, dims, 3) == INFMOE_OK) (void)infmoe_workspace_size(p, dims, 3, &ws);
    if (infmoe_serialization_size(p, &n) == INFMOE_OK) {
        std::vector<unsigned char> out(n);
        infmoe_plugin* back = nullptr;
        if (infmoe_serialize(p, out.data(), out.size()) == INFMOE_OK &&
            infmoe_deserialize("again", out.data(), out.size(), &back) == INFMOE_OK)
            infmoe_destroy(back);
    }
    float w[8] = {0};
    (void)infmoe_set_expert_weights(p, 0, "wi_weight", w, 8);
    (void)infmoe_set_expert_weights(p, 1 << 20, "wo_weight", w, 8);
    (void)infmoe_set_expert_weights(p, 0, "no_such_key", w, 8);
    (void)infmoe_set_score_bias(p, nullptr);
    infmoe_plugin* twin = nullptr;
    if (infmoe_clone(p, &twin) == INFMOE_OK) infmoe_destroy(twin);
}

static int fuzz_create(unsigned seed, int count) {
    unsigned state = seed * 2654435761u + 12345u;
    auto rnd = [&](unsigned n) { state = state * 1664525u + 1013904223u; return (state >> 10) % n; };
    int accepted = 0;
    for (int it = 0; it < count; ++it) {
        const int sizes[] = {0, -1, 1, 2, 3, 4, 8, 16, 130};
        int E = sizes[rnd(9)], d = sizes[rnd(9)], h = sizes[rnd(9)], mc = sizes[rnd(9)];
        if (rnd(4)) E = 1 + (int)rnd(6), d = 4 << rnd(3), h = 8 << rnd(3), mc = 1 + (int)rnd(4);  // mostly sane sizes
        const size_t nc = rnd(5) == 0 ? rnd(40) : (size_t)(E > 0 ? E : 0) * (size_t)(d > 0 ? d : 0);
        const size_t nl = rnd(5) == 0 ? rnd(40) : (size_t)(d > 0 ? d : 0);
        std::vector<float> cent(nc, 0.25f), gamma(nl, 1.0f);
        const char* variants[] = {"cpm_2", "base_layer", "default", "Default", "", "cpm_2x"};
        const char* subs[] = {"T5_FF", "Identity", "t5_ff", ""};
        const char* norms[] = {"rms", "centered", "none"};
        const char* ffns[] = {"relu", "gated_gelu", "gelu"};
        // strings are handed over length-delimited, in exactly sized buffers without a terminator
        auto text = [&](const char* v) { return std::vector<char>(v, v + strlen(v)); };
        const unsigned vi = rnd(5) ? rnd(3) : rnd(6), si = rnd(6) ? rnd(2) : rnd(4);  // mostly names that exist
        const std::vector<char> variant = text(variants[vi]), sub = text(subs[si]), norm = text(norms[rnd(6) ? rnd(2) : 2]),
                                ffn = text(ffns[rnd(6) ? rnd(2) : 2]), file = text(rnd(2) ? "/nonexistent/weights.npz" : "/tmp");
        std::vector<infmoe_field> f;
        auto add = [&](const char* name, const void* data, int type, int length) {
            if (rnd(40) == 0) return;                       // missing
            infmoe_field x{name, data, type, length};
            if (rnd(60) == 0) x.length = 0;
            if (rnd(60) == 0) x.data = nullptr;
            if (rnd(60) == 0) x.type = INFMOE_FIELD_INT32 + (int)rnd(4);
            f.push_back(x);
            if (rnd(20) == 0) f.push_back(x);               // doubled
        };
        add("expert_count", &E, INFMOE_FIELD_INT32, 1);
        add("embedding_size", &d, INFMOE_FIELD_INT32, 1);
        add("hidden_size", &h, INFMOE_FIELD_INT32, 1);
        add("max_concurrency", &mc, INFMOE_FIELD_INT32, 1);
        add("expert_centroids", cent.data(), INFMOE_FIELD_FLOAT32, (int)cent.size());
        if (vi == 0 ? rnd(10) != 0 : rnd(2)) add("layernorm_weight", gamma.data(), INFMOE_FIELD_FLOAT32, (int)gamma.size());
        add("expert_sublayer_type", sub.data(), INFMOE_FIELD_UNKNOWN, (int)sub.size());
        add("moe_variant", variant.data(), INFMOE_FIELD_UNKNOWN, (int)variant.size());
        if (rnd(3) == 0) add("norm_kind", norm.data(), INFMOE_FIELD_CHAR, (int)norm.size());
        if (rnd(3) == 0) add("ffn_kind", ffn.data(), INFMOE_FIELD_CHAR, (int)ffn.size());
        if (rnd(4) == 0) add("expert_weight_file", file.data(), INFMOE_FIELD_CHAR, (int)file.size());
        if (rnd(15) == 0) add("no_such_field", &E, INFMOE_FIELD_INT32, 1);
        infmoe_plugin* p = nullptr;
        const int32_t status = infmoe_create(rnd(5) ? "layer" : nullptr, f.empty() ? nullptr : f.data(), (int)f.size(), &p);
        if (status == INFMOE_OK && p != nullptr) {
            ++accepted;
            exercise(p, d);
            infmoe_destroy(p);
        } else if (infmoe_last_error()[0] == 0) {
            printf("status %d without a message\n", (int)status);
            return -1;
        }
    }
    return accepted;
}

int main(int argc, char** argv) {
    if (argc == 4 && strcmp(argv[1], "--create") == 0) {
        const int accepted = fuzz_create((unsigned)strtoul(argv[2], nullptr, 10), atoi(argv[3]));
        printf("accepted %d\n", accepted);
        return accepted < 0;
    }
    for (int i = 1; i < argc; ++i) {
        // an exactly sized heap copy, so that a read past the end is a report and not a lucky zero
        const std::vector<unsigned char> blob = slurp(argv[i]);
        unsigned char* exact = static_cast<unsigned char*>(malloc(blob.size() ? blob.size() : 1));
        for (size_t k = 0; k < blob.size(); ++k) exact[k] = blob[k];
        infmoe_plugin* p = nullptr;
        const int32_t status = infmoe_deserialize("fuzzed", exact, blob.size(), &p);
        free(exact);
        size_t again = 0;
        if (status == INFMOE_OK && p != nullptr) {
            const int32_t dims[3] = {2, 8, 0};
            int32_t d3[3] = {dims[0], dims[1], 0};
            size_t ws = 0;
            for (int d = 1; d <= 4096; d *= 2) {  // the embedding size is not known here: try until one configures
                d3[2] = d;
                if (infmoe_configure(p, d3, 3) == INFMOE_OK) {
                    (void)infmoe_workspace_size(p, d3, 3, &ws);
                    break;
                }
            }
            if (infmoe_serialization_size(p, &again) == INFMOE_OK) {
                std::vector<unsigned char> out(again);
                if (infmoe_serialize(p, out.data(), out.size()) != INFMOE_OK) again = 0;
            }
            infmoe_plugin* twin = nullptr;
            if (infmoe_clone(p, &twin) == INFMOE_OK) infmoe_destroy(twin);
            infmoe_destroy(p);
        }
        printf("%d %zu\n", (int)status, again);
    }
    return 0;
}
