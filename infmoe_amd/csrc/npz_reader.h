// Reader for numpy .npz archives of float32 arrays: what the reference gets from its modified
// copy of cnpy (plugin/thirdparty/cnpy/cnpy.cpp:109-276), written from the zip and npy format
// descriptions.  It reads the central directory (so zip64 archives larger than 4 GiB and entries
// whose local header carries no sizes both work), supports stored and deflated members, and
// honours `fortran_order` for 2-D arrays (cnpy parses the flag but ignores it, and the
// reference's own generator saves a transposed view, python/infmoe/config.py:52).
#pragma once

#include <cstdint>
#include <cstdio>
#include <map>
#include <string>
#include <vector>

#include "status.h"

namespace infmoe {

class NpzReader {
   public:
    ~NpzReader();
    Status open(const char* path);
    bool has(const char* name) const;
    // Reads member `name` (with or without the ".npy" suffix) into dst as C-ordered float32; fails
    // unless it is '<f4' of shape (rows, cols), or (rows,) when cols == 0.
    Status read_f32(const char* name, float* dst, size_t rows, size_t cols);
    std::vector<std::string> names() const;

   private:
    struct Entry {
        uint64_t local_offset, comp_size, uncomp_size;
        uint16_t method;
    };
    FILE* mFile = nullptr;
    std::string mPath;
    uint64_t mFileSize = 0;
    std::map<std::string, Entry> mEntries;
    Status read_at(uint64_t off, void* dst, size_t n);
};

}  // namespace infmoe
