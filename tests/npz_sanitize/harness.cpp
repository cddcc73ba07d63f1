// Host-only harness of the npz reader (infmoe_amd/csrc/npz_reader.cpp), built with AddressSanitizer and
// UndefinedBehaviorSanitizer by tests/test_npz_sanitize.py: the reader is the one piece of the library that
// parses a file somebody else wrote (the reference hands the same job to a modified cnpy,
// plugin/thirdparty/cnpy/cnpy.cpp:109-276).
//   harness ROWS COLS FILE...
// For every file: open it, list its members, and read each as float32 of shape (ROWS, COLS), (COLS, ROWS) and
// (ROWS,) into exactly sized buffers.  Whatever the file holds, every call has to come back with a status -
// no crash, no report from a sanitizer.  Prints one line per file: <OK|status of open> <members> <reads that succeeded>.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "npz_reader.h"

namespace infmoe {
std::string& last_error_slot() {
    static thread_local std::string slot;
    return slot;
}
}  // namespace infmoe

int main(int argc, char** argv) {
    if (argc < 4) return 2;
    const size_t rows = strtoul(argv[1], nullptr, 10), cols = strtoul(argv[2], nullptr, 10);
    for (int i = 3; i < argc; ++i) {
        infmoe::NpzReader npz;
        const infmoe::Status opened = npz.open(argv[i]);
        size_t members = 0, good = 0;
        if (opened == INFMOE_OK) {
            const std::vector<std::string> names = npz.names();
            members = names.size();
            for (const std::string& n : names) {
                std::vector<float> a(rows * cols), b(rows * cols), c(rows);
                good += npz.read_f32(n.c_str(), a.data(), rows, cols) == INFMOE_OK;
                good += npz.read_f32(n.c_str(), b.data(), cols, rows) == INFMOE_OK;
                good += npz.read_f32(n.c_str(), c.data(), rows, 0) == INFMOE_OK;
            }
            (void)npz.has("no/such member");
        }
        printf("%d %zu %zu\n", (int)opened, members, good);
    }
    return 0;
}
