// Minimal reader for NumPy ``.npy`` files holding little-endian float32 data.
//
// Replaces the part of the vendored cnpy the reference's loader uses
// (cuda_bert/cnpy/cnpy.cpp:108-165 header parse, :339-349 npy_load).  Unlike
// cnpy it accepts format versions 1.0, 2.0 and 3.0, rejects Fortran order
// (cnpy parses the flag at :119-123 and then ignores it) and reports errors
// as values rather than C++ exceptions thrown across the C boundary.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace cubert {

struct NpyArray {
    std::vector<size_t> shape;
    std::vector<float> data;
    size_t numel() const {
        size_t n = 1;
        for (size_t s : shape) n *= s;
        return n;
    }
};

// Parses the header dictionary text.  Returns false and fills `err` on any
// malformed or unsupported header.
bool npy_parse_header(const std::string& header, std::vector<size_t>* shape,
                      std::string* descr, bool* fortran, std::string* err);

// Reads one file.  Only descr '<f4' (or '|f4'/'=f4' on this little-endian
// host) is accepted.
bool npy_load_f32(const std::string& path, NpyArray* out, std::string* err);

}  // namespace cubert
