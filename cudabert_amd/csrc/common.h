// Shared host/device definitions for the gfx950 BERT encoder engine.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

namespace cubert {

enum Precision : int { kF32 = 0, kBF16 = 1 };

struct Dims {
    int hidden = 768;
    int layers = 12;
    int heads = 12;
    int inter = 3072;
    int vocab = 30522;
    int max_pos = 512;
    int type_vocab = 2;
};

// bf16 storage type used on the host side of the launch interface.
typedef uint16_t bf16_t;

// Round-to-nearest-even float -> bf16 (host).
inline bf16_t f32_to_bf16_host(float f) {
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t((u >> 16) | 0x40);   // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return bf16_t(u >> 16);
}

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }

// Thread-local last error text (returned by cubert_last_error()).
void set_error(const std::string& msg);
const char* get_error();

#define CUBERT_HIP_OK(expr)                                                              \
    do {                                                                                 \
        hipError_t _e = (expr);                                                          \
        if (_e != hipSuccess) {                                                          \
            ::cubert::set_error(std::string(#expr) + " failed: " + hipGetErrorString(_e)); \
            return false;                                                                \
        }                                                                                \
    } while (0)

}  // namespace cubert
