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

// ---- packed operand layout ----------------------------------------------
// A matrix [rows, row_bytes] that feeds a GEMM as a K-contiguous operand can be
// kept "packed": 16 KiB blocks of 256 rows x 64 bytes, block (rt, kb) at
// (rt * KB + kb) * 16384 with KB = row_bytes / 64, and inside a block the
// 16-byte chunk c of row r at r * 64 + ((c ^ swz(r)) * 16),
// swz(r) = (r >> 2) & 3.  A block is exactly the LDS image the GEMM kernels
// compute from, so a tile load is a contiguous copy made of full cache lines.
// Rows are padded to a multiple of 256.  With this swizzle the kernels'
// ds_read_b128 fragment reads (lane = row, 64-byte row pitch) run at the full
// 256 bytes per clock of the LDS; measured alternatives: none 85, xor of
// (r>>1)^(r>>3) 158 bytes per clock.
__host__ __device__ inline int packed_swizzle(int r) { return (r >> 2) & 3; }
__host__ __device__ inline size_t packed_bytes(size_t rows, size_t row_bytes) {
    return (rows + 255) / 256 * (row_bytes / 64) * 16384;
}
// Byte offset of the byte `kbyte` (within its row) of row r; KB = row_bytes / 64.
__host__ __device__ inline size_t packed_offset(int r, int kbyte, int KB) {
    const int rp = r & 255;
    const int sw = packed_swizzle(rp);
    return ((size_t)(r >> 8) * KB + (kbyte >> 6)) * 16384 + rp * 64 + ((((kbyte >> 4) & 3) ^ sw) << 4) +
           (kbyte & 15);
}

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
