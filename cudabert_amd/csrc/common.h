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
// Attention kernels (launch_attention's `variant`).
constexpr int kAttnAuto = 0, kAttnPerHead = 1, kAttnSplitKeys = 2;
constexpr int kAttnSplitMaxWorkgroups = 768; // B * heads * ceil(S / 32) up to which kAttnAuto takes the key-split kernel

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

// ---- LayerNorm statistics -------------------------------------------------
// Every LayerNorm of the engine (the row kernels and the GEMM epilogue that normalises) forms its
// row statistics the same way, so that a row gets the same bits whichever kernel handles it.
// The row is cut into slots of 128 features; in a slot 32 lanes hold four consecutive features each.
// Per slot (ln_slot_stats): the sum, (a + b) + (c + d) per lane combined by ln_half_wave_sum, and M2, the
// sum of squared distances from the slot's own mean, taken the same way.  ln_row_mean adds the slot sums
// in slot order starting from zero; ln_merge_slot adds, again in slot order, M2_s + n_s (mean_s - mean)^2
// (the pairwise update of Chan et al. for a known total mean); ln_finalize turns the total into
// 1 / sigma (biased variance, eps 1e-12 inside the square root: modeling.py:168-172).  No difference of
// large squares is formed anywhere, so a row whose mean is many sigma away from zero keeps its
// precision, as with the running (Welford) statistics of cuda_bert/ops/layernorm.cu:27-67, 100-135.
// The helpers spell out their fused multiply-adds so that every caller compiles to the same arithmetic.
#if defined(__HIPCC__)
template <int CTRL>
__device__ __forceinline__ float ln_dpp_lanes(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// Sum over the 32 lanes that share lane / 32; every lane gets the same bits (the additions are
// pairwise and commutative).
// v combined with the value of the lane 32 further (or back): gfx950's v_permlane32_swap exchanges the upper half of
// one register with the lower half of another, so of two copies of v one ends up holding v of the lower lane of each
// pair in both halves and the other v of the upper lane; sum and maximum commute, so the result has the bits of
// v + shfl_xor(v, 32) / max(v, shfl_xor(v, 32)) without the trip through the LDS crossbar.  (Inline asm, with the wait
// states the instruction needs after a vector write of its operands and before a vector read of its results: the
// compiler's builtin returns the first register twice.)
__device__ __forceinline__ void half_swap(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float half_swap_sum(float v) {
    float a = v, b = v;
    half_swap(a, b);
    return a + b;
}
__device__ __forceinline__ float half_swap_max(float v) {
    float a = v, b = v;
    half_swap(a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float ln_half_wave_sum(float v) {
    v += ln_dpp_lanes<0xB1>(v);       // quad_perm [1,0,3,2]: lane ^ 1
    v += ln_dpp_lanes<0x4E>(v);       // quad_perm [2,3,0,1]: lane ^ 2
    v += ln_dpp_lanes<0x141>(v);      // row_half_mirror: the other quad of 8 lanes
    v += ln_dpp_lanes<0x140>(v);      // row_mirror: the other 8 of 16 lanes
    v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));   // lane ^ 16
    return v;
}
__device__ __forceinline__ float ln_sum4(float a, float b, float c, float d) { return (a + b) + (c + d); }
__device__ __forceinline__ float ln_sumsq4(float a, float b, float c, float d) {
#pragma clang fp contract(off)
    return __builtin_fmaf(a, a, b * b) + __builtin_fmaf(c, c, d * d);
}
// Statistics of one slot.  (a, b, c, d): this lane's four features, zeros if the lane lies past the end of
// the row (`in` false); inv_count = 1 / (features of the row inside this slot), 1 / 128 for a full slot.
__device__ __forceinline__ void ln_slot_stats(float a, float b, float c, float d, bool in, float inv_count, float* sum,
                                              float* m2) {
#pragma clang fp contract(off)
    const float s = ln_half_wave_sum(ln_sum4(a, b, c, d));
    const float mu = s * inv_count;
    const float da = in ? a - mu : 0.0f, db = in ? b - mu : 0.0f, dc = in ? c - mu : 0.0f, dd = in ? d - mu : 0.0f;
    *sum = s;
    *m2 = ln_half_wave_sum(ln_sumsq4(da, db, dc, dd));
}
__device__ __forceinline__ float ln_row_mean(float sum_of_slot_sums, float inv_n) {
#pragma clang fp contract(off)
    return sum_of_slot_sums * inv_n;
}
// m2 + (M2 of a slot about the row mean); count = features in the slot (0: the slot lies past the row).
__device__ __forceinline__ float ln_merge_slot(float m2, float slot_sum, float slot_m2, float count, float inv_count, float mean) {
#pragma clang fp contract(off)
    const float dm = slot_sum * inv_count - mean;
    return m2 + __builtin_fmaf(count * dm, dm, slot_m2);
}
__device__ __forceinline__ float ln_finalize(float m2, float inv_n) {
#pragma clang fp contract(off)
    return 1.0f / sqrtf(m2 * inv_n + 1e-12f);
}
__device__ __forceinline__ float ln_apply(float x, float mean, float rstd, float gamma, float beta) {
#pragma clang fp contract(off)
    return __builtin_fmaf(gamma, (x - mean) * rstd, beta);
}
#endif

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
