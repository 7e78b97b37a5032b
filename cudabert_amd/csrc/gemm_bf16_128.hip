// bf16 GEMM, 128 x 128 macro tile, hand-scheduled main loop, three workgroups per CU (gfx950).
//
// For problems whose 256-row tiles would leave most of the chip idle (a few hundred to a few thousand
// token rows: short batches, the latency regime) and for the split-K launches of such batches.  Same
// operand roles and epilogue as the other kernels (gemm.hip, gemm_bf16_256.hip); the K loop is
// gemm_bf16_128_loop.inc ("quarter" mode of gen_gemm_asm.py, which describes the pipeline).  A wave owns
// 64 features x 64 tokens = 2 x 2 accumulator blocks (64 AGPRs) and the kernel stays within 168
// registers and 48 KiB of LDS, so every SIMD holds three waves of three different workgroups: while one
// workgroup waits for its first tiles or stores its results, the other two have the matrix pipe.
#include "gemm_common.h"

namespace cubert {
namespace {

using namespace gemm_detail;

#define CUBERT_ACC_OPERANDS_Q [c00] "=&a"(acc[0][0]), [c01] "=&a"(acc[0][1]), [c10] "=&a"(acc[1][0]), [c11] "=&a"(acc[1][1])
#define CUBERT_V10(b) "v" #b "0", "v" #b "1", "v" #b "2", "v" #b "3", "v" #b "4", "v" #b "5", "v" #b "6", "v" #b "7", "v" #b "8", "v" #b "9"

template <int OUT, int EPI>
__global__ __launch_bounds__(256, 3) void gemm_bf16_t128_kernel(const GemmDev p) {
    // Three stages of 16 KiB: W tile (128 rows x 64 B) at +0, X tile (128 rows x 64 B) at +0x2000.
    __shared__ __attribute__((aligned(1024))) unsigned char lds[3 * 16384];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave >> 1, wm = wave & 1;
    const int l32 = lane & 31, g = lane >> 5;

    int tile_n, tile_m;
    tile_of_block<8>(blockIdx.x, p.tiles_n * p.tiles_m, p.tiles_n, p.xn_parts, &tile_n, &tile_m);
    const int n0 = tile_n * 128, m0 = tile_m * 128;

    // Buffer descriptors as plain SGPR quads; rows outside the matrix read as zero (bounds check on the lane offset).
    const unsigned long long wa = reinterpret_cast<unsigned long long>(p.W);
    const unsigned long long xa = reinterpret_cast<unsigned long long>(p.X);
    const unsigned wsize = p.w_packed ? (unsigned)packed_bytes(p.N, (size_t)p.K * 2) : (unsigned)((size_t)p.N * p.K * 2);
    const unsigned xsize = p.x_packed ? (unsigned)packed_bytes(p.M, (size_t)p.K * 2)
                                      : (unsigned)((((size_t)p.M - 1) * p.ldx + p.K) * 2);
    const u32x4_t wres = {(unsigned)wa, (unsigned)(wa >> 32) & 0xffffu, wsize, 0x00020000u};
    const u32x4_t xres = {(unsigned)xa, (unsigned)(xa >> 32) & 0xffffu, xsize, 0x00020000u};
    const int w_rowb = p.K * 2, x_rowb = p.ldx * 2;
    const int KB = p.K * 2 / 64;
    // One load moves 16 rows x 64 bytes.  Wave w moves the row groups w and w + 4 of the W tile and of the X
    // tile (unpacked source: the lane fetches the chunk that belongs into its LDS slot, see the 256 x 256 kernel).
    const int dc = (lane & 3) ^ packed_swizzle(lane >> 2);
    const int w_v0 = p.w_packed ? ((n0 >> 8) * KB * 16384 + (n0 & 255) * 64 + wave * 1024 + lane * 16)
                                : ((n0 + 16 * wave + (lane >> 2)) * w_rowb + (dc << 4));
    const int x_v0 = p.x_packed ? ((m0 >> 8) * KB * 16384 + (m0 & 255) * 64 + wave * 1024 + lane * 16)
                                : ((m0 + 16 * wave + (lane >> 2)) * x_rowb + (dc << 4));
    const int w64 = p.w_packed ? 4096 : 64 * w_rowb, x64 = p.x_packed ? 4096 : 64 * x_rowb;
    const int wkstep = p.w_packed ? 16384 : 64, xkstep = p.x_packed ? 16384 : 64;
    const int lds_base = (int)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const int sw = packed_swizzle(l32);
    const int wb = lds_base + (wn * 64 + l32) * 64 + ((g ^ sw) << 4);
    const int xb = lds_base + (wm * 64 + l32) * 64 + ((g ^ sw) << 4);       // + 0x2000 is in the read offsets
    const int m0b = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
    // half-steps of this workgroup: all of K, or (split K) the blockIdx.y-th share of it
    const int hs = p.K / 32;
    const int h0 = (int)((long)hs * blockIdx.y / p.splits), h1 = (int)((long)hs * (blockIdx.y + 1) / p.splits);
    const int ht = h1 - h0;
    const int wk0 = h0 * wkstep, xk0 = h0 * xkstep;
    const int wkmax = (h1 - 1) * wkstep, xkmax = (h1 - 1) * xkstep;      // K offset of my last tile

    f32x16_t acc[2][2];       // zeroed inside the asm block
    asm volatile(
#include "gemm_bf16_128_loop.inc"
        : CUBERT_ACC_OPERANDS_Q
        : [wb] "v"(wb), [xb] "v"(xb), [wv0] "v"(w_v0), [xv0] "v"(x_v0), [wres] "s"(wres), [xres] "s"(xres),
          [w64] "s"(w64), [x64] "s"(x64), [ht] "s"(ht), [m0b] "s"(m0b), [wkstep] "s"(wkstep), [xkstep] "s"(xkstep),
          [wkmax] "s"(wkmax), [xkmax] "s"(xkmax), [wk0] "s"(wk0), [xk0] "s"(xk0)
        : "memory", "scc", "m0", "s92", "s93", "s94", "s96", "s97", "s98", "v48", "v49", CUBERT_V10(5), CUBERT_V10(6),
          CUBERT_V10(7), CUBERT_V10(8), "v90", "v91");

    // The block ends with all loads landed and a barrier: the whole LDS is free for staging (8 KiB per wave).
    f32x4_t bias[8];
    constexpr bool SPLITK = (EPI == kEpiBias || EPI == kEpiBiasRes) && OUT == kF32;      // the only combinations launch_gemm splits
    if constexpr (!gemm_bias_at_readout<OUT, EPI>()) gemm_load_bias<2, SPLITK>(p, n0 + wn * 64, g, bias);
    gemm_epilogue<OUT, EPI, 2, 2, SPLITK, 4, true>(p, acc, bias, n0 + wn * 64, m0 + wm * 64, l32, g, lds + wave * 8192);
}

template <int OUT>
bool launch_epi(const GemmDev& d, int epi, hipStream_t stream) {
    const dim3 grid(d.tiles_n * d.tiles_m, d.splits), block(256);
    switch (epi) {
        case kEpiBias: hipLaunchKernelGGL((gemm_bf16_t128_kernel<OUT, kEpiBias>), grid, block, 0, stream, d); break;
        case kEpiBiasGelu: hipLaunchKernelGGL((gemm_bf16_t128_kernel<OUT, kEpiBiasGelu>), grid, block, 0, stream, d); break;
        case kEpiBiasTanh: hipLaunchKernelGGL((gemm_bf16_t128_kernel<OUT, kEpiBiasTanh>), grid, block, 0, stream, d); break;
        case kEpiQKV: hipLaunchKernelGGL((gemm_bf16_t128_kernel<OUT, kEpiQKV>), grid, block, 0, stream, d); break;
        case kEpiQKVMap: hipLaunchKernelGGL((gemm_bf16_t128_kernel<OUT, kEpiQKVMap>), grid, block, 0, stream, d); break;
        case kEpiBiasRes:
            if constexpr (OUT == kF32) {
                hipLaunchKernelGGL((gemm_bf16_t128_kernel<OUT, kEpiBiasRes>), grid, block, 0, stream, d);
                break;
            }
            [[fallthrough]];
        default: set_error("gemm: unknown epilogue"); return false;
    }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

}  // namespace

// 128 x 128 tile: d.tiles_n / d.tiles_m for 128 features / tokens; d.K % 32 == 0; 1 <= d.splits <= K / 32.
bool launch_gemm_bf16_t128(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream) {
    if (d.K % 32 != 0 || d.K < 32 || d.splits < 1 || d.splits > d.K / 32) {
        set_error("gemm: the hand-scheduled 128 tile needs K to be a multiple of 32 and at most K / 32 splits");
        return false;
    }
    return out_elt == kBF16 ? launch_epi<kBF16>(d, epilogue, stream) : launch_epi<kF32>(d, epilogue, stream);
}

}  // namespace cubert
