// bf16 GEMM, 256x256 macro tile, hand-scheduled main loop (gfx950).
//
// Same operand roles (weights feed the MFMA "A" operand, activations "B") and
// the same epilogue as the generic kernel in gemm.hip.  The whole K loop is one
// inline-asm block (gemm_bf16_256_loop.inc, produced by gen_gemm_asm.py; the
// pipeline, LDS map and register plan are described there) so that the order
// of MFMAs, LDS fragment reads, global->LDS loads and waits is exactly the one
// that keeps a single wave per SIMD busy.  Used when K is a multiple of 128
// elements and the problem has enough tiles.
#include "gemm_common.h"

namespace cubert {
namespace {

using namespace gemm_detail;

#define CUBERT_ACC_OPERANDS                                                                              \
    [c00] "=&a"(acc[0][0]), [c01] "=&a"(acc[0][1]), [c02] "=&a"(acc[0][2]), [c03] "=&a"(acc[0][3]),         \
    [c10] "=&a"(acc[1][0]), [c11] "=&a"(acc[1][1]), [c12] "=&a"(acc[1][2]), [c13] "=&a"(acc[1][3]),         \
    [c20] "=&a"(acc[2][0]), [c21] "=&a"(acc[2][1]), [c22] "=&a"(acc[2][2]), [c23] "=&a"(acc[2][3]),         \
    [c30] "=&a"(acc[3][0]), [c31] "=&a"(acc[3][1]), [c32] "=&a"(acc[3][2]), [c33] "=&a"(acc[3][3])

#define CUBERT_V10(b) "v" #b "0", "v" #b "1", "v" #b "2", "v" #b "3", "v" #b "4", "v" #b "5", "v" #b "6", "v" #b "7", "v" #b "8", "v" #b "9"

template <int OUT, int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_t256_kernel(const GemmDev p) {
    constexpr int BT = 256;
    // Four stages of 32 KiB: W tile (256 rows x 64 B) then X tile.
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * 32768];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave >> 1, wm = wave & 1;
    const int l32 = lane & 31, g = lane >> 5;

    int tile_n, tile_m;
    if constexpr (EPI == kEpiBiasResLN) {
        ln_tile_of_block(blockIdx.x, p.tiles_n, &tile_n, &tile_m);
        if (tile_m >= p.tiles_m) return;          // the grid is padded to whole groups of eight bands
    } else {
        tile_of_block(blockIdx.x, p.tiles_n * p.tiles_m, p.tiles_n, p.xn_parts, &tile_n, &tile_m);
    }
    const int n0 = tile_n * BT, m0 = tile_m * BT;

    // Buffer descriptors as plain SGPR quads: base, base_hi (stride 0), num_records, flags.
    // Rows outside the matrix read as zero (bounds check on the lane offset).
    const unsigned long long wa = reinterpret_cast<unsigned long long>(p.W);
    const unsigned long long xa = reinterpret_cast<unsigned long long>(p.X);
    const unsigned wsize = p.w_packed ? (unsigned)packed_bytes(p.N, (size_t)p.K * 2) : (unsigned)((size_t)p.N * p.K * 2);
    const unsigned xsize = p.x_packed ? (unsigned)packed_bytes(p.M, (size_t)p.K * 2)
                                      : (unsigned)((((size_t)p.M - 1) * p.ldx + p.K) * 2);
    const u32x4_t wres = {(unsigned)wa, (unsigned)(wa >> 32) & 0xffffu, wsize, 0x00020000u};
    const u32x4_t xres = {(unsigned)xa, (unsigned)(xa >> 32) & 0xffffu, xsize, 0x00020000u};
    const int w_rowb = p.K * 2, x_rowb = p.ldx * 2;
    const int KB = p.K * 2 / 64;
    // global->LDS: one load moves 16 rows x 64 bytes.  Wave w moves the row groups w, w+4,
    // w+8, w+12 of each tile.
    //   unpacked source: lane fetches row 16*group + lane/4 and the chunk that belongs into
    //     its LDS slot lane%4 (slot = chunk ^ swz(row)); row groups start at multiples of 16, so
    //     swz only depends on the lane.  One half-step further along K is +64 bytes.
    //   packed source: a tile's half-step is one contiguous 16 KiB block, the next one follows it.
    const int dc = (lane & 3) ^ packed_swizzle(lane >> 2);
    const int w_v0 = p.w_packed ? (tile_n * KB * 16384 + wave * 1024 + lane * 16)
                                : ((n0 + 16 * wave + (lane >> 2)) * w_rowb + (dc << 4));
    const int x_v0 = p.x_packed ? (tile_m * KB * 16384 + wave * 1024 + lane * 16)
                                : ((m0 + 16 * wave + (lane >> 2)) * x_rowb + (dc << 4));
    const int w64 = p.w_packed ? 4096 : 64 * w_rowb, x64 = p.x_packed ? 4096 : 64 * x_rowb;
    const int wkstep = p.w_packed ? 16384 : 64, xkstep = p.x_packed ? 16384 : 64;
    // fragment reads: chunk g of my row in the W / X tile of stage 0, k-phase 0
    const int lds_base = (int)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const int sw = packed_swizzle(l32);
    const int wb = lds_base + (wn * 128 + l32) * 64 + ((g ^ sw) << 4);
    const int xb = lds_base + 16384 + (wm * 128 + l32) * 64 + ((g ^ sw) << 4);
    const int m0b = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
    const int ht = p.K / 32;          // half-steps; a multiple of 4

    f32x16_t acc[4][4];       // zeroed inside the asm block
    f32x4_t bias[16];
    if constexpr (!gemm_bias_at_readout<OUT, EPI>()) gemm_load_bias<4>(p, n0 + wn * 128, g, bias);

    asm volatile(
#include "gemm_bf16_256_loop.inc"
        : CUBERT_ACC_OPERANDS
        : [wb] "v"(wb), [xb] "v"(xb), [wv0] "v"(w_v0), [xv0] "v"(x_v0), [wres] "s"(wres), [xres] "s"(xres),
          [w64] "s"(w64), [x64] "s"(x64), [ht] "s"(ht), [m0b] "s"(m0b), [wkstep] "s"(wkstep), [xkstep] "s"(xkstep)
        : "memory", "scc", "m0", "s92", "s93", "s94", "s95", "s96", "s97", "s98", "v96", "v97", "v98", "v99",
          CUBERT_V10(10), CUBERT_V10(11), CUBERT_V10(12), CUBERT_V10(13), CUBERT_V10(14), CUBERT_V10(15), CUBERT_V10(16),
          "v170", "v171", "v172", "v173", "v174", "v175");

    // Stages 0 and 1 were last read two barriers ago; the tail of the loop only reads stages
    // 2 and 3, so the first 64 KiB are free for the epilogue's staging while slower waves finish.
    // (The LayerNorm epilogue keeps its row statistics above them, after a barrier of its own.)
    if constexpr (EPI == kEpiBiasResLN)
        gemm_epilogue_ln<4, 4>(p, acc, n0 + wn * 128, m0 + wm * 128, l32, g, tile_m, 2 * tile_n + wn, lds + wave * 16384,
                               reinterpret_cast<float*>(lds + 65536 + wave * 1024));
    else
        gemm_epilogue<OUT, EPI, 4, 4, false, 8, true>(p, acc, bias, n0 + wn * 128, m0 + wm * 128, l32, g, lds + wave * 16384);
}

// ---------------------------------------------------------------------------
// 256 features x 128 tokens per workgroup, two workgroups per CU (loop:
// gemm_bf16_256x128_loop.inc, "half" mode of gen_gemm_asm.py).  A wave owns 128 x 64
// = 4 x 2 accumulator blocks and stays below 128 VGPRs, so each SIMD holds one wave of
// each workgroup: the prologue, epilogue and launch gap of one workgroup overlap the
// other's main loop.  Costs 1.5x the LDS fragment traffic per flop of the 256 x 256 tile.
#define CUBERT_ACC_OPERANDS_H                                                                            \
    [c00] "=&a"(acc[0][0]), [c01] "=&a"(acc[0][1]), [c10] "=&a"(acc[1][0]), [c11] "=&a"(acc[1][1]),         \
    [c20] "=&a"(acc[2][0]), [c21] "=&a"(acc[2][1]), [c30] "=&a"(acc[3][0]), [c31] "=&a"(acc[3][1])

template <int OUT, int EPI>
__global__ __launch_bounds__(256, 2) void gemm_bf16_t256x128_kernel(const GemmDev p) {
    // Three stages of 24 KiB: W tile (256 rows x 64 B) at +0, X tile (128 rows x 64 B) at +0x4000.
    __shared__ __attribute__((aligned(1024))) unsigned char lds[3 * 24576];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave >> 1, wm = wave & 1;
    const int l32 = lane & 31, g = lane >> 5;

    int tile_n, tile_m;
    if constexpr (EPI == kEpiBiasResLN) {
        ln_tile_of_block(blockIdx.x, p.tiles_n, &tile_n, &tile_m);
        if (tile_m >= p.tiles_m) return;          // the grid is padded to whole groups of eight bands
    } else {
        tile_of_block<8>(blockIdx.x, p.tiles_n * p.tiles_m, p.tiles_n, p.xn_parts, &tile_n, &tile_m);
    }
    const int n0 = tile_n * 256, m0 = tile_m * 128;

    const unsigned long long wa = reinterpret_cast<unsigned long long>(p.W);
    const unsigned long long xa = reinterpret_cast<unsigned long long>(p.X);
    const unsigned wsize = p.w_packed ? (unsigned)packed_bytes(p.N, (size_t)p.K * 2) : (unsigned)((size_t)p.N * p.K * 2);
    const unsigned xsize = p.x_packed ? (unsigned)packed_bytes(p.M, (size_t)p.K * 2)
                                      : (unsigned)((((size_t)p.M - 1) * p.ldx + p.K) * 2);
    const u32x4_t wres = {(unsigned)wa, (unsigned)(wa >> 32) & 0xffffu, wsize, 0x00020000u};
    const u32x4_t xres = {(unsigned)xa, (unsigned)(xa >> 32) & 0xffffu, xsize, 0x00020000u};
    const int w_rowb = p.K * 2, x_rowb = p.ldx * 2;
    const int KB = p.K * 2 / 64;
    // One load moves 16 rows x 64 bytes.  Wave w moves the W row groups w, w+4, w+8, w+12 and the
    // X row groups w, w+4 of each tile (see the 256 x 256 kernel for the chunk choice `dc`).
    const int dc = (lane & 3) ^ packed_swizzle(lane >> 2);
    const int w_v0 = p.w_packed ? (tile_n * KB * 16384 + wave * 1024 + lane * 16)
                                : ((n0 + 16 * wave + (lane >> 2)) * w_rowb + (dc << 4));
    const int x_v0 = p.x_packed ? ((m0 >> 8) * KB * 16384 + (m0 & 255) * 64 + wave * 1024 + lane * 16)
                                : ((m0 + 16 * wave + (lane >> 2)) * x_rowb + (dc << 4));
    const int w64 = p.w_packed ? 4096 : 64 * w_rowb, x64 = p.x_packed ? 4096 : 64 * x_rowb;
    const int wkstep = p.w_packed ? 16384 : 64, xkstep = p.x_packed ? 16384 : 64;
    const int lds_base = (int)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const int sw = packed_swizzle(l32);
    const int wb = lds_base + (wn * 128 + l32) * 64 + ((g ^ sw) << 4);
    const int xb = lds_base + (wm * 64 + l32) * 64 + ((g ^ sw) << 4);       // + 0x4000 is in the read offsets
    const int m0b = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
    const int ht = p.K / 32;
    const int wkmax = (ht - 1) * wkstep, xkmax = (ht - 1) * xkstep;      // K offset of the last tile

    f32x16_t acc[4][2];       // zeroed inside the asm block

    asm volatile(
#include "gemm_bf16_256x128_loop.inc"
        : CUBERT_ACC_OPERANDS_H
        : [wb] "v"(wb), [xb] "v"(xb), [wv0] "v"(w_v0), [xv0] "v"(x_v0), [wres] "s"(wres), [xres] "s"(xres),
          [w64] "s"(w64), [x64] "s"(x64), [ht] "s"(ht), [m0b] "s"(m0b), [wkstep] "s"(wkstep), [xkstep] "s"(xkstep),
          [wkmax] "s"(wkmax), [xkmax] "s"(xkmax)
        : "memory", "scc", "m0", "s92", "s93", "s94", "s96", "s97", "s98", "v64", "v65", "v66", "v67", "v68", "v69",
          CUBERT_V10(7), CUBERT_V10(8), CUBERT_V10(9), CUBERT_V10(10), CUBERT_V10(11), "v120", "v121", "v122",
          "v123", "v124", "v125");

    // The block ends with all loads landed and a barrier: the whole LDS is free for staging.
    f32x4_t bias[16];
    if constexpr (!gemm_bias_at_readout<OUT, EPI>()) gemm_load_bias<4>(p, n0 + wn * 128, g, bias);
    if constexpr (EPI == kEpiBiasResLN)
        gemm_epilogue_ln<4, 2>(p, acc, n0 + wn * 128, m0 + wm * 64, l32, g, tile_m, 2 * tile_n + wn, lds + wave * 16384,
                               reinterpret_cast<float*>(lds + 65536 + wave * 1024));
    else
        gemm_epilogue<OUT, EPI, 4, 2, false, 8, true>(p, acc, bias, n0 + wn * 128, m0 + wm * 64, l32, g, lds + wave * 16384);
}

// ---------------------------------------------------------------------------
// The same 256 features x 128 tokens tile for launches of at most one workgroup per CU (a few thousand token
// rows): loop gemm_bf16_256x128_deep_loop.inc ("deep" mode of gen_gemm_asm.py), i.e. the four-stage pipeline of the
// 256 x 256 kernel -- loads three half-steps ahead, fragment reads one k-phase ahead across the barrier.  The two-per-CU
// kernel above leaves the matrix pipe idle about half of the time when a workgroup has its CU to itself (it waits
// for the last fragment reads of every half-step and then for the barrier, with nothing running beside it).
// Needs K to be a multiple of 128; plain, GELU, QKV and residual epilogues.
template <int OUT, int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_t256x128_deep_kernel(const GemmDev p) {
    // Four stages of 24 KiB: W tile (256 rows x 64 B) at +0, X tile (128 rows x 64 B) at +0x4000.
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * 24576];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave >> 1, wm = wave & 1;
    const int l32 = lane & 31, g = lane >> 5;

    int tile_n, tile_m;
    tile_of_block<8>(blockIdx.x, p.tiles_n * p.tiles_m, p.tiles_n, p.xn_parts, &tile_n, &tile_m);
    const int n0 = tile_n * 256, m0 = tile_m * 128;

    const unsigned long long wa = reinterpret_cast<unsigned long long>(p.W);
    const unsigned long long xa = reinterpret_cast<unsigned long long>(p.X);
    const unsigned wsize = p.w_packed ? (unsigned)packed_bytes(p.N, (size_t)p.K * 2) : (unsigned)((size_t)p.N * p.K * 2);
    const unsigned xsize = p.x_packed ? (unsigned)packed_bytes(p.M, (size_t)p.K * 2)
                                      : (unsigned)((((size_t)p.M - 1) * p.ldx + p.K) * 2);
    const u32x4_t wres = {(unsigned)wa, (unsigned)(wa >> 32) & 0xffffu, wsize, 0x00020000u};
    const u32x4_t xres = {(unsigned)xa, (unsigned)(xa >> 32) & 0xffffu, xsize, 0x00020000u};
    const int w_rowb = p.K * 2, x_rowb = p.ldx * 2;
    const int KB = p.K * 2 / 64;
    const int dc = (lane & 3) ^ packed_swizzle(lane >> 2);
    const int w_v0 = p.w_packed ? (tile_n * KB * 16384 + wave * 1024 + lane * 16)
                                : ((n0 + 16 * wave + (lane >> 2)) * w_rowb + (dc << 4));
    const int x_v0 = p.x_packed ? ((m0 >> 8) * KB * 16384 + (m0 & 255) * 64 + wave * 1024 + lane * 16)
                                : ((m0 + 16 * wave + (lane >> 2)) * x_rowb + (dc << 4));
    const int w64 = p.w_packed ? 4096 : 64 * w_rowb, x64 = p.x_packed ? 4096 : 64 * x_rowb;
    const int wkstep = p.w_packed ? 16384 : 64, xkstep = p.x_packed ? 16384 : 64;
    const int lds_base = (int)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const int sw = packed_swizzle(l32);
    const int wb = lds_base + (wn * 128 + l32) * 64 + ((g ^ sw) << 4);
    const int xb = lds_base + 0x4000 + (wm * 64 + l32) * 64 + ((g ^ sw) << 4);
    const int m0b = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
    const int ht = p.K / 32;          // half-steps; a multiple of 4

    f32x16_t acc[4][2];       // zeroed inside the asm block

    asm volatile(
#include "gemm_bf16_256x128_deep_loop.inc"
        : CUBERT_ACC_OPERANDS_H
        : [wb] "v"(wb), [xb] "v"(xb), [wv0] "v"(w_v0), [xv0] "v"(x_v0), [wres] "s"(wres), [xres] "s"(xres),
          [w64] "s"(w64), [x64] "s"(x64), [ht] "s"(ht), [m0b] "s"(m0b), [wkstep] "s"(wkstep), [xkstep] "s"(xkstep)
        : "memory", "scc", "m0", "s92", "s93", "s94", "s95", "s96", "s97", "s98", "v64", "v65", "v66", "v67", "v68", "v69",
          CUBERT_V10(7), CUBERT_V10(8), CUBERT_V10(9), CUBERT_V10(10), CUBERT_V10(11), "v120", "v121", "v122",
          "v123", "v124", "v125");

    // Slower waves may still be multiplying out of the last two stages: everybody is through before the
    // epilogue reuses the memory.  (All loads have landed: the tail waits for them.)
    __syncthreads();
    f32x4_t bias[16];
    if constexpr (!gemm_bias_at_readout<OUT, EPI>()) gemm_load_bias<4>(p, n0 + wn * 128, g, bias);
    gemm_epilogue<OUT, EPI, 4, 2, false, 8, true>(p, acc, bias, n0 + wn * 128, m0 + wm * 64, l32, g, lds + wave * 16384);
}

template <int OUT>
bool launch_epi_half_deep(const GemmDev& d, int epi, hipStream_t stream) {
    const dim3 grid(d.tiles_n * d.tiles_m), block(256);
    switch (epi) {
        case kEpiBias: hipLaunchKernelGGL((gemm_bf16_t256x128_deep_kernel<OUT, kEpiBias>), grid, block, 0, stream, d); break;
        case kEpiBiasGelu: hipLaunchKernelGGL((gemm_bf16_t256x128_deep_kernel<OUT, kEpiBiasGelu>), grid, block, 0, stream, d); break;
        case kEpiBiasTanh: hipLaunchKernelGGL((gemm_bf16_t256x128_deep_kernel<OUT, kEpiBiasTanh>), grid, block, 0, stream, d); break;
        case kEpiQKV: hipLaunchKernelGGL((gemm_bf16_t256x128_deep_kernel<OUT, kEpiQKV>), grid, block, 0, stream, d); break;
        case kEpiQKVMap: hipLaunchKernelGGL((gemm_bf16_t256x128_deep_kernel<OUT, kEpiQKVMap>), grid, block, 0, stream, d); break;
        case kEpiBiasRes:
            if constexpr (OUT == kF32) {
                hipLaunchKernelGGL((gemm_bf16_t256x128_deep_kernel<OUT, kEpiBiasRes>), grid, block, 0, stream, d);
                break;
            }
            [[fallthrough]];
        default: set_error("gemm: unknown epilogue"); return false;
    }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

// LayerNorm epilogue: eight XCDs x whole groups of bands x the workgroups of a band (ln_tile_of_block);
// workgroups whose band does not exist leave at once.
dim3 ln_grid(const GemmDev& d) { return dim3(8 * d.tiles_n * ((d.tiles_m + 7) / 8)); }

template <int OUT>
bool launch_epi_half(const GemmDev& d, int epi, hipStream_t stream) {
    const dim3 grid(d.tiles_n * d.tiles_m), block(256);
    switch (epi) {
        case kEpiBias: hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiBias>), grid, block, 0, stream, d); break;
        case kEpiBiasGelu: hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiBiasGelu>), grid, block, 0, stream, d); break;
        case kEpiBiasTanh: hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiBiasTanh>), grid, block, 0, stream, d); break;
        case kEpiQKV: hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiQKV>), grid, block, 0, stream, d); break;
        case kEpiQKVMap: hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiQKVMap>), grid, block, 0, stream, d); break;
        case kEpiBiasRes:
            if constexpr (OUT == kF32) {
                hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiBiasRes>), grid, block, 0, stream, d);
                break;
            }
            [[fallthrough]];
        case kEpiBiasResLN:
            if constexpr (OUT == kF32) {
                if (epi == kEpiBiasResLN) {
                    hipLaunchKernelGGL((gemm_bf16_t256x128_kernel<OUT, kEpiBiasResLN>), ln_grid(d), block, 0, stream, d);
                    break;
                }
            }
            [[fallthrough]];
        default: set_error("gemm: unknown epilogue"); return false;
    }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

template <int OUT>
bool launch_epi(const GemmDev& d, int epi, hipStream_t stream) {
    const dim3 grid(d.tiles_n * d.tiles_m), block(256);
    switch (epi) {
        case kEpiBias: hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiBias>), grid, block, 0, stream, d); break;
        case kEpiBiasGelu: hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiBiasGelu>), grid, block, 0, stream, d); break;
        case kEpiBiasTanh: hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiBiasTanh>), grid, block, 0, stream, d); break;
        case kEpiQKV: hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiQKV>), grid, block, 0, stream, d); break;
        case kEpiQKVMap: hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiQKVMap>), grid, block, 0, stream, d); break;
        case kEpiBiasRes:
            if constexpr (OUT == kF32) {
                hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiBiasRes>), grid, block, 0, stream, d);
                break;
            }
            [[fallthrough]];
        case kEpiBiasResLN:
            if constexpr (OUT == kF32) {
                if (epi == kEpiBiasResLN) {
                    hipLaunchKernelGGL((gemm_bf16_t256_kernel<OUT, kEpiBiasResLN>), ln_grid(d), block, 0, stream, d);
                    break;
                }
            }
            [[fallthrough]];
        default: set_error("gemm: unknown epilogue"); return false;
    }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

}  // namespace

// d.tiles_n / d.tiles_m must have been computed for a 256 tile and d.K % 128 == 0.
bool launch_gemm_bf16_t256(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream) {
    if (d.K % 128 != 0 || d.K < 128) { set_error("gemm: the 256 tile needs K to be a multiple of 128"); return false; }
    return out_elt == kBF16 ? launch_epi<kBF16>(d, epilogue, stream) : launch_epi<kF32>(d, epilogue, stream);
}


// 256 x 128 tile, one workgroup per CU: d.tiles_n for 256 features, d.tiles_m for 128 tokens; d.K % 128 == 0.
bool launch_gemm_bf16_t256x128_deep(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream) {
    if (d.K % 128 != 0 || d.K < 128) { set_error("gemm: the one-per-CU 256x128 tile needs K to be a multiple of 128"); return false; }
    return out_elt == kBF16 ? launch_epi_half_deep<kBF16>(d, epilogue, stream) : launch_epi_half_deep<kF32>(d, epilogue, stream);
}

// 256 x 128 tile: d.tiles_n for 256 features, d.tiles_m for 128 tokens; d.K % 32 == 0, K >= 64.
bool launch_gemm_bf16_t256x128(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream) {
    if (d.K % 32 != 0 || d.K < 64) { set_error("gemm: the 256x128 tile needs K to be a multiple of 32, at least 64"); return false; }
    return out_elt == kBF16 ? launch_epi_half<kBF16>(d, epilogue, stream) : launch_epi_half<kF32>(d, epilogue, stream);
}

}  // namespace cubert
