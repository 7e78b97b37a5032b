// MFMA GEMM for gfx950 (MI355X):  Y = epilogue(X * W^T + bias).
//
// Both operands are K-contiguous ([rows, K]); a workgroup of four wave64s
// computes a BT x BT macro tile (BT features x BT tokens), each wave a
// (BT/2) x (BT/2) quadrant built from 32x32 MFMA blocks.  Per K step a slab of
// 128 bytes per row (64 bf16 / 32 f32) of both operands is staged through LDS
// (double buffered, one barrier per step).  LDS rows are 128 bytes = eight
// 16-byte chunks; chunk c of row r lives at position c ^ ((r ^ (r >> 3)) & 7)
// so that the 16-byte fragment reads of 8 (or 16) consecutive rows hit
// distinct banks.
//
// The weight tile feeds the MFMA "A" operand and the activation tile the "B"
// operand, i.e. the hardware computes Y^T blocks: a lane then owns one token
// and four consecutive output features per accumulator quad, which makes the
// row-major stores 8/16-byte vectors and lets the QKV epilogue write per-head
// layouts directly.
//
// The k index inside one MFMA is only a label: lane (row, g = lane / 32) feeds
// the 16-byte chunk 2*kk + g of its row for both operands, so A and B always
// pair identical k.  For f32 each chunk holds four k values consumed by four
// 32x32x2 MFMAs; for bf16 it holds eight consumed by one 32x32x16 MFMA.
#include "kernels.h"

namespace cubert {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

struct GemmDev {
    const unsigned char* X;
    const unsigned char* W;
    const float* bias;
    unsigned char* Y;
    unsigned char* q;
    unsigned char* k;
    unsigned char* vt;
    int M, N, K, ldx;
    int S, Sp, heads, hidden;
    int tiles_n, tiles_m;
};

__device__ __forceinline__ float gelu_erf(float x) {
    return x * 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
}

template <int ELT>
__device__ __forceinline__ void mfma_chunk(const u32x4_t& a, const u32x4_t& b, f32x16_t& acc) {
    if constexpr (ELT == kBF16) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                      __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
    } else {
        const f32x4_t fa = __builtin_bit_cast(f32x4_t, a);
        const f32x4_t fb = __builtin_bit_cast(f32x4_t, b);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0], fb[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1], fb[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[2], fb[2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[3], fb[3], acc, 0, 0, 0);
    }
}

template <int OUT>
__device__ __forceinline__ void store4(unsigned char* base, size_t elem_index, const float v[4]) {
    if constexpr (OUT == kBF16) {
        bf16x4_t o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
        *reinterpret_cast<bf16x4_t*>(base + elem_index * 2) = o;
    } else {
        f32x4_t o = {v[0], v[1], v[2], v[3]};
        *reinterpret_cast<f32x4_t*>(base + elem_index * 4) = o;
    }
}

template <int OUT>
__device__ __forceinline__ void store1(unsigned char* base, size_t elem_index, float v) {
    if constexpr (OUT == kBF16) {
        *reinterpret_cast<__bf16*>(base + elem_index * 2) = (__bf16)v;
    } else {
        *reinterpret_cast<float*>(base + elem_index * 4) = v;
    }
}

// Workgroup id -> (tile_n, tile_m).  Hardware hands consecutive workgroup ids
// to the eight XCDs round-robin; the remap gives every XCD one contiguous run
// of the tile sequence so tiles sharing operand rows share an L2.
__device__ __forceinline__ void tile_of_block(int pid, int total, int tiles_n, int* tn, int* tm) {
    const int xcd = pid & 7, idx = pid >> 3;
    const int base = total >> 3, rem = total & 7;
    const int start = xcd * base + (xcd < rem ? xcd : rem);
    const int t = start + idx;
    *tm = t / tiles_n;
    *tn = t - *tm * tiles_n;
}

template <int ELT, int OUT, int EPI, int BT>
__global__ __launch_bounds__(256) void gemm_kernel(const GemmDev p) {
    constexpr int ES = (ELT == kBF16) ? 2 : 4;       // operand element size
    constexpr int NB = BT / 64;                      // 32x32 blocks per wave and dimension
    constexpr int PASSES = BT / 32;                  // 32 tile rows are loaded per pass
    constexpr int TILE_BYTES = BT * 128;             // one operand tile in LDS
    constexpr int BK = 128 / ES;                     // K elements per step

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave >> 1, wm = wave & 1;
    const int l32 = lane & 31, g = lane >> 5;

    int tile_n, tile_m;
    tile_of_block(blockIdx.x, p.tiles_n * p.tiles_m, p.tiles_n, &tile_n, &tile_m);
    const int n0 = tile_n * BT, m0 = tile_m * BT;

    // ---- global -> register staging through buffer resources ----
    // Out-of-range rows (edge tiles) read as zero: the hardware bounds check of
    // the buffer descriptor replaces per-row clamping.  The check covers the
    // lane offset only, so the row part lives there and just the K offset
    // (always in range) goes into the scalar offset.
    const int ld_row = tid >> 3, ld_chunk = tid & 7;
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char*>(p.W), 0, (int)((size_t)p.N * p.K * ES), 0x00020000);
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char*>(p.X), 0, (int)((((size_t)p.M - 1) * p.ldx + p.K) * ES), 0x00020000);
    const int w_rowb = p.K * ES, x_rowb = p.ldx * ES;
    const int w_voff = ld_row * w_rowb + ld_chunk * 16;
    const int x_voff = ld_row * x_rowb + ld_chunk * 16;
    const int c0 = ld_chunk ^ ((ld_row ^ (ld_row >> 3)) & 7);
    const int st_even = ld_row * 128 + (c0 << 4);
    const int st_odd = ld_row * 128 + ((c0 ^ 4) << 4);

    u32x4_t wreg[PASSES], xreg[PASSES];
#define CUBERT_LOAD_GLOBAL(kt)                                                                         \
    do {                                                                                               \
        _Pragma("unroll") for (int i = 0; i < PASSES; ++i) {                                           \
            wreg[i] = __builtin_amdgcn_raw_buffer_load_b128(wres, w_voff + (n0 + i * 32) * w_rowb, (kt) * 128, 0); \
            xreg[i] = __builtin_amdgcn_raw_buffer_load_b128(xres, x_voff + (m0 + i * 32) * x_rowb, (kt) * 128, 0); \
        }                                                                                              \
    } while (0)
#define CUBERT_STORE_LDS(buf)                                                                          \
    do {                                                                                               \
        unsigned char* wt_ = smem + (buf) * 2 * TILE_BYTES;                                            \
        unsigned char* xt_ = wt_ + TILE_BYTES;                                                         \
        _Pragma("unroll") for (int i = 0; i < PASSES; ++i) {                                           \
            const int off = i * 4096 + ((i & 1) ? st_odd : st_even);                                   \
            *reinterpret_cast<u32x4_t*>(wt_ + off) = wreg[i];                                          \
            *reinterpret_cast<u32x4_t*>(xt_ + off) = xreg[i];                                          \
        }                                                                                              \
    } while (0)

    // ---- fragment read addressing ----
    const int s0 = (l32 ^ (l32 >> 3)) & 7;
    const int wrow0 = wn * (BT / 2) + l32;       // + 32*i
    const int xrow0 = wm * (BT / 2) + l32;       // + 32*j

    f32x16_t acc[NB][NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int KT = p.K / BK;
    CUBERT_LOAD_GLOBAL(0);
    CUBERT_STORE_LDS(0);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) CUBERT_LOAD_GLOBAL(kt + 1);
        const unsigned char* wt = smem + cur * 2 * TILE_BYTES;
        const unsigned char* xt = wt + TILE_BYTES;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            u32x4_t wf[NB], xf[NB];
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int row = wrow0 + 32 * i;
                const int sw = s0 ^ ((((wn * (BT / 64)) + i) & 1) << 2);
                wf[i] = *reinterpret_cast<const u32x4_t*>(wt + row * 128 + (((2 * kk + g) ^ sw) << 4));
            }
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int row = xrow0 + 32 * j;
                const int sw = s0 ^ ((((wm * (BT / 64)) + j) & 1) << 2);
                xf[j] = *reinterpret_cast<const u32x4_t*>(xt + row * 128 + (((2 * kk + g) ^ sw) << 4));
            }
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) mfma_chunk<ELT>(wf[i], xf[j], acc[i][j]);
        }
        if (kt + 1 < KT) CUBERT_STORE_LDS(cur ^ 1);
        __syncthreads();
    }

#undef CUBERT_LOAD_GLOBAL
#undef CUBERT_STORE_LDS

    // ---- epilogue: lane owns token (column) l32 and feature rows 8q+4g+e ----
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int m = m0 + wm * (BT / 2) + 32 * j + l32;
        if (m >= p.M) continue;
        int bidx = 0, sidx = 0;
        if constexpr (EPI == kEpiQKV) {
            bidx = m / p.S;
            sidx = m - bidx * p.S;
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int n = n0 + wn * (BT / 2) + 32 * i + 8 * qd + 4 * g;
                if (n >= p.N) continue;
                const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(p.bias + n);
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t = acc[i][j][4 * qd + e] + b4[e];
                    if constexpr (EPI == kEpiBiasGelu) t = gelu_erf(t);
                    if constexpr (EPI == kEpiBiasTanh) t = tanhf(t);
                    v[e] = t;
                }
                if constexpr (EPI == kEpiQKV) {
                    const int which = n / p.hidden;
                    const int hn = n - which * p.hidden;
                    const int head = hn >> 6, dd = hn & 63;
                    const size_t bh = (size_t)bidx * p.heads + head;
                    if (which == 2) {
                        const size_t base = (bh * 64 + dd) * p.Sp + sidx;
#pragma unroll
                        for (int e = 0; e < 4; ++e) store1<OUT>(p.vt, base + (size_t)e * p.Sp, v[e]);
                    } else {
                        store4<OUT>(which == 0 ? p.q : p.k, (bh * p.S + sidx) * 64 + dd, v);
                    }
                } else {
                    store4<OUT>(p.Y, (size_t)m * p.N + n, v);
                }
            }
        }
    }
}

template <int ELT, int OUT, int EPI, int BT>
bool launch_one(const GemmDev& d, hipStream_t stream) {
    const size_t lds = (size_t)4 * BT * 128;     // two buffers x two operand tiles
    auto kern = gemm_kernel<ELT, OUT, EPI, BT>;
    static bool attr_done = false;               // per instantiation
    if (!attr_done) {
        CUBERT_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_done = true;
    }
    hipLaunchKernelGGL(kern, dim3(d.tiles_n * d.tiles_m), dim3(256), lds, stream, d);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

template <int ELT, int OUT, int EPI>
bool launch_tile(const GemmDev& d, int bt, hipStream_t stream) {
    switch (bt) {
        case 64: return launch_one<ELT, OUT, EPI, 64>(d, stream);
        case 128: return launch_one<ELT, OUT, EPI, 128>(d, stream);
        case 256: return launch_one<ELT, OUT, EPI, 256>(d, stream);
    }
    set_error("gemm: tile must be 64, 128 or 256");
    return false;
}

template <int ELT, int OUT>
bool launch_epi(const GemmDev& d, int epi, int bt, hipStream_t stream) {
    switch (epi) {
        case kEpiBias: return launch_tile<ELT, OUT, kEpiBias>(d, bt, stream);
        case kEpiBiasGelu: return launch_tile<ELT, OUT, kEpiBiasGelu>(d, bt, stream);
        case kEpiBiasTanh: return launch_tile<ELT, OUT, kEpiBiasTanh>(d, bt, stream);
        case kEpiQKV: return launch_tile<ELT, OUT, kEpiQKV>(d, bt, stream);
    }
    set_error("gemm: unknown epilogue");
    return false;
}

}  // namespace

int gemm_pick_tile(int M, int N) {
    // Largest tile that still yields a few workgroups per CU-round; the 256
    // tile has the best MFMA:LDS ratio, the small ones fill the chip when the
    // problem is short.
    auto tiles = [&](int bt) { return (long)((M + bt - 1) / bt) * ((N + bt - 1) / bt); };
    if (tiles(256) >= 256) return 256;
    if (tiles(128) >= 256) return 128;
    return 64;
}

bool launch_gemm(const GemmParams& p, hipStream_t stream) {
    const int es = (p.elt == kBF16) ? 2 : 4;
    const int bk = 128 / es;
    if (p.elt != kBF16 && p.elt != kF32) { set_error("gemm: bad operand type"); return false; }
    if (p.M <= 0 || p.N <= 0 || p.K <= 0) { set_error("gemm: empty problem"); return false; }
    if (p.K % bk != 0) { set_error("gemm: K must be a multiple of " + std::to_string(bk)); return false; }
    if (p.N % 4 != 0) { set_error("gemm: N must be a multiple of 4"); return false; }
    if (p.ldx < p.K || (p.ldx * es) % 16 != 0) { set_error("gemm: bad ldx"); return false; }
    if (!p.X || !p.W || !p.bias) { set_error("gemm: null operand"); return false; }
    if (((size_t)p.M + 256) * p.ldx * es >= (1ull << 31) || ((size_t)p.N + 256) * p.K * es >= (1ull << 31)) {
        set_error("gemm: operand exceeds the 2 GiB addressable through one buffer descriptor");
        return false;
    }
    if ((reinterpret_cast<uintptr_t>(p.X) | reinterpret_cast<uintptr_t>(p.W) |
         reinterpret_cast<uintptr_t>(p.bias)) & 15) {
        set_error("gemm: operands must be 16-byte aligned");
        return false;
    }
    GemmDev d{};
    d.X = static_cast<const unsigned char*>(p.X);
    d.W = static_cast<const unsigned char*>(p.W);
    d.bias = p.bias;
    d.Y = static_cast<unsigned char*>(p.Y);
    d.M = p.M; d.N = p.N; d.K = p.K; d.ldx = p.ldx;
    int out = p.out_elt;
    if (p.epilogue == kEpiQKV) {
        if (!p.q || !p.k || !p.vt || p.S <= 0 || p.heads <= 0 || p.N != 3 * p.heads * 64 ||
            p.M % p.S != 0 || p.Sp < p.S || p.Sp % 4 != 0) {
            set_error("gemm: bad QKV epilogue arguments");
            return false;
        }
        d.q = static_cast<unsigned char*>(p.q);
        d.k = static_cast<unsigned char*>(p.k);
        d.vt = static_cast<unsigned char*>(p.vt);
        d.S = p.S; d.Sp = p.Sp; d.heads = p.heads; d.hidden = p.heads * 64;
        out = p.elt;
    } else {
        if (!p.Y || (reinterpret_cast<uintptr_t>(p.Y) & 15)) { set_error("gemm: bad Y"); return false; }
        if (out != kBF16 && out != kF32) { set_error("gemm: bad output type"); return false; }
    }
    const int bt = p.tile ? p.tile : gemm_pick_tile(p.M, p.N);
    d.tiles_n = (p.N + bt - 1) / bt;
    d.tiles_m = (p.M + bt - 1) / bt;
    if (p.elt == kBF16) {
        return out == kBF16 ? launch_epi<kBF16, kBF16>(d, p.epilogue, bt, stream)
                            : launch_epi<kBF16, kF32>(d, p.epilogue, bt, stream);
    }
    if (out != kF32) { set_error("gemm: f32 operands require f32 output"); return false; }
    return launch_epi<kF32, kF32>(d, p.epilogue, bt, stream);
}

}  // namespace cubert
