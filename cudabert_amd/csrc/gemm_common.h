// Pieces shared by the GEMM kernels: the launch descriptor, small device
// helpers, the workgroup -> tile mapping and the epilogue.
#pragma once
#include "kernels.h"

namespace cubert {
namespace gemm_detail {

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
    int x_packed, w_packed, y_packed;     // operand / result in the packed layout (common.h)
    int xn_parts;                         // how the XCDs divide the tile grid (tile_of_block)
    const int* rowmap;                    // QKV epilogue: row m -> token b * S + s (nullptr: m itself)
    const float* R;                       // kEpiBiasRes: [M, N] float32 row-major, added to the result
    int splits;                           // split K: blockIdx.y owns a K range, results go to Y + y * M * N (f32)
};

__device__ __forceinline__ float gelu_erf(float x) {
    return x * 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
}

// GELU for results that are stored as bf16, without transcendentals:
//   gelu(x) = max(x, 0) - T(|x|),   T(a) = a (1 - Phi(a)),
// T(a) = s R(s) with s = min(a / 4.25, 1) and R a degree-9 polynomial fitted
// (weighted minimax, weights a) to 4.25 (1 - Phi(4.25 s)) on [0, 1].  Beyond
// 4.25 the result keeps the constant T(4.25) = 4.5e-5 instead of decaying to 0.
// In float32 arithmetic the absolute error is below 7e-5 everywhere and the
// relative error below 1.1e-4 wherever |gelu(x)| > 0.05: more than an order of
// magnitude under the bf16 rounding applied to the result (2^-9 relative).
// gelu(0) = 0 exactly.
__device__ __forceinline__ float gelu_fast(float x) {
    const float s = fminf(fabsf(x) * 0.23529411764705882f, 1.0f);
    float r = -3.026185036e+01f;
    r = fmaf(r, s, 1.650908966e+02f);
    r = fmaf(r, s, -3.731475220e+02f);
    r = fmaf(r, s, 4.392153320e+02f);
    r = fmaf(r, s, -2.677408752e+02f);
    r = fmaf(r, s, 5.936063385e+01f);
    r = fmaf(r, s, 1.166716862e+01f);
    r = fmaf(r, s, 9.375342727e-01f);
    r = fmaf(r, s, -7.246768475e+00f);
    r = fmaf(r, s, 2.125523567e+00f);
    return fmaf(-s, r, fmaxf(x, 0.0f));
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

// Workgroup id -> (tile_n, tile_m).  Hardware hands consecutive workgroup ids to
// the eight XCDs round-robin, and every XCD has its own 4 MiB L2.  xn_parts = 4 or
// 2 (chosen by gemm_pick_partition on the host, only when the grid divides): the
// XCDs own the cells of a 2 x 4 or 4 x 2 partition of the tile grid (rows x
// columns), so a quarter or half of the weight rows stays resident in an XCD's L2
// and every activation row is fetched by 4 or 2 XCDs.  xn_parts = 0: each XCD gets
// one contiguous run of the tile sequence, i.e. a band of token rows with all the
// weight columns: activations are fetched once, the weights stream through every
// XCD.  Inside its share an XCD walks groups of kGroupM tile rows column by
// column, so that the tiles in flight at one time span few operand slabs and the
// next ones reuse the same activation rows.  (kGroupM: 4 for the 256 x 256 tile
// with 32 workgroups per XCD in flight, 8 for the 256 x 128 tile with 64.)
template <int kGroupM = 4>
__device__ __forceinline__ void tile_of_block(int pid, int total, int tiles_n, int xn_parts, int* tn, int* tm) {
    const int xcd = pid & 7, idx = pid >> 3;
    const int tiles_m = total / tiles_n;
    if (xn_parts && ((total & 7) != 0 || tiles_n % xn_parts != 0 || tiles_m % (8 / xn_parts) != 0)) xn_parts = 0;
    int n_first = 0, m_first = 0, n_count = tiles_n, m_count = tiles_m, t = idx;
    if (xn_parts) {
        n_count = tiles_n / xn_parts;
        m_count = tiles_m / (8 / xn_parts);
        n_first = (xcd % xn_parts) * n_count;
        m_first = (xcd / xn_parts) * m_count;
    } else {
        const int base = total >> 3, rem = total & 7;
        t = xcd * base + (xcd < rem ? xcd : rem) + idx;
    }
    const int per_group = kGroupM * n_count;
    const int group = t / per_group, r = t - group * per_group;
    const int left = m_count - group * kGroupM;
    const int gm = left < kGroupM ? left : kGroupM;       // the last group may be shorter
    const int c = r / gm;
    *tn = n_first + c;
    *tm = m_first + group * kGroupM + (r - c * gm);
}

// Host side of tile_of_block: the partition with the smaller estimated traffic between memory and
// the L2s.  A 2-D partition fetches the activations xn_parts times and each XCD's share of the
// weights once if it fits beside the streaming activations (else once per group of tile rows); a
// contiguous run fetches the activations once and streams all the weights through every XCD once
// per group.  x_bytes / w_bytes: size of the operands; group_m: the kernel's kGroupM.
inline int gemm_pick_partition(double x_bytes, double w_bytes, int tiles_n, int tiles_m, int group_m) {
    const double l2_fit = 2.5 * 1024 * 1024;
    auto groups = [&](int rows) { return (double)((rows + group_m - 1) / group_m); };
    const int rows_per_xcd = (tiles_m + 7) / 8;
    double best = x_bytes + 8.0 * w_bytes * (w_bytes <= l2_fit ? 1.0 : groups(rows_per_xcd));
    int pick = 0;
    if ((((long)tiles_n * tiles_m) & 7) == 0) {
        for (int xn = 2; xn <= 4; xn += 2) {
            if (tiles_n % xn != 0 || tiles_m % (8 / xn) != 0) continue;
            const double share = w_bytes / xn;
            const double f = x_bytes * xn + share * 8.0 * (share <= l2_fit ? 1.0 : groups(tiles_m / (8 / xn)));
            if (f < best) { best = f; pick = xn; }
        }
    }
    return pick;
}

// float32 results without an activation take their bias in the read-out phase of the epilogue, where
// a lane serves one group of four features for all rows (one quad instead of 4 NB): gemm_load_bias is
// not needed for them and the epilogue ignores its `bias` argument.
template <int OUT, int EPI>
constexpr bool gemm_bias_at_readout() { return OUT == kF32 && (EPI == kEpiBias || EPI == kEpiBiasRes); }

// The bias values a lane needs (4 NB quads) are fetched by gemm_load_bias before the
// K loop so that their latency is hidden; features past N read the last valid quad
// (their results are never stored).
template <int NBI, bool SPLITK = false>
__device__ __forceinline__ void gemm_load_bias(const GemmDev& p, int n_base, int g, f32x4_t (&bias)[4 * NBI]) {
#pragma unroll
    for (int t = 0; t < 4 * NBI; ++t) {
        const int n = n_base + 8 * t + 4 * g;
        bias[t] = *reinterpret_cast<const f32x4_t*>(p.bias + (n < p.N ? n : p.N - 4));
        if constexpr (SPLITK)
            if (blockIdx.y != 0) bias[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};     // split K: the bias is added once
    }
}

// SPLITK: the launch may have several workgroups per tile (blockIdx.y = K share), each writing
// its partial result to its own copy of Y.
// The wave's quadrant is NBI x NBJ accumulator blocks (features x tokens).
//
// kEpiBiasRes (float32 row-major result): the read-out adds R[m][n] to every element, fetched in the
// layout of the stores (whole row segments).  The fetches go out RPB read-out steps at a time; with RDB
// the next batch is requested before the current one is consumed (two batches of registers), which a
// kernel with one workgroup per CU needs because nothing else covers the latency there.
template <int OUT, int EPI, int NBI, int NBJ, bool SPLITK = false, int RPB = 4, bool RDB = false>
__device__ __forceinline__ void gemm_epilogue(const GemmDev& p, f32x16_t (&acc)[NBI][NBJ], const f32x4_t (&bias)[4 * NBI],
                                              int n_base, int m_base, int l32, int g, unsigned char* scratch) {
    constexpr int OES = (OUT == kBF16) ? 2 : 4;
    constexpr int RB = 32 * NBI * OES;      // bytes per token row of the staging block
    constexpr int CH = RB / 16;             // 16-byte chunks per row
    constexpr int RPI = 64 / CH;            // rows one store instruction covers
    constexpr int EPC = 16 / OES;           // elements per chunk
    constexpr bool RES = EPI == kEpiBiasRes;
    static_assert(!RES || OUT == kF32, "the residual epilogue writes float32");
    constexpr int NIT = 32 / RPI;                               // read-out steps per block column
    constexpr int PB = RES ? (NIT < RPB ? NIT : RPB) : NIT;     // steps per residual batch
    constexpr int NBATCH = NIT / PB;
    const int lane = l32 + 32 * g;
    const int rrow = lane / CH, rc = lane % CH;
    f32x4_t res[RES && RDB ? 2 : 1][PB];
    bool addres = RES;
    if constexpr (SPLITK) addres = RES && blockIdx.y == 0;      // split K: the residual is added once
    // rows / features outside the matrix fetch a valid neighbour; their sums are never stored
    auto fetch_res = [&](int j, int bt, f32x4_t (&r)[PB]) {
#pragma unroll
        for (int s = 0; s < PB; ++s) {
            const int mm = m_base + 32 * j + (bt * PB + s) * RPI + rrow;
            const int n = n_base + rc * EPC;
            r[s] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p.R + (size_t)(mm < p.M ? mm : p.M - 1) * p.N + (n < p.N ? n : p.N - 4)));
        }
    };
    if constexpr (RES && RDB)
        if (addres) fetch_res(0, 0, res[0]);
    constexpr bool BIAS_RO = gemm_bias_at_readout<OUT, EPI>();
    f32x4_t bias_ro = {0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (BIAS_RO) {
        bool addb = true;
        if constexpr (SPLITK) addb = blockIdx.y == 0;           // split K: the bias is added once
        const int n = n_base + rc * EPC;
        if (addb) bias_ro = *reinterpret_cast<const f32x4_t*>(p.bias + (n < p.N ? n : p.N - 4));
    }
    // compact rows: the token of this lane's row in every block row, fetched together up front;
    // the read-out phase takes a row's token from the lane that owns it
    int tokj[NBJ];
    if constexpr (EPI == kEpiQKVMap) {
#pragma unroll
        for (int j = 0; j < NBJ; ++j) {
            const int m = m_base + 32 * j + l32;
            tokj[j] = p.rowmap[m < p.M ? m : p.M - 1];
        }
    }
#pragma unroll
    for (int j = 0; j < NBJ; ++j) {
        unsigned char* buf = scratch + ((OES == 2 && (j & 1)) ? 32 * RB : 0);
        const int m = m_base + 32 * j + l32;
        int bidx = 0, sidx = 0;
        if constexpr (EPI == kEpiQKV || EPI == kEpiQKVMap) {
            int tok = m;
            if constexpr (EPI == kEpiQKVMap) tok = tokj[j];
            bidx = tok / p.S;
            sidx = tok - bidx * p.S;
        }
#pragma unroll
        for (int i = 0; i < NBI; ++i) {
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int fq = 32 * i + 8 * qd + 4 * g;          // feature within the quadrant
                const int n = n_base + fq;
                f32x4_t b4 = {0.0f, 0.0f, 0.0f, 0.0f};
                if constexpr (!BIAS_RO) b4 = bias[4 * i + qd];
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t = acc[i][j][4 * qd + e];
                    if constexpr (!BIAS_RO) t += b4[e];
                    if constexpr (EPI == kEpiBiasGelu) t = (OUT == kBF16) ? gelu_fast(t) : gelu_erf(t);
                    if constexpr (EPI == kEpiBiasTanh) t = tanhf(t);
                    v[e] = t;
                }
                if constexpr (EPI == kEpiQKV || EPI == kEpiQKVMap) {
                    if (n >= 2 * p.hidden) {
                        if (m < p.M && n < p.N) {
                            const int hn = n - 2 * p.hidden;
                            const size_t bh = (size_t)bidx * p.heads + (hn >> 6);
                            const size_t base = (bh * 64 + (hn & 63)) * p.Sp + sidx;
#pragma unroll
                            for (int e = 0; e < 4; ++e) store1<OUT>(p.vt, base + (size_t)e * p.Sp, v[e]);
                        }
                        continue;
                    }
                }
                const int fb = fq * OES;
                store4<OUT>(buf + l32 * RB + ((((fb >> 4) ^ l32) & (CH - 1)) << 4) + (fb & 15), 0, v);
            }
        }
        // Results leave with ordinary stores: the next kernel reads them at once (as an operand, or the
        // LayerNorm its addend) and the whole pass measured faster with them cached, although a launch
        // on its own fetches 20 % less through L2 when they are non-temporal.
#pragma unroll
        for (int s = 0; s < NIT; ++s) {
            const int row = s * RPI + rrow;
            u32x4_t d = *reinterpret_cast<const u32x4_t*>(buf + row * RB + (((rc ^ row) & (CH - 1)) << 4));
            if constexpr (RES) {
                const int batch = j * NBATCH + s / PB;          // compile-time after unrolling
                if (s % PB == 0 && addres) {
                    if constexpr (RDB) {
                        if (batch + 1 < NBJ * NBATCH) fetch_res((batch + 1) / NBATCH, (batch + 1) % NBATCH, res[(batch + 1) & 1]);
                    } else {
                        fetch_res(j, s / PB, res[0]);
                    }
                }
                if (addres) d = __builtin_bit_cast(u32x4_t, (__builtin_bit_cast(f32x4_t, d) + bias_ro) + res[RDB ? (batch & 1) : 0][s % PB]);
                else d = __builtin_bit_cast(u32x4_t, __builtin_bit_cast(f32x4_t, d) + bias_ro);
            } else if constexpr (BIAS_RO) {
                d = __builtin_bit_cast(u32x4_t, __builtin_bit_cast(f32x4_t, d) + bias_ro);
            }
            const int mm = m_base + 32 * j + row;
            const int n = n_base + rc * EPC;
            int tok = mm;
            if constexpr (EPI == kEpiQKVMap) tok = __shfl(tokj[j], row);      // before any lane leaves
            if (mm >= p.M || n >= p.N) continue;
            if constexpr (EPI == kEpiQKV || EPI == kEpiQKVMap) {
                if (n >= 2 * p.hidden) continue;
                const int b2 = tok / p.S, s2 = tok - b2 * p.S;
                const int which = n >= p.hidden ? 1 : 0;
                const int hn = n - which * p.hidden;
                const size_t bh = (size_t)b2 * p.heads + (hn >> 6);
                *reinterpret_cast<u32x4_t*>((which ? p.k : p.q) + ((bh * p.S + s2) * 64 + (hn & 63)) * OES) = d;
            } else if (p.y_packed) {
                // packed bf16 result: the next GEMM's activation operand
                *reinterpret_cast<u32x4_t*>(p.Y + packed_offset(mm, n * 2, p.N * 2 / 64)) = d;
            } else {
                const size_t part = SPLITK ? (size_t)blockIdx.y * p.M : 0;
                *reinterpret_cast<u32x4_t*>(p.Y + ((part + mm) * p.N + n) * OES) = d;
            }
        }
    }
}

}  // namespace gemm_detail
}  // namespace cubert
