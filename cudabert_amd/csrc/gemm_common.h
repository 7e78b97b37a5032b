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
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2_t;

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
    int v_rowmajor;                       // QKV epilogue: V is stored like q / k instead of transposed
    const float* R;                       // kEpiBiasRes: [M, N] float32 row-major, added to the result
    int splits;                           // split K: blockIdx.y owns a K range, results go to Y + y * M * N (f32)
    // kEpiBiasResLN: LayerNorm in the epilogue (gemm_epilogue_ln)
    const float* ln_gamma;
    const float* ln_beta;
    unsigned char* ln_xb;                 // bf16 copy of the result (may be null)
    int ln_xb_packed;
    int* ln_cnt;                          // [0] error flag, [1] poll limit (0: default), [kLnCntFirst + band] arrivals, [.. + ln_bands + band] departures
    unsigned long long* ln_stats;         // [row][2 * tiles_n] (sum, M2 about the slot's mean) as two floats in 64 bits
    int ln_bands;
};

constexpr int kLnCntFirst = 64;           // first counter word of the workspace (the words before it: flags)
constexpr int kLnSpinLimit = 1 << 21;     // polls of a band's arrival counter before a workgroup gives up

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
constexpr bool gemm_bias_at_readout() { return OUT == kF32 && (EPI == kEpiBias || EPI == kEpiBiasRes || EPI == kEpiBiasResLN); }

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
// What the read-out phase of a float32 epilogue adds to the first rows it handles: the bias quad of the lane's features
// and (kEpiBiasRes) the first batch of residual rows.  gemm_epilogue fetches them itself; a kernel whose launch is too
// short to hide that round trip behind anything else (a few K steps per workgroup) asks for them before its K loop
// with gemm_epilogue_prefetch and hands them in.
template <int PB>
struct EpiPrefetch {
    f32x4_t bias_ro;
    f32x4_t res0[PB];
};

template <int OUT, int EPI, int NBI, bool SPLITK = false, int RPB = 4>
struct EpiGeometry {
    static constexpr int OES = (OUT == kBF16) ? 2 : 4;
    static constexpr int RB = 32 * NBI * OES;      // bytes per token row of the staging block
    static constexpr int CH = RB / 16;             // 16-byte chunks per row
    static constexpr int RPI = 64 / CH;            // rows one store instruction covers
    static constexpr int EPC = 16 / OES;           // elements per chunk
    static constexpr bool RES = EPI == kEpiBiasRes;
    static constexpr int NIT = 32 / RPI;                               // read-out steps per block column
    static constexpr int PB = RES ? (NIT < RPB ? NIT : RPB) : NIT;     // steps per residual batch
};

template <int OUT, int EPI, int NBI, bool SPLITK = false, int RPB = 4>
__device__ __forceinline__ void gemm_epilogue_prefetch(const GemmDev& p, int n_base, int m_base, int l32, int g,
                                                       EpiPrefetch<EpiGeometry<OUT, EPI, NBI, SPLITK, RPB>::PB>* pre) {
    typedef EpiGeometry<OUT, EPI, NBI, SPLITK, RPB> G;
    static_assert(gemm_bias_at_readout<OUT, EPI>(), "only float32 results take their bias in the read-out phase");
    const int lane = l32 + 32 * g;
    const int rrow = lane / G::CH, rc = lane % G::CH;
    bool first = true;
    if constexpr (SPLITK) first = blockIdx.y == 0;          // split K: bias and residual are added once
    const int n = n_base + rc * G::EPC;
    pre->bias_ro = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    if (first) pre->bias_ro = *reinterpret_cast<const f32x4_t*>(p.bias + (n < p.N ? n : p.N - 4));
    if constexpr (G::RES) {
#pragma unroll
        for (int s = 0; s < G::PB; ++s) {
            const int mm = m_base + s * G::RPI + rrow;
            pre->res0[s] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            if (first) pre->res0[s] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p.R + (size_t)(mm < p.M ? mm : p.M - 1) * p.N + (n < p.N ? n : p.N - 4)));
        }
    }
}

template <int OUT, int EPI, int NBI, int NBJ, bool SPLITK = false, int RPB = 4, bool RDB = false>
__device__ __forceinline__ void gemm_epilogue(const GemmDev& p, f32x16_t (&acc)[NBI][NBJ], const f32x4_t (&bias)[4 * NBI],
                                              int n_base, int m_base, int l32, int g, unsigned char* scratch,
                                              const EpiPrefetch<EpiGeometry<OUT, EPI, NBI, SPLITK, RPB>::PB>* pre = nullptr) {
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
    if constexpr (RES && RDB) {
        if (pre) {
#pragma unroll
            for (int s = 0; s < PB; ++s) res[0][s] = pre->res0[s];
        } else if (addres) {
            fetch_res(0, 0, res[0]);
        }
    }
    constexpr bool BIAS_RO = gemm_bias_at_readout<OUT, EPI>();
    f32x4_t bias_ro = {0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (BIAS_RO) {
        bool addb = true;
        if constexpr (SPLITK) addb = blockIdx.y == 0;           // split K: the bias is added once
        const int n = n_base + rc * EPC;
        if (pre) bias_ro = pre->bias_ro;
        else if (addb) bias_ro = *reinterpret_cast<const f32x4_t*>(p.bias + (n < p.N ? n : p.N - 4));
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
                    if (n >= 2 * p.hidden && !p.v_rowmajor) {
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
                if (n >= 2 * p.hidden && !p.v_rowmajor) continue;           // left transposed, straight from the accumulators
                const int b2 = tok / p.S, s2 = tok - b2 * p.S;
                const int which = n >= 2 * p.hidden ? 2 : n >= p.hidden ? 1 : 0;
                const int hn = n - which * p.hidden;
                const size_t bh = (size_t)b2 * p.heads + (hn >> 6);
                *reinterpret_cast<u32x4_t*>((which == 2 ? p.vt : which ? p.k : p.q) + ((bh * p.S + s2) * 64 + (hn & 63)) * OES) = d;
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

// ---------------------------------------------------------------------------
// LayerNorm in the epilogue (kEpiBiasResLN): Y = LayerNorm(acc + bias + R) * gamma + beta over rows of
// N = 256 * tiles_n features, float32 row-major, plus an optional bf16 copy (the next GEMM's operand).
//
// A workgroup holds 256 of a row's features, so the tiles_n workgroups of one band of rows have to
// agree on the row statistics.  Every wave (128 features of its rows) publishes (sum, M2 about its own mean)
// per row in device memory, the workgroup counts itself in on the band's arrival counter, waits until
// all tiles_n workgroups have, and reads the 2 * tiles_n partial sums of its rows.  The accumulators go
// through the wave's LDS staging once (whole row segments come out, bias and residual are added to
// them); the sums go back into the registers the accumulators came from and wait there, in read-out
// order, until the statistics are known, and are then normalised and stored.
//
// Workgroup order (ln_tile_of_block): XCD x (= workgroup id % 8) owns the bands x, x + 8, ...; the
// workgroups of a band have consecutive positions on that XCD, i.e. ids 8 apart.  Workgroups are
// dispatched in id order per XCD, so whenever 32 workgroups of the launch are resident the partners of
// the oldest unfinished one are resident or done, and it can finish: no deadlock however many CUs
// other launches occupy (two such launches cannot both hold fewer than 32 of the 256 CUs for ever).
// The wait is bounded all the same (kLnSpinLimit polls); a workgroup that gives up raises the error
// word of the workspace and stores what it has.
//
// The counters of a band are put back to zero by the last workgroup to leave it, so the workspace
// needs no clearing between launches (and none inside a captured graph).
__device__ __forceinline__ void ln_tile_of_block(int pid, int tiles_n, int* tn, int* tm) {
    const int xcd = pid & 7, idx = pid >> 3;
    *tm = (idx / tiles_n) * 8 + xcd;
    *tn = idx % tiles_n;
}

// One trip of the accumulators through the wave's LDS staging block: block column j is written in
// accumulator order (row = token, chunk swizzled by the row) and read back as whole row segments, lane
// (rrow, rc) taking features 4 rc .. 4 rc + 3 of row 2 s + rrow in step s; bias and residual are added on
// the way out and `use(j, s, d)` receives the sums.  The residual rows come in batches of PB steps, the
// next batch requested before the current one is consumed.
template <int NBI, int NBJ, int SCHED, typename Use>
__device__ __forceinline__ void ln_stream_rows(f32x16_t (&acc)[NBI][NBJ], unsigned char* buf, int l32, int g, int rrow, int rc,
                                               const f32x4_t& bias4, __amdgpu_buffer_rsrc_t r_rsrc, int lane_off, int row_bytes,
                                               Use use) {
    constexpr int RB = 512, RPI = 2, NIT = 16, PB = 8;
    constexpr int NBATCH = NBJ * NIT / PB;
    f32x4_t res[2][PB];
    auto fetch_res = [&](int batch, f32x4_t (&r)[PB]) {
#pragma unroll
        for (int u = 0; u < PB; ++u)      // row 32 j + 2 s (+ rrow) with j * NIT + s = batch * PB + u
            r[u] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(r_rsrc, lane_off + (batch * PB + u) * RPI * row_bytes, 0, 0));
    };
    fetch_res(0, res[0]);
#pragma unroll
    for (int j = 0; j < NBJ; ++j) {
#pragma unroll
        for (int i = 0; i < NBI; ++i)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int fb = (32 * i + 8 * qd + 4 * g) * 4;
                const f32x4_t v = {acc[i][j][4 * qd], acc[i][j][4 * qd + 1], acc[i][j][4 * qd + 2], acc[i][j][4 * qd + 3]};
                *reinterpret_cast<f32x4_t*>(buf + l32 * RB + ((((fb >> 4) ^ l32) & 31) << 4)) = v;
            }
#pragma unroll
        for (int s = 0; s < NIT; ++s) {
            const int batch = (j * NIT + s) / PB;             // compile-time after unrolling
            if (s % PB == 0 && batch + 1 < NBATCH) fetch_res(batch + 1, res[(batch + 1) & 1]);
            const int row = s * RPI + rrow;
            const f32x4_t staged = *reinterpret_cast<const f32x4_t*>(buf + row * RB + (((rc ^ row) & 31) << 4));
            use(j, s, (staged + bias4) + res[batch & 1][s % PB]);
            if (s % SCHED == SCHED - 1) __builtin_amdgcn_sched_barrier(0);     // bounds how many steps the scheduler interleaves
        }
    }
}

template <int NBI, int NBJ>
__device__ __forceinline__ void gemm_epilogue_ln(const GemmDev& p, f32x16_t (&acc)[NBI][NBJ], int n_base, int m_base,
                                                 int l32, int g, int band, int slot, unsigned char* buf,
                                                 float* statbuf) {
    static_assert(NBI == 4 && NBJ % 2 == 0, "a wave holds 128 features and a multiple of 64 rows");
    constexpr int RPI = 2;                   // rows one read-out step covers
    constexpr int NIT = 16;                  // read-out steps per block column of 32 rows
    constexpr int NP = NBJ * NIT / 32;       // (block column, step) pairs whose row a lane publishes
    const int slots = 2 * p.tiles_n;
    const float invn = 1.0f / (float)p.N;
    // Residual and result through buffer descriptors: a row's address is one lane offset plus a
    // wave-uniform row term, rows past M read as zero and are not stored.  (The whole offset goes
    // into the lane operand: the descriptor's range check does not look at the scalar offset.)
    const int row_bytes = p.N * 4;
    const __amdgpu_buffer_rsrc_t r_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.R), 0, p.M * row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.Y, 0, p.M * row_bytes, 0x00020000);

    // ---- first pass: row sums of (acc + bias + R) over this wave's 128 features ----
    float ksum[NP], ksq[NP];
#pragma unroll
    for (int t = 0; t < NP; ++t) ksum[t] = ksq[t] = 0.0f;
    {
        const int lane = l32 + 32 * g, rrow = lane >> 5, rc = lane & 31;
        const int n = n_base + rc * 4;           // this lane's four features on the way out (N % 256 == 0: in range)
        const f32x4_t bias4 = *reinterpret_cast<const f32x4_t*>(p.bias + n);
        ln_stream_rows<NBI, NBJ, 4>(acc, buf, l32, g, rrow, rc, bias4, r_rsrc, (m_base + rrow) * row_bytes + n * 4, row_bytes,
                                 [&](int j, int s, const f32x4_t& d) {
            float t, q;                                       // the slot's sum and M2 about the slot's mean
            ln_slot_stats(d[0], d[1], d[2], d[3], true, 0.0078125f, &t, &q);
            const int pair = j * NIT + s;                     // compile-time after unrolling
            if (rc == (pair & 31)) { ksum[pair >> 5] = t; ksq[pair >> 5] = q; }
            // The sums stay in the registers of the accumulators they were made from (block column j
            // has been staged completely by now): step s of column j in acc[s / 4][j][4 (s % 4) ..].
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[s / 4][j][4 * (s % 4) + e] = d[e];
            // the selection happens here (left to itself the compiler postpones all of them past the
            // loop and spills every step's sums until then)
            asm volatile("" : "+v"(ksum[pair >> 5]), "+v"(ksq[pair >> 5]));
        });
        // lane (rrow, rc) publishes the rows of the pairs t * 32 + rc
#pragma unroll
        for (int t = 0; t < NP; ++t) {
            const int pair = t * 32 + rc;
            const int mm = m_base + 32 * (pair / NIT) + RPI * (pair % NIT) + rrow;
            if (mm < p.M) {
                const unsigned long long bits = (unsigned long long)__builtin_bit_cast(unsigned, ksum[t]) |
                                                ((unsigned long long)__builtin_bit_cast(unsigned, ksq[t]) << 32);
                __hip_atomic_store(p.ln_stats + (size_t)mm * slots + slot, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // the sums are in place before the workgroup counts itself in
    __syncthreads();
    int* arrivals = p.ln_cnt + kLnCntFirst + band;
    int* departures = arrivals + p.ln_bands;
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(arrivals, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int wish = p.ln_cnt[1];                         // word 1 of the workspace: the host's own poll limit, if positive
        const int limit = wish > 0 ? wish : kLnSpinLimit;
        int polls = 0;
        while (__hip_atomic_load(arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < p.tiles_n) {
            if (++polls > limit) {
                __hip_atomic_store(p.ln_cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
    }
    __syncthreads();

    // What the registers of the accumulators hold now (the sums, in read-out order) has to survive
    // the wait in place: the empty statements keep the compiler from moving the values elsewhere.
#pragma unroll
    for (int i = 0; i < NBI; ++i)
#pragma unroll
        for (int j = 0; j < NBJ; ++j) asm volatile("" : "+a"(acc[i][j]));
    // (Likewise the lane coordinates: from laundered copies, so that the addresses of the second pass
    // are formed after the wait instead of being carried, and spilled, through the first.)
    int l32b = l32, gb = g;
    asm volatile("" : "+v"(l32b), "+v"(gb));
    const int lane = l32b + 32 * gb, rrow = lane >> 5, rc = lane & 31;
    const int n = n_base + rc * 4;

    // ---- statistics of my rows: all partial sums, in slot order ----
    // The partners' sums are read with cache-bypassing buffer loads (sc0 | sc1), all requested before the
    // first one is used.  A row's slots are contiguous: a load past 2 * tiles_n reads the next row's or,
    // at the end, nothing (zero); those values are not added.
    {
        const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.ln_stats, 0, p.M * slots * 8, 0x00020000);
        f32x4_t raw[NP][4];
#pragma unroll
        for (int t = 0; t < NP; ++t) {
            const int pair = t * 32 + rc;
            const int mm = m_base + 32 * (pair / NIT) + RPI * (pair % NIT) + rrow;
#pragma unroll
            for (int c = 0; c < 4; ++c)          // two slots per load; rows past M fall outside the descriptor as well
                raw[t][c] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, (mm * slots + 2 * c) * 8, 0, 17));
        }
#pragma unroll
        for (int t = 0; t < NP; ++t) {
            const int pair = t * 32 + rc;
            const int rl = 32 * (pair / NIT) + RPI * (pair % NIT) + rrow;     // row within the wave's rows
            float sum = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (2 * c < slots) {          // a wave-uniform branch; slots is even
                    sum += raw[t][c][0];
                    sum += raw[t][c][2];
                }
            }
            const float mean = ln_row_mean(sum, invn);
            float m2 = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (2 * c < slots) {
                    m2 = ln_merge_slot(m2, raw[t][c][0], raw[t][c][1], 128.0f, 0.0078125f, mean);
                    m2 = ln_merge_slot(m2, raw[t][c][2], raw[t][c][3], 128.0f, 0.0078125f, mean);
                }
            }
            statbuf[2 * rl] = mean;
            statbuf[2 * rl + 1] = ln_finalize(m2, invn);
        }
    }
    __syncthreads();                                       // every wave holds its statistics: the band can be left
    if (threadIdx.x == 0) {
        if (__hip_atomic_fetch_add(departures, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.tiles_n - 1) {
            __hip_atomic_store(arrivals, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(departures, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    // ---- second pass: normalise the kept sums and store ----
    const f32x4_t gamma4 = *reinterpret_cast<const f32x4_t*>(p.ln_gamma + n);
    const f32x4_t beta4 = *reinterpret_cast<const f32x4_t*>(p.ln_beta + n);
    // bf16 copy: row-major, or packed (common.h): block of 256 rows x 64 bytes, chunk c of row r in slot
    // c ^ ((r >> 2) & 3).  The wave's rows start at a multiple of 64, so with r = m_base + 32 j + 2 s + rrow
    // the row's block and its swizzle (s >> 1) & 3 are known per step; only the chunk is the lane's.
    const bool xb_on = p.ln_xb != nullptr;
    const int xb_size = p.ln_xb_packed ? (int)packed_bytes(p.M, (size_t)p.N * 2) : p.M * p.N * 2;
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(xb_on ? p.ln_xb : p.Y, 0, xb_on ? xb_size : 0, 0x00020000);
    const int kb_per_row = p.N * 2 / 64;
    const int xb_chunk = (n * 2 >> 4) & 3;
    const int xb_lane = p.ln_xb_packed
        ? (((m_base >> 8) * kb_per_row + (n * 2 >> 6)) * 16384 + ((m_base & 255) + rrow) * 64 + ((n * 2) & 15))
        : ((m_base + rrow) * p.N + n) * 2;
    const int lane_off = (m_base + rrow) * row_bytes + n * 4;
#pragma unroll
    for (int j = 0; j < NBJ; ++j) {
#pragma unroll
        for (int s = 0; s < NIT; ++s) {
            const int step_rows = 32 * j + s * RPI;
            const int rl = step_rows + rrow;
            const float mean = statbuf[2 * rl], rstd = statbuf[2 * rl + 1];
            f32x4_t o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = ln_apply(acc[s / 4][j][4 * (s % 4) + e], mean, rstd, gamma4[e], beta4[e]);
            // rows past M: the descriptor drops the float32 store; the copy is predicated
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, o), y_rsrc, lane_off + step_rows * row_bytes, 0, 0);
            if (xb_on && m_base + rl < p.M) {
                const bf16x4_t ob = {(__bf16)o[0], (__bf16)o[1], (__bf16)o[2], (__bf16)o[3]};
                const int off = p.ln_xb_packed ? xb_lane + step_rows * 64 + ((xb_chunk ^ ((s >> 1) & 3)) << 4)
                                               : xb_lane + step_rows * p.N * 2;
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2_t, ob), x_rsrc, off, 0, 0);
            }
        }
    }
}

}  // namespace gemm_detail
}  // namespace cubert
