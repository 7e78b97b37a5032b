// Bandwidth-bound row kernels for gfx950: residual-add + LayerNorm, embedding
// gather + add + LayerNorm, scale + mask + softmax, classifier head and the
// load-time weight transpose.  One wave64 owns one row; reductions are
// butterfly shuffles over the 64 lanes, no LDS.
#include "kernels.h"
#include <type_traits>

namespace cubert {
namespace {

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int kMaxChunks = 4;        // 4 chunks x 64 lanes x 4 elements = rows up to 1024

__device__ __forceinline__ float wave_sum(float v) {
    v = half_swap_sum(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = half_swap_max(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// Features of a row of H that fall into 128-feature slot s, and the reciprocal (0 for an empty slot).
__device__ __forceinline__ void ln_slot_count(int H, int s, float* cnt, float* inv) {
    const int left = H - 128 * s;
    const int c = left < 0 ? 0 : (left > 128 ? 128 : left);
    *cnt = (float)c;
    *inv = c > 0 ? 1.0f / (float)c : 0.0f;
}

// Row mean and 1 / sigma from the (sum, M2) of the row's slots, in the engine's canonical order (common.h):
// slots past the row's end hold no features and add nothing.
__device__ __forceinline__ void ln_combine_slots(const float (&ssum)[2 * kMaxChunks], const float (&sm2)[2 * kMaxChunks], int H,
                                                 float* mean_out, float* rstd_out) {
    const float inv_n = 1.0f / (float)H;
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < 2 * kMaxChunks; ++s) sum += ssum[s];
    const float mean = ln_row_mean(sum, inv_n);
    float m2 = 0.0f;
#pragma unroll
    for (int s = 0; s < 2 * kMaxChunks; ++s) {
        float cnt, inv;
        ln_slot_count(H, s, &cnt, &inv);
        if (128 * s < H) m2 = ln_merge_slot(m2, ssum[s], sm2[s], cnt, inv, mean);
    }
    *mean_out = mean;
    *rstd_out = ln_finalize(m2, inv_n);
}

// (sum, M2) of the two slots of chunk c (features c * 256 + lane * 4 ..): every lane gets both, lower slot first.
__device__ __forceinline__ void ln_chunk_stats(const float (&v)[4], int c, int H, int lane, float* sum_lo, float* m2_lo,
                                               float* sum_hi, float* m2_hi) {
    const bool upper = lane >= 32;
    float cnt, inv_lo, inv_hi;
    ln_slot_count(H, 2 * c, &cnt, &inv_lo);
    ln_slot_count(H, 2 * c + 1, &cnt, &inv_hi);
    const bool in = c * 256 + lane * 4 < H;
    float t, q;
    ln_slot_stats(in ? v[0] : 0.0f, in ? v[1] : 0.0f, in ? v[2] : 0.0f, in ? v[3] : 0.0f, in, upper ? inv_hi : inv_lo, &t, &q);
    const float t_other = __shfl_xor(t, 32), q_other = __shfl_xor(q, 32);
    *sum_lo = upper ? t_other : t;
    *m2_lo = upper ? q_other : q;
    *sum_hi = upper ? t : t_other;
    *m2_hi = upper ? q : q_other;
}

// Normalises features i .. i + 3 of a row (mean, rstd known) and writes them to x (f32) and optionally to the bf16
// copy xb: row-major when xb_packed == 0, else in the packed GEMM-operand layout (common.h).
__device__ __forceinline__ void ln_store4(const float (&v)[4], float mean, float rstd, const f32x4_t& g4, const f32x4_t& b4,
                                          float* xrow, bf16_t* xb, int row, int i, int H, int xb_packed) {
    f32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = ln_apply(v[e], mean, rstd, g4[e], b4[e]);
    __builtin_nontemporal_store(o, reinterpret_cast<f32x4_t*>(xrow + i));
    if (xb) {
        bf16x4_t ob = {(__bf16)o[0], (__bf16)o[1], (__bf16)o[2], (__bf16)o[3]};
        unsigned char* dst = reinterpret_cast<unsigned char*>(xb);
        const size_t off = xb_packed ? packed_offset(row, i * 2, H * 2 / 64) : ((size_t)row * H + i) * 2;
        *reinterpret_cast<bf16x4_t*>(dst + off) = ob;
    }
}

// Normalises the row held in v[][] (lane owns elements c*256 + lane*4 + e) and
// writes it to x (f32) and optionally xb (bf16).
__device__ __forceinline__ void normalise_store(float (&v)[kMaxChunks][4], int H, int lane,
                                                const float* __restrict__ gamma,
                                                const float* __restrict__ beta, float* xrow,
                                                bf16_t* xb, int row, int xb_packed) {
    float ssum[2 * kMaxChunks], sm2[2 * kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        ln_chunk_stats(v[c], c, H, lane, &ssum[2 * c], &sm2[2 * c], &ssum[2 * c + 1], &sm2[2 * c + 1]);
    float mean, rstd;
    ln_combine_slots(ssum, sm2, H, &mean, &rstd);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c) {
        const int i = c * 256 + lane * 4;
        if (i < H) {
            const f32x4_t g4 = *reinterpret_cast<const f32x4_t*>(gamma + i);
            const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(beta + i);
            ln_store4(v[c], mean, rstd, g4, b4, xrow, xb, row, i, H, xb_packed);
        }
    }
}

template <int YELT>   // -1: no addend
__global__ __launch_bounds__(256) void add_layernorm_kernel(float* __restrict__ x,
                                                            const unsigned char* __restrict__ y,
                                                            const float* __restrict__ gamma,
                                                            const float* __restrict__ beta,
                                                            bf16_t* __restrict__ xb, int rows, int H,
                                                            int xb_packed, int y_parts, int add_x) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    float* xrow = x + (size_t)row * H;
    float v[kMaxChunks][4];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c) {
        const int i = c * 256 + lane * 4;
        if (i < H) {
            // add_x == 0: y already holds the sum with the residual stream (the producing GEMM added it),
            // x is only written
            f32x4_t a = {0.0f, 0.0f, 0.0f, 0.0f};
            if (YELT == -1 || add_x) a = *reinterpret_cast<const f32x4_t*>(xrow + i);
            if constexpr (YELT == kF32) {
                f32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(y + ((size_t)row * H + i) * 4));
                for (int part = 1; part < y_parts; ++part)     // partial sums of a split-K GEMM, [part][rows][H]
                    t += *reinterpret_cast<const f32x4_t*>(y + (((size_t)part * rows + row) * H + i) * 4);
                a += t;
            } else if constexpr (YELT == kBF16) {
                const bf16x4_t t = *reinterpret_cast<const bf16x4_t*>(y + ((size_t)row * H + i) * 2);
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] += (float)t[e];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) v[c][e] = a[e];
        }
    }
    normalise_store(v, H, lane, gamma, beta, xrow, xb, row, xb_packed);
}

// The same operation for a short batch whose addend comes as the partial sums of a split-K GEMM
// ([part][rows][H] float32): one workgroup per row, so that the few rows still spread over the
// chip.  Such a launch is a chain of round trips and little else, so everything it needs -- the row,
// every partial sum, gamma and beta -- is requested before the first value is used.  Wave w adds up the
// parts of features 256 w .. 256 w + 255 and forms the statistics of its two slots; the waves exchange
// those through the LDS, every wave combines them (the same arithmetic in the same order as
// add_layernorm_kernel, hence the same bits) and normalises its own features.
__global__ __launch_bounds__(256) void add_layernorm_parts_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                                  const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta,
                                                                  bf16_t* __restrict__ xb, int rows, int H,
                                                                  int xb_packed, int y_parts, int add_x) {
    __shared__ float stats[kMaxChunks][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x;
    float* xrow = x + (size_t)row * H;
    const int i = wave * 256 + lane * 4;
    const bool in = i < H;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    f32x4_t g4 = {0.0f, 0.0f, 0.0f, 0.0f}, b4 = {0.0f, 0.0f, 0.0f, 0.0f};
    if (in) {
        f32x4_t a = {0.0f, 0.0f, 0.0f, 0.0f};
        if (add_x) a = *reinterpret_cast<const f32x4_t*>(xrow + i);
        f32x4_t t = *reinterpret_cast<const f32x4_t*>(y + (size_t)row * H + i);
        g4 = *reinterpret_cast<const f32x4_t*>(gamma + i);
        b4 = *reinterpret_cast<const f32x4_t*>(beta + i);
        for (int p0 = 1; p0 < y_parts; p0 += 8) {
            f32x4_t u[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int part = p0 + j < y_parts ? p0 + j : 0;        // a repeat of part 0 is not added
                u[j] = *reinterpret_cast<const f32x4_t*>(y + ((size_t)part * rows + row) * H + i);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (p0 + j < y_parts) t += u[j];
        }
        a += t;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = a[e];
    }
    float s_lo, q_lo, s_hi, q_hi;
    ln_chunk_stats(v, wave, H, lane, &s_lo, &q_lo, &s_hi, &q_hi);
    if (lane == 0) {
        stats[wave][0] = s_lo; stats[wave][1] = q_lo; stats[wave][2] = s_hi; stats[wave][3] = q_hi;
    }
    __syncthreads();
    float ssum[2 * kMaxChunks], sm2[2 * kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c) {
        ssum[2 * c] = stats[c][0]; sm2[2 * c] = stats[c][1]; ssum[2 * c + 1] = stats[c][2]; sm2[2 * c + 1] = stats[c][3];
    }
    float mean, rstd;
    ln_combine_slots(ssum, sm2, H, &mean, &rstd);
    if (in) ln_store4(v, mean, rstd, g4, b4, xrow, xb, row, i, H, xb_packed);
}

__global__ __launch_bounds__(256) void embed_layernorm_kernel(
    const int* __restrict__ ids, const int* __restrict__ seg, const int* __restrict__ mask,
    const float* __restrict__ word, const float* __restrict__ pos, const float* __restrict__ type,
    const float* __restrict__ gamma, const float* __restrict__ beta, float* __restrict__ x,
    bf16_t* __restrict__ xb, float* __restrict__ maskadd, int B, int S, int Sp, int H, int vocab,
    int type_vocab, int xb_packed, const int* __restrict__ rowmap, const int* __restrict__ cu, int nrows) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);        // output row
    if (row >= nrows) return;
    const int tok = rowmap ? rowmap[row] : row;                 // b * S + s
    const int b = tok / S, s = tok - b * S;
    int id = ids[tok];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    int tt = seg ? seg[tok] : 0;
    tt = tt < 0 ? 0 : (tt >= type_vocab ? type_vocab - 1 : tt);
    // additive attention mask: 0 valid, -10000 masked, -inf on the padding S..Sp-1
    if (!rowmap) {
        if (lane == 0) {
            const int mk = mask ? mask[tok] : 1;
            maskadd[(size_t)b * Sp + s] = (1.0f - (float)mk) * -10000.0f;
        }
        if (s == 0 && S + lane < Sp) maskadd[(size_t)b * Sp + S + lane] = -INFINITY;   // Sp - S < 32
    } else if (s == 0) {
        // compact rows: the first token of a sequence writes the whole mask row from the length
        const int len = cu[b + 1] - cu[b];
        for (int i = lane; i < Sp; i += 64)
            maskadd[(size_t)b * Sp + i] = i < len ? 0.0f : (i < S ? -10000.0f : -INFINITY);
    }
    const float* wr = word + (size_t)id * H;
    const float* pr = pos + (size_t)s * H;
    const float* tr = type + (size_t)tt * H;
    float v[kMaxChunks][4];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c) {
        const int i = c * 256 + lane * 4;
        if (i < H) {
            const f32x4_t a = *reinterpret_cast<const f32x4_t*>(wr + i);
            const f32x4_t p4 = *reinterpret_cast<const f32x4_t*>(pr + i);
            const f32x4_t t4 = *reinterpret_cast<const f32x4_t*>(tr + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[c][e] = (a[e] + p4[e]) + t4[e];
        }
    }
    normalise_store(v, H, lane, gamma, beta, x + (size_t)row * H, xb, row, xb_packed);
}

// One wave per score row of length S <= 512 (8 elements per lane, strided by
// 64 so that consecutive lanes touch consecutive elements).
template <int ELT>
__global__ __launch_bounds__(256) void mask_softmax_kernel(unsigned char* __restrict__ scores,
                                                           const int* __restrict__ mask, long rows,
                                                           int rows_per_batch, int S, float scale) {
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int b = (int)(row / rows_per_batch);
    const int* mrow = mask ? mask + (size_t)b * S : nullptr;
    unsigned char* base = scores + (size_t)row * S * (ELT == kBF16 ? 2 : 4);
    float v[8];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = c * 64 + lane;
        if (i < S) {
            float s = (ELT == kBF16) ? (float)reinterpret_cast<const __bf16*>(base)[i]
                                     : reinterpret_cast<const float*>(base)[i];
            s = s * scale + (mrow ? (1.0f - (float)mrow[i]) * -10000.0f : 0.0f);
            v[c] = s;
            mx = fmaxf(mx, s);
        }
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c)
        if (c * 64 + lane < S) {
            v[c] = expf(v[c] - mx);
            sum += v[c];
        }
    const float inv = 1.0f / wave_sum(sum);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = c * 64 + lane;
        if (i < S) {
            if constexpr (ELT == kBF16) reinterpret_cast<__bf16*>(base)[i] = (__bf16)(v[c] * inv);
            else reinterpret_cast<float*>(base)[i] = v[c] * inv;
        }
    }
}

// Maximum / sum over a group of `lpr` (8, 16, 32 or 64; wave-uniform) consecutive lanes, result in every lane of the
// group: quad permutes, the mirrors of 8 and of 16 lanes, a swizzle for the other half of 32 and one exchange across
// the halves of the wave -- no trip through the LDS crossbar until the last two.
template <bool MAX>
__device__ __forceinline__ float lane_group_reduce(float v, int lpr) {
    auto comb = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
    v = comb(v, ln_dpp_lanes<0xB1>(v));        // lane ^ 1
    v = comb(v, ln_dpp_lanes<0x4E>(v));        // lane ^ 2
    v = comb(v, ln_dpp_lanes<0x141>(v));       // the other quad of 8 lanes
    if (lpr >= 16) v = comb(v, ln_dpp_lanes<0x140>(v));       // the other 8 of 16 lanes
    if (lpr >= 32) v = comb(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)));   // lane ^ 16
    if (lpr >= 64) v = MAX ? half_swap_max(v) : half_swap_sum(v);
    return v;
}

// Vectorised form for rows whose byte length is a multiple of 16 (S % 4 == 0 for
// float32, S % 8 == 0 for bf16): a row is cut into 16-byte chunks, a group of LPR
// lanes (a power of two, 8..64) owns one row and each lane U chunks, so a wave
// moves 64/LPR whole rows with full-width loads and stores and the reductions
// stay inside the lane group.
template <int ELT, int U, int RU>
__global__ __launch_bounds__(256) void mask_softmax_vec_kernel(unsigned char* __restrict__ scores,
                                                               const int* __restrict__ mask, long rows,
                                                               int rows_per_batch, int S, float scale, int lpr) {
    constexpr int ES = (ELT == kBF16) ? 2 : 4;
    constexpr int EPC = 16 / ES;                 // elements per chunk
    const int lane = threadIdx.x & 63;
    const int sub = lane / lpr, sl = lane - sub * lpr;
    // a lane group works on RU consecutive rows at a time: RU * U independent loads in flight per lane
    const long row0 = (((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / lpr) + sub) * RU;
    const int chunks = S / EPC;
    uint4 raw[RU][U];
#pragma unroll
    for (int r = 0; r < RU; ++r)
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ci = u * lpr + sl;
            if (row0 + r < rows && ci < chunks)
                raw[r][u] = *reinterpret_cast<const uint4*>(scores + ((size_t)(row0 + r) * S * ES + (size_t)ci * 16));
        }
    // Softmax in the exp2 domain: t = s * (scale log2 e) + (1 - m) * (-10000 log2 e).  The mask
    // terms of this lane's chunks are shared by all rows of a batch entry; they are rebuilt
    // only when the row group crosses into the next entry.
    const float c2 = scale * 1.4426950408889634f;
    float madd[U][EPC];
    int madd_b = -1;
#pragma unroll
    for (int r = 0; r < RU; ++r) {
        const long row = row0 + r;
        const bool live = row < rows;
        const int b = live ? (int)(row / rows_per_batch) : 0;
        if (b != madd_b) {
            madd_b = b;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ci = u * lpr + sl;
#pragma unroll
                for (int e4 = 0; e4 < EPC / 4; ++e4) {
                    int4 m4 = {1, 1, 1, 1};
                    if (mask && ci < chunks) m4 = *reinterpret_cast<const int4*>(mask + (size_t)b * S + ci * EPC + 4 * e4);
                    const int mm[4] = {m4.x, m4.y, m4.z, m4.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) madd[u][4 * e4 + e] = (1.0f - (float)mm[e]) * -14426.950408889634f;
                }
            }
        }
        float v[U][EPC];
        float mx = -INFINITY;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ci = u * lpr + sl;
            if (live && ci < chunks) {
                if constexpr (ELT == kBF16) {
                    const unsigned w[4] = {raw[r][u].x, raw[r][u].y, raw[r][u].z, raw[r][u].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[u][2 * e] = __uint_as_float(w[e] << 16);
                        v[u][2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                    }
                } else {
                    v[u][0] = __uint_as_float(raw[r][u].x); v[u][1] = __uint_as_float(raw[r][u].y);
                    v[u][2] = __uint_as_float(raw[r][u].z); v[u][3] = __uint_as_float(raw[r][u].w);
                }
#pragma unroll
                for (int e = 0; e < EPC; ++e) {
                    const float t = fmaf(v[u][e], c2, madd[u][e]);
                    v[u][e] = t;
                    mx = fmaxf(mx, t);
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPC; ++e) v[u][e] = -INFINITY;
            }
        }
        mx = lane_group_reduce<true>(mx, lpr);
        if (!live) mx = 0.0f;                      // keeps exp(-inf - mx) well defined for absent rows
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < EPC; ++e) {
                v[u][e] = __builtin_amdgcn_exp2f(v[u][e] - mx);     // 0 for the chunks this lane does not own
                sum += v[u][e];
            }
        sum = lane_group_reduce<false>(sum, lpr);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ci = u * lpr + sl;
            if (live && ci < chunks) {
                uint4 o;
                if constexpr (ELT == kBF16) {
                    unsigned w[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const __bf16 lo = (__bf16)(v[u][2 * e] * inv), hi = (__bf16)(v[u][2 * e + 1] * inv);
                        w[e] = (unsigned)__builtin_bit_cast(unsigned short, lo) |
                               ((unsigned)__builtin_bit_cast(unsigned short, hi) << 16);
                    }
                    o = make_uint4(w[0], w[1], w[2], w[3]);
                } else {
                    o = make_uint4(__float_as_uint(v[u][0] * inv), __float_as_uint(v[u][1] * inv),
                                   __float_as_uint(v[u][2] * inv), __float_as_uint(v[u][3] * inv));
                }
                *reinterpret_cast<uint4*>(scores + ((size_t)row * S * ES + (size_t)ci * 16)) = o;
            }
        }
    }
}

// probs[b, :] = softmax(pooled[b, :] @ kernel[H, C] + bias); one wave per row.
__global__ __launch_bounds__(64) void classifier_kernel(const float* __restrict__ pooled,
                                                        const float* __restrict__ kernel,
                                                        const float* __restrict__ bias,
                                                        float* __restrict__ probs, int H, int C) {
    const int lane = threadIdx.x, b = blockIdx.x;
    float acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = 0.0f;
    for (int i = lane; i < H; i += 64) {
        const float p = pooled[(size_t)b * H + i];
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (c < C) acc[c] += p * kernel[(size_t)i * C + c];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < 8; ++c)
        if (c < C) {
            acc[c] = wave_sum(acc[c]) + bias[c];
            mx = fmaxf(mx, acc[c]);
        }
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c)
        if (c < C) {
            acc[c] = expf(acc[c] - mx);
            sum += acc[c];
        }
    if (lane == 0) {
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (c < C) probs[(size_t)b * C + c] = acc[c] / sum;
    }
}

// dst[n, k] = src[k, n]; 32x32 tiles through LDS (padded against conflicts).
template <int ELT>
__global__ __launch_bounds__(256) void transpose_convert_kernel(const float* __restrict__ src,
                                                                unsigned char* __restrict__ dst, int K,
                                                                int N, int packed, int row0) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;      // 32 x 8
    const int n0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int kk = k0 + r, nn = n0 + tx;
        tile[r][tx] = (kk < K && nn < N) ? src[(size_t)kk * N + nn] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int nn = n0 + r, kk = k0 + tx;
        if (nn < N && kk < K) {
            const float val = tile[tx][r];
            if constexpr (ELT == kBF16) {
                const size_t off = packed ? packed_offset(row0 + nn, kk * 2, K * 2 / 64) : ((size_t)nn * K + kk) * 2;
                *reinterpret_cast<__bf16*>(dst + off) = (__bf16)val;
            } else {
                reinterpret_cast<float*>(dst)[(size_t)nn * K + kk] = val;
            }
        }
    }
}

__global__ void fill_f32_kernel(float* dst, float value, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = value;
}

// pooled[b, n] = tanh(bias[n] + sum_k x[b * S, k] * W[n, k]): the first-token
// gather (row stride S*H of the float32 sequence output), the dense layer and
// the tanh in one pass.  A workgroup handles one batch row and 16 outputs; each
// wave 4 outputs, lanes split K.  W is [H, H] row-major ([out, in]).
template <int ELT>
__global__ __launch_bounds__(256) void pooler_kernel(const float* __restrict__ x, const unsigned char* __restrict__ W,
                                                     const float* __restrict__ bias, float* __restrict__ pooled,
                                                     int S, int H, const int* __restrict__ cu) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.x;
    const float* xr = x + (cu ? (size_t)cu[b] : (size_t)b * S) * H;      // first token of sequence b
    float xv[kMaxChunks][4];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c) {
        const int i = c * 256 + lane * 4;
        if (i < H) {
            const f32x4_t t = *reinterpret_cast<const f32x4_t*>(xr + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) xv[c][e] = t[e];
        }
    }
    // the wave's four weight rows are requested together: a one-sequence batch has nothing else to
    // hide the latency behind
    constexpr int WES = ELT == kBF16 ? 2 : 4;
    typedef typename std::conditional<ELT == kBF16, bf16x4_t, f32x4_t>::type wvec_t;
    wvec_t w4[4][kMaxChunks];
#pragma unroll
    for (int o = 0; o < 4; ++o) {
        const int n = blockIdx.y * 16 + wave * 4 + o;
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c) {
            const int i = c * 256 + lane * 4;
            if (i < H) w4[o][c] = *reinterpret_cast<const wvec_t*>(W + ((size_t)(n < H ? n : H - 1) * H + i) * WES);
        }
    }
#pragma unroll
    for (int o = 0; o < 4; ++o) {
        const int n = blockIdx.y * 16 + wave * 4 + o;
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c) {
            const int i = c * 256 + lane * 4;
            if (i < H) {
#pragma unroll
                for (int e = 0; e < 4; ++e) acc += xv[c][e] * (float)w4[o][c][e];
            }
        }
        acc = wave_sum(acc);
        if (lane == 0 && n < H) pooled[(size_t)b * H + n] = tanhf(acc + bias[n]);
    }
}

// out[b, s, :] = s < len(b) ? xc[cu[b] + s, :] : 0; one wave per padded token row.
__global__ __launch_bounds__(256) void unpad_rows_kernel(const float* __restrict__ xc, const int* __restrict__ cu,
                                                         float* __restrict__ out, int B, int S, int H) {
    const int lane = threadIdx.x & 63;
    const long tok = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= (long)B * S) return;
    const int b = (int)(tok / S), s = (int)(tok - (long)b * S);
    const int first = cu[b], len = cu[b + 1] - first;
    const float* src = xc + (size_t)(first + s) * H;
    float* dst = out + (size_t)tok * H;
    for (int i = lane * 4; i < H; i += 256) {
        f32x4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (s < len) v = *reinterpret_cast<const f32x4_t*>(src + i);
        *reinterpret_cast<f32x4_t*>(dst + i) = v;
    }
}

// out[b, :] = x[first row of sequence b, :]; one wave per sequence.
__global__ __launch_bounds__(256) void gather_first_rows_kernel(const float* __restrict__ x, const int* __restrict__ cu,
                                                                float* __restrict__ out, int B, int S, int H) {
    const int lane = threadIdx.x & 63;
    const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= B) return;
    const float* src = x + (cu ? (size_t)cu[b] : (size_t)b * S) * H;
    for (int i = lane * 4; i < H; i += 256)
        *reinterpret_cast<f32x4_t*>(out + (size_t)b * H + i) = *reinterpret_cast<const f32x4_t*>(src + i);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

bool launch_add_layernorm(float* x, const void* y, int y_elt, const float* gamma, const float* beta,
                          bf16_t* xb, bool xb_packed, int rows, int H, hipStream_t stream, int y_parts, bool add_x) {
    if (!add_x && !y) { set_error("layernorm: without the residual stream an addend is required"); return false; }
    if (y_parts < 1 || (y_parts > 1 && (!y || y_elt != kF32))) { set_error("layernorm: partial addends must be float32"); return false; }
    if (xb && xb_packed && H % 32 != 0) { set_error("layernorm: a packed copy needs H to be a multiple of 32"); return false; }
    const int xp = xb_packed ? 1 : 0;
    if (rows <= 0 || H <= 0 || H % 4 != 0 || H > kMaxChunks * 256) {
        set_error("layernorm: H must be a multiple of 4 and at most 1024");
        return false;
    }
    if (!x || !gamma || !beta || !aligned16(x) || !aligned16(gamma) || !aligned16(beta) ||
        (y && !aligned16(y)) || (xb && !aligned16(xb))) {
        set_error("layernorm: null or misaligned operand");
        return false;
    }
    dim3 grid((rows + 3) / 4), block(256);
    const unsigned char* yc = static_cast<const unsigned char*>(y);
    if (!y) hipLaunchKernelGGL(add_layernorm_kernel<-1>, grid, block, 0, stream, x, yc, gamma, beta, xb, rows, H, xp, y_parts, add_x ? 1 : 0);
    else if (y_elt == kF32 && y_parts > 1) hipLaunchKernelGGL(add_layernorm_parts_kernel, dim3(rows), block, 0, stream, x, static_cast<const float*>(y), gamma, beta, xb, rows, H, xp, y_parts, add_x ? 1 : 0);
    else if (y_elt == kF32) hipLaunchKernelGGL(add_layernorm_kernel<kF32>, grid, block, 0, stream, x, yc, gamma, beta, xb, rows, H, xp, y_parts, add_x ? 1 : 0);
    else if (y_elt == kBF16) hipLaunchKernelGGL(add_layernorm_kernel<kBF16>, grid, block, 0, stream, x, yc, gamma, beta, xb, rows, H, xp, y_parts, add_x ? 1 : 0);
    else { set_error("layernorm: bad addend type"); return false; }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_embed_layernorm(const int* ids, const int* seg, const int* mask, const float* word,
                            const float* pos, const float* type, const float* gamma, const float* beta,
                            float* x, bf16_t* xb, bool xb_packed, float* maskadd, int B, int S, int Sp, int H,
                            int vocab, int type_vocab, hipStream_t stream, const Compact* compact) {
    if (compact && (!compact->rowmap || !compact->cu || compact->rows <= 0 || compact->rows > (long)B * S)) {
        set_error("embedding: bad compact-row description");
        return false;
    }
    if (xb && xb_packed && H % 32 != 0) { set_error("embedding: a packed copy needs H to be a multiple of 32"); return false; }
    if (B <= 0 || S <= 0 || H <= 0 || H % 4 != 0 || H > kMaxChunks * 256) {
        set_error("embedding: H must be a multiple of 4 and at most 1024");
        return false;
    }
    if (Sp < S || Sp - S >= 32 || Sp % 32 != 0) { set_error("embedding: bad padded length"); return false; }
    if (!ids || !word || !pos || !type || !gamma || !beta || !x || !maskadd || vocab <= 0 || type_vocab <= 0) {
        set_error("embedding: null operand");
        return false;
    }
    if (!aligned16(word) || !aligned16(pos) || !aligned16(type) || !aligned16(gamma) || !aligned16(beta) ||
        !aligned16(x) || (xb && !aligned16(xb))) {
        set_error("embedding: misaligned operand");
        return false;
    }
    const long rows = compact ? compact->rows : (long)B * S;
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    hipLaunchKernelGGL(embed_layernorm_kernel, grid, block, 0, stream, ids, seg, mask, word, pos, type, gamma,
                       beta, x, xb, maskadd, B, S, Sp, H, vocab, type_vocab, xb_packed ? 1 : 0,
                       compact ? compact->rowmap : nullptr, compact ? compact->cu : nullptr, (int)rows);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

// rows a lane group of the vector softmax kernel holds at a time when a row fits one 16-byte chunk per lane
// (bf16: eight rows in flight measured 2 % faster than four)
constexpr int kSoftmaxRowsBf16 = 8;

bool launch_mask_softmax(void* scores, int elt, const int* mask, int B, int rows_per_batch, int S, float scale,
                         hipStream_t stream) {
    if (B <= 0 || rows_per_batch <= 0 || S <= 0 || S > 512) {
        set_error("softmax: row length must be in 1..512");
        return false;
    }
    if (!scores) { set_error("softmax: null operand"); return false; }
    const long rows = (long)B * rows_per_batch;
    unsigned char* sc = static_cast<unsigned char*>(scores);
    if (elt != kBF16 && elt != kF32) { set_error("softmax: bad element type"); return false; }
    const int es = elt == kBF16 ? 2 : 4;
    if ((S * es) % 16 == 0 && (reinterpret_cast<uintptr_t>(scores) & 15) == 0 &&
        (!mask || (reinterpret_cast<uintptr_t>(mask) & 15) == 0)) {
        const int chunks = S * es / 16;
        const int u = chunks > 64 ? 2 : 1;
        int lpr = 8;
        while (lpr * u < chunks) lpr *= 2;
        const int ru = u == 1 ? (elt == kBF16 ? kSoftmaxRowsBf16 : 4) : 2;
        const long per_wave = (long)(64 / lpr) * ru;
        const long waves = (rows + per_wave - 1) / per_wave;
        const long nblk = (waves + 3) / 4;
        if (nblk > 0x7fffffffL) { set_error("softmax: too many rows"); return false; }
        dim3 g((unsigned)nblk), blk(256);
        if (elt == kBF16 && u == 1) hipLaunchKernelGGL((mask_softmax_vec_kernel<kBF16, 1, kSoftmaxRowsBf16>), g, blk, 0, stream, sc, mask, rows, rows_per_batch, S, scale, lpr);
        else if (elt == kBF16) hipLaunchKernelGGL((mask_softmax_vec_kernel<kBF16, 2, 2>), g, blk, 0, stream, sc, mask, rows, rows_per_batch, S, scale, lpr);
        else if (u == 1) hipLaunchKernelGGL((mask_softmax_vec_kernel<kF32, 1, 4>), g, blk, 0, stream, sc, mask, rows, rows_per_batch, S, scale, lpr);
        else hipLaunchKernelGGL((mask_softmax_vec_kernel<kF32, 2, 2>), g, blk, 0, stream, sc, mask, rows, rows_per_batch, S, scale, lpr);
        CUBERT_HIP_OK(hipGetLastError());
        return true;
    }
    const long blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffffL) { set_error("softmax: too many rows"); return false; }
    dim3 grid((unsigned)blocks), block(256);
    if (elt == kBF16) hipLaunchKernelGGL(mask_softmax_kernel<kBF16>, grid, block, 0, stream, sc, mask, rows, rows_per_batch, S, scale);
    else if (elt == kF32) hipLaunchKernelGGL(mask_softmax_kernel<kF32>, grid, block, 0, stream, sc, mask, rows, rows_per_batch, S, scale);
    else { set_error("softmax: bad element type"); return false; }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_classifier(const float* pooled, const float* kernel, const float* bias, float* probs, int B, int H,
                       int C, hipStream_t stream) {
    if (B <= 0 || H <= 0 || C <= 0 || C > 8) { set_error("classifier: supports 1..8 classes"); return false; }
    if (!pooled || !kernel || !bias || !probs) { set_error("classifier: null operand"); return false; }
    hipLaunchKernelGGL(classifier_kernel, dim3(B), dim3(64), 0, stream, pooled, kernel, bias, probs, H, C);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_pooler(const float* x, const void* W, int w_elt, const float* bias, float* pooled, int B, int S, int H,
                   hipStream_t stream, const int* cu) {
    if (B <= 0 || S <= 0 || H <= 0 || H % 4 != 0 || H > kMaxChunks * 256) {
        set_error("pooler: H must be a multiple of 4 and at most 1024");
        return false;
    }
    if (!x || !W || !bias || !pooled || !aligned16(x) || !aligned16(W)) { set_error("pooler: null or misaligned operand"); return false; }
    if (B > 65535) { set_error("pooler: batch too large"); return false; }
    dim3 grid(B, (H + 15) / 16), block(256);
    const unsigned char* wc = static_cast<const unsigned char*>(W);
    if (w_elt == kBF16) hipLaunchKernelGGL(pooler_kernel<kBF16>, grid, block, 0, stream, x, wc, bias, pooled, S, H, cu);
    else if (w_elt == kF32) hipLaunchKernelGGL(pooler_kernel<kF32>, grid, block, 0, stream, x, wc, bias, pooled, S, H, cu);
    else { set_error("pooler: bad weight type"); return false; }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_gather_first_rows(const float* x, const int* cu, float* out, int B, int S, int H, hipStream_t stream) {
    if (!x || !out || B <= 0 || S <= 0 || H <= 0 || H % 4 != 0 || !aligned16(x) || !aligned16(out)) {
        set_error("gather: bad arguments");
        return false;
    }
    hipLaunchKernelGGL(gather_first_rows_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, stream, x, cu, out, B, S, H);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_unpad_rows(const float* xc, const int* cu, float* out, int B, int S, int H, hipStream_t stream) {
    if (!xc || !cu || !out || B <= 0 || S <= 0 || H <= 0 || H % 4 != 0 || !aligned16(xc) || !aligned16(out)) {
        set_error("unpad: bad arguments");
        return false;
    }
    const long rows = (long)B * S;
    hipLaunchKernelGGL(unpad_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, xc, cu, out, B, S, H);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_transpose_convert(const float* src, void* dst, int K, int N, int elt, bool packed, int row0,
                              hipStream_t stream) {
    if (!src || !dst || K <= 0 || N <= 0) { set_error("transpose: bad arguments"); return false; }
    if (packed && (elt != kBF16 || K % 32 != 0)) { set_error("transpose: packed output is bf16 with K a multiple of 32"); return false; }
    const int pk = packed ? 1 : 0;
    dim3 grid((N + 31) / 32, (K + 31) / 32), block(256);
    unsigned char* d = static_cast<unsigned char*>(dst);
    if (elt == kBF16) hipLaunchKernelGGL(transpose_convert_kernel<kBF16>, grid, block, 0, stream, src, d, K, N, pk, row0);
    else if (elt == kF32) hipLaunchKernelGGL(transpose_convert_kernel<kF32>, grid, block, 0, stream, src, d, K, N, pk, row0);
    else { set_error("transpose: bad element type"); return false; }
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

bool launch_fill_f32(float* dst, float value, size_t n, hipStream_t stream) {
    if (!dst || n == 0) return true;
    size_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, dst, value, n);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

}  // namespace cubert
