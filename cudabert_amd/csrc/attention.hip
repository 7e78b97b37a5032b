// Fused self-attention for head dim 64 on gfx950:
//   ctx = softmax(Q K^T * scale + maskadd) V        per (batch, head)
//
// One wave64 owns 32 query rows and walks the keys in blocks of 32 with an
// online softmax, so the [S, S] score matrix never leaves registers.
//
// The score block is computed TRANSPOSED (keys x queries): K rows feed the
// MFMA "A" operand and Q rows the "B" operand.  In the 32x32 accumulator
// layout a lane then owns ONE query (column lane % 32) and 16 keys
// (8*(v/4) + 4*(lane/32) + v%4), so the row maximum and row sum of the softmax
// are 16 in-register operations plus one exchange with lane ^ 32.  The
// probabilities stay in registers and feed the second MFMA as its "B" operand
// (k = key); V is read from a pre-transposed [64, Sp] layout (written by the
// QKV GEMM epilogue) so that the "A" operand lane (d, g) picks up the keys
// that match the probability lane's k slots with 8/16-byte loads.  The
// context comes out transposed too: a lane holds one query and four
// consecutive head features per accumulator quad -> vector stores into the
// row-major [tokens, hidden] context matrix.
#include <atomic>

#include "kernels.h"

namespace cubert {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;

template <int ELT>
__global__ __launch_bounds__(256) void attention_kernel(
    const unsigned char* __restrict__ q, const unsigned char* __restrict__ k,
    const unsigned char* __restrict__ vt, const float* __restrict__ maskadd,
    unsigned char* __restrict__ ctx, int heads, int S, int Sp, float scale, int ctx_packed,
    const int* __restrict__ cu, int first_only) {
    constexpr int ES = (ELT == kBF16) ? 2 : 4;
    constexpr int ROWB = 64 * ES;            // bytes per Q/K row
    constexpr int KK = ROWB / 32;            // MFMA k-steps over the head dim (4 bf16 / 8 f32)

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, g = lane >> 5;
    const int h = blockIdx.y, b = blockIdx.z;
    const int q0 = (blockIdx.x * 4 + wave) * 32;
    // compact rows: only queries below the sequence's length exist, at rows cu[b] + query
    const int qlen = cu ? cu[b + 1] - cu[b] : S;
    // first_only: only query 0 of every sequence is wanted, as row b of a [B, hidden] context
    const size_t row_base = first_only ? (size_t)b : cu ? (size_t)cu[b] : (size_t)b * S;
    if (q0 >= qlen || (first_only && q0 != 0)) return;      // whole wave leaves; no barriers below

    const size_t bh = (size_t)b * heads + h;
    const unsigned char* qb = q + bh * S * ROWB;
    const unsigned char* kb = k + bh * S * ROWB;
    const unsigned char* vb = vt + bh * 64 * (size_t)Sp * ES;
    const float* mrow = maskadd + (size_t)b * Sp;

    // Q fragments ("B" operand: column = query), kept for the whole key loop.
    int qrow = q0 + l32;
    qrow = qrow < S ? qrow : S - 1;
    uint4 qf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
        qf[kk] = *reinterpret_cast<const uint4*>(qb + (size_t)qrow * ROWB + (2 * kk + g) * 16);

    f32x16_t o[2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.0f;
    float run_max = -INFINITY, run_sum = 0.0f;

    // Key blocks in which every key is masked are skipped: with at least one visible key in the row
    // their probabilities are exactly zero in float32 (exp of less than -9000), whether they are met
    // before or after a visible block (the rescaling by exp(-9000) = 0 wipes what they added), so the
    // result has the bits of walking them.  If no key at all is visible nothing is skipped.
    unsigned long long live = 0ull;
    for (int blk = 0; blk * 32 < S && blk < 64; ++blk) {
        const float m = lane < 32 ? mrow[blk * 32 + lane] : -INFINITY;       // mrow has Sp entries
        if (__ballot(m > -5000.0f) != 0ull) live |= 1ull << blk;
    }
    if (live == 0ull || S > 64 * 32) live = ~0ull;

    for (int k0 = 0; k0 < S; k0 += 32) {
        if (!((live >> ((k0 >> 5) & 63)) & 1ull)) continue;
        // ---- scores^T block: rows = keys k0..k0+31, column = my query ----
        int krow = k0 + l32;
        krow = krow < S ? krow : S - 1;
        f32x16_t sc;
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const uint4 kf = *reinterpret_cast<const uint4*>(kb + (size_t)krow * ROWB + (2 * kk + g) * 16);
            if constexpr (ELT == kBF16) {
                sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf),
                                                             __builtin_bit_cast(bf16x8_t, qf[kk]), sc, 0, 0, 0);
            } else {
                const f32x4_t fa = __builtin_bit_cast(f32x4_t, kf);
                const f32x4_t fb = __builtin_bit_cast(f32x4_t, qf[kk]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    sc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[e], fb[e], sc, 0, 0, 0);
            }
        }
        // ---- scale + additive mask (padding columns carry -inf) ----
        float blk_max = -INFINITY;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4_t m4 = *reinterpret_cast<const f32x4_t*>(mrow + k0 + 8 * j + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float s = sc[4 * j + e] * scale + m4[e];
                sc[4 * j + e] = s;
                blk_max = fmaxf(blk_max, s);
            }
        }
        blk_max = half_swap_max(blk_max);
        const float new_max = fmaxf(run_max, blk_max);    // finite: key 0 is never padding
        const float alpha = __expf(run_max - new_max);    // exp(-inf) = 0 on the first block
        float blk_sum = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float pv = __expf(sc[v] - new_max);
            sc[v] = pv;
            blk_sum += pv;
        }
        blk_sum = half_swap_sum(blk_sum);
        run_sum = run_sum * alpha + blk_sum;
        run_max = new_max;
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[db][v] *= alpha;

        // ---- ctx^T += V^T (rows = head features) x P^T (column = my query) ----
        if constexpr (ELT == kBF16) {
#pragma unroll
            for (int f = 0; f < 2; ++f) {        // keys k0 + 16 f + {4g..4g+3, 8+4g..8+4g+3}
                bf16x8_t pf;
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[e] = (__bf16)sc[8 * f + e];
#pragma unroll
                for (int db = 0; db < 2; ++db) {
                    const unsigned char* vrow = vb + ((size_t)(32 * db + l32) * Sp + k0 + 16 * f + 4 * g) * 2;
                    const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
                    const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 16);
                    const uint4 vf = {lo.x, lo.y, hi.x, hi.y};
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf), pf,
                                                                  o[db], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {    // keys k0 + 8 j + 4 g + e
                    const f32x4_t v4 = *reinterpret_cast<const f32x4_t*>(
                        vb + ((size_t)(32 * db + l32) * Sp + k0 + 8 * j + 4 * g) * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(v4[e], sc[4 * j + e], o[db], 0, 0, 0);
                }
            }
        }
    }

    // ---- normalise and store: lane owns query q0 + l32, features 32 db + 8 j + 4 g + e ----
    const int qi = q0 + l32;
    if (qi >= qlen || (first_only && qi != 0)) return;
    const float inv = 1.0f / run_sum;
    const size_t hidden = (size_t)heads * 64;
    unsigned char* orow = ctx + ((row_base + qi) * hidden + (size_t)h * 64) * ES;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = 32 * db + 8 * j + 4 * g;
            if constexpr (ELT == kBF16) {
                bf16x4_t w = {(__bf16)(o[db][4 * j] * inv), (__bf16)(o[db][4 * j + 1] * inv),
                              (__bf16)(o[db][4 * j + 2] * inv), (__bf16)(o[db][4 * j + 3] * inv)};
                if (ctx_packed)
                    *reinterpret_cast<bf16x4_t*>(ctx + packed_offset((int)row_base + qi, (h * 64 + d) * 2, (int)hidden * 2 / 64)) = w;
                else
                    *reinterpret_cast<bf16x4_t*>(orow + d * 2) = w;
            } else {
                f32x4_t w = {o[db][4 * j] * inv, o[db][4 * j + 1] * inv, o[db][4 * j + 2] * inv,
                             o[db][4 * j + 3] * inv};
                *reinterpret_cast<f32x4_t*>(orow + d * 4) = w;
            }
        }
}


// ---------------------------------------------------------------------------
// bf16, S <= 512: one workgroup per (batch, head) with one wave per block of 32
// queries.  K [S, 64] and V^T [64, Sp] of the head are brought into LDS once
// (instead of once per wave through the vector memory path) and every wave
// takes its MFMA operands from there:
//   K    rows of 128 bytes, 16-byte chunk c of row r in slot c ^ (r & 7)
//        (the 32 lanes of a fragment read hit 8 different slots);
//   V^T  rows `vstride` = 8 (mod 256) bytes apart, so that the 32 rows a
//        fragment read touches start in 32 different bank pairs;
//   the additive mask row, premultiplied by log2(e): the softmax runs in the
//        exp2 domain, s' = score * (scale * log2 e) + mask * log2 e.
// Key blocks in which every key is masked are skipped: with at least one
// visible key in the row their probabilities are exactly zero in float32
// (exp2 of less than -14000), so the result is bit-identical to walking them.
// If no key at all is visible nothing is skipped.
//
// VROW: V arrives as [S, 64] rows like K (the QKV GEMM then stores it in whole row segments instead
// of two bytes at a time).  It sits in the LDS as rows of 128 bytes whose four 32-byte blocks are
// permuted by (row >> 1) & 3, and the transposition the second MFMA needs happens in the read:
// ds_read_b64_tr_b16 hands lane i of a group of 16 the i-th 16-bit element of each of the four
// 32-byte pieces that lanes 4r .. 4r+3 (r = 0..3) point at, so with piece r = 16 features of key
// kb + r a lane receives its feature for four consecutive keys.  The block permutation puts the
// four pieces of a group into four different bank ranges.
template <bool VROW>
__global__ __launch_bounds__(1024) void attention_lds_kernel(
    const unsigned char* __restrict__ q, const unsigned char* __restrict__ k,
    const unsigned char* __restrict__ vt, const float* __restrict__ maskadd,
    unsigned char* __restrict__ ctx, int heads, int S, int Sp, int vstride, float scale_log2e, int ctx_packed,
    const int* __restrict__ cu, int first_only) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* sK = smem;
    unsigned char* sV = smem + (size_t)Sp * 128;
    float* sM = reinterpret_cast<float*>(sV + (VROW ? (size_t)Sp * 128 : 64 * (size_t)vstride));
    int* sLive = reinterpret_cast<int*>(sM + Sp);

    const int tid = threadIdx.x, nthr = blockDim.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g = lane >> 5;
    const int nblk = Sp >> 5;                  // == number of waves
    const int h = blockIdx.x, b = blockIdx.y;
    const size_t bh = (size_t)b * heads + h;
    const unsigned char* qb = q + bh * S * 128;
    const unsigned char* kb = k + bh * S * 128;
    const unsigned char* vb = vt + (VROW ? bh * S * 128 : bh * 64 * (size_t)Sp * 2);

    // Q fragments ("B" operand: column = query), kept for the whole key loop.  Requested first, together with the
    // K / V loads below: a short batch's launch is one chain of round trips, and this one is then not a link of it.
    const int q0 = wave * 32;
    // compact rows: only queries below the sequence's length exist, at rows cu[b] + query
    const int qlen = cu ? cu[b + 1] - cu[b] : S;
    uint4 qf[4];
    {
        int qrow = q0 + l32;
        qrow = qrow < qlen ? qrow : qlen - 1;       // qlen >= 1; a wave past the end leaves after the barrier, its loads are harmless
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            qf[kk] = *reinterpret_cast<const uint4*>(qb + (size_t)qrow * 128 + (2 * kk + g) * 16);
    }
    // ---- stage K (rows S..Sp-1 zero), V^T and the mask row ----
    // The workgroup has 2 Sp threads, K is 8 Sp and V^T 8 Sp 16-byte chunks: four of each per
    // thread.  All eight loads are issued before the first LDS write so that their latencies
    // overlap instead of adding up.
    const int vchunks = Sp >> 3;               // 16-byte chunks per V^T row
    uint4 kd[4], vd[4];
    int vrow_i[4], vch_i[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + i * nthr;
        kd[i] = make_uint4(0u, 0u, 0u, 0u);
        if ((c >> 3) < S) kd[i] = *reinterpret_cast<const uint4*>(kb + (size_t)c * 16);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + i * nthr;
        if constexpr (VROW) {
            vrow_i[i] = c >> 3;
            vch_i[i] = c & 7;
            vd[i] = make_uint4(0u, 0u, 0u, 0u);
            if (vrow_i[i] < S) vd[i] = *reinterpret_cast<const uint4*>(vb + (size_t)c * 16);
        } else {
            vrow_i[i] = c / vchunks;
            vch_i[i] = c - vrow_i[i] * vchunks;
            vd[i] = *reinterpret_cast<const uint4*>(vb + ((size_t)vrow_i[i] * Sp + vch_i[i] * 8) * 2);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + i * nthr;
        const int row = c >> 3, ch = c & 7;
        *reinterpret_cast<uint4*>(sK + row * 128 + ((ch ^ (row & 7)) << 4)) = kd[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (VROW) {
            const int row = vrow_i[i], ch = vch_i[i];
            *reinterpret_cast<uint4*>(sV + row * 128 + ((((ch >> 1) ^ ((row >> 1) & 3)) << 5) | ((ch & 1) << 4))) = vd[i];
        } else {
            uint2* dst = reinterpret_cast<uint2*>(sV + (size_t)vrow_i[i] * vstride + vch_i[i] * 16);     // rows are 8-byte aligned
            dst[0] = make_uint2(vd[i].x, vd[i].y);
            dst[1] = make_uint2(vd[i].z, vd[i].w);
        }
    }
    {
        // wave w looks at mask block w
        const float m = lane < 32 ? maskadd[(size_t)b * Sp + wave * 32 + lane] : -INFINITY;
        if (lane < 32) sM[wave * 32 + lane] = m * 1.4426950408889634f;
        const unsigned long long vis = __ballot(m > -5000.0f);
        const unsigned long long zero = __ballot(lane < 32 && m == 0.0f);
        // bit 0: some key of the block is visible; bit 1: all 32 are, with a zero mask term
        if (lane == 0) sLive[wave] = (vis != 0ull ? 1 : 0) | (zero == 0xffffffffull ? 2 : 0);
    }
    __syncthreads();
    unsigned live = 0, plain = 0;
    for (int i = 0; i < nblk; ++i) {
        const int f = sLive[i];
        live |= (f & 1) ? (1u << i) : 0u;
        plain |= (f & 2) ? (1u << i) : 0u;
    }
    if (live == 0) live = 0xffffffffu;
    live = __builtin_amdgcn_readfirstlane(live);
    plain = __builtin_amdgcn_readfirstlane(plain);

    // first_only: only query 0 of every sequence is wanted, as row b of a [B, hidden] context.  Wave 0 still works on
    // its 32 queries (a query's bits depend on when its wave moves the reference exponent, i.e. on its wave mates)
    // and stores one of them.
    const size_t row_base = first_only ? (size_t)b : cu ? (size_t)cu[b] : (size_t)b * S;
    if (q0 >= qlen || (first_only && wave != 0)) return;      // past the last barrier: a whole wave may leave
    f32x16_t o[2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] = 0.0f;
    float run_max = -INFINITY, run_sum = 0.0f;
    const int ksw = l32 & 7;
    // VROW: where my 8-byte piece of a transposing read lies for key block 0, f = 0, per feature block db.
    // Row 4 g + (i >> 2), i = l32 & 15; logical 32-byte block 2 db + (l32 >> 4), permuted by (row >> 1) & 3,
    // which the multiples of 8 that k0, f and the second read add to the row do not change.
    const unsigned char* vpiece[2];
    {
        const int i16 = l32 & 15, prow = 4 * g + (i16 >> 2), psw = (prow >> 1) & 3;
#pragma unroll
        for (int db = 0; db < 2; ++db)
            vpiece[db] = sV + prow * 128 + (((2 * db + (l32 >> 4)) ^ psw) << 5) + (i16 & 3) * 8;
    }

    for (int kblk = 0; kblk < nblk; ++kblk) {
        if (!((live >> kblk) & 1u)) continue;
        const int k0 = kblk * 32;
        // ---- scores^T block: rows = keys k0..k0+31, column = my query ----
        f32x16_t sc;
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = 0.0f;
        const unsigned char* krow = sK + (k0 + l32) * 128;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const uint4 kf = *reinterpret_cast<const uint4*>(krow + (((2 * kk + g) ^ ksw) << 4));
            sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf),
                                                         __builtin_bit_cast(bf16x8_t, qf[kk]), sc, 0, 0, 0);
        }
        // Softmax with a lazily moved reference exponent: p = exp2(t - ref), where ref is the row
        // maximum seen when it was last moved.  It only moves (and the sums are rescaled) when a
        // block exceeds it by more than 2^20, so that in almost every block there is no rescaling
        // of the 32 context accumulators and no second exponential; p stays below 2^20 and the
        // final division by the row sum removes the common factor.  The first processed block
        // (ref = -inf) always takes the move.
        const bool is_plain = (plain >> kblk) & 1u;           // every key visible, mask term zero
        float blk_max = -INFINITY;
        if (is_plain) {
#pragma unroll
            for (int v = 0; v < 16; ++v) blk_max = fmaxf(blk_max, sc[v]);
            blk_max *= scale_log2e;                          // scale_log2e > 0
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4_t m4 = *reinterpret_cast<const f32x4_t*>(sM + k0 + 8 * j + 4 * g);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float t = fmaf(sc[4 * j + e], scale_log2e, m4[e]);
                    sc[4 * j + e] = t;
                    blk_max = fmaxf(blk_max, t);
                }
            }
        }
        blk_max = half_swap_max(blk_max);
        if (__ballot(blk_max > run_max + 20.0f) != 0ull) {    // finite blk_max: a processed block holds a real key column
            const float new_max = fmaxf(run_max, blk_max);
            const float alpha = __builtin_amdgcn_exp2f(run_max - new_max);     // 1 for the lanes that stay
            run_sum *= alpha;
            run_max = new_max;
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[db][v] *= alpha;
        }
        float blk_sum = 0.0f;
        if (is_plain) {
            const float neg_ref = -run_max;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float pv = __builtin_amdgcn_exp2f(fmaf(sc[v], scale_log2e, neg_ref));
                sc[v] = pv;
                blk_sum += pv;
            }
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float pv = __builtin_amdgcn_exp2f(sc[v] - run_max);
                sc[v] = pv;
                blk_sum += pv;
            }
        }
        blk_sum = half_swap_sum(blk_sum);
        run_sum += blk_sum;

        // ---- ctx^T += V^T (rows = head features) x P^T (column = my query) ----
#pragma unroll
        for (int f = 0; f < 2; ++f) {        // keys k0 + 16 f + {4g..4g+3, 8+4g..8+4g+3}
            bf16x8_t pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = (__bf16)sc[8 * f + e];
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                if constexpr (VROW) {
                    // my piece: 4 features of key k0 + 16 f + 4 g + (i >> 2) (and of the key 8 further), i = l32 & 15
                    const unsigned char* piece = vpiece[db] + (k0 + 16 * f) * 128;
                    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        reinterpret_cast<__attribute__((address_space(3))) s16x4_t*>((__attribute__((address_space(3))) unsigned char*)piece));
                    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        reinterpret_cast<__attribute__((address_space(3))) s16x4_t*>((__attribute__((address_space(3))) unsigned char*)(piece + 8 * 128)));
                    const s16x8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf), pf, o[db], 0, 0, 0);
                } else {
                    const unsigned char* vrow = sV + (size_t)(32 * db + l32) * vstride + (k0 + 16 * f + 4 * g) * 2;
                    const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
                    const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 16);
                    const uint4 vf = {lo.x, lo.y, hi.x, hi.y};
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf), pf, o[db], 0, 0, 0);
                }
            }
        }
    }

    // ---- normalise and store: lane owns query q0 + l32, features 32 db + 8 j + 4 g + e ----
    const int qi = q0 + l32;
    if (qi >= qlen || (first_only && qi != 0)) return;
    const float inv = 1.0f / run_sum;
    const size_t hidden = (size_t)heads * 64;
    unsigned char* orow = ctx + ((row_base + qi) * hidden + (size_t)h * 64) * 2;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = 32 * db + 8 * j + 4 * g;
            bf16x4_t w = {(__bf16)(o[db][4 * j] * inv), (__bf16)(o[db][4 * j + 1] * inv),
                          (__bf16)(o[db][4 * j + 2] * inv), (__bf16)(o[db][4 * j + 3] * inv)};
            if (ctx_packed)
                *reinterpret_cast<bf16x4_t*>(ctx + packed_offset((int)row_base + qi, (h * 64 + d) * 2, (int)hidden * 2 / 64)) = w;
            else
                *reinterpret_cast<bf16x4_t*>(orow + d * 2) = w;
        }
}


// ---------------------------------------------------------------------------
// Short batches (bf16, S <= 512, V as [B, heads, S, 64]): with one workgroup per (batch, head) a batch of one
// occupies 16 CUs and every wave walks all key blocks one after the other.  Here a workgroup owns one block
// of 32 queries of one (batch, head) and its NW waves share the KEYS: wave w takes the key blocks w, w + NW, ...
// Nothing is staged for the workgroup: a wave requests its Q fragments, its K fragments (straight into the
// MFMA operand layout), its V rows and its mask values in one go, drops the V rows into wave-private LDS (the
// transposing read of the kernel above needs them there) and runs the same block arithmetic.  Each wave ends
// with a partial (reference exponent, row sum, context) per query; the partials meet in LDS and every thread
// finishes 32 / NW features of one query: ctx = sum_w 2^(ref_w - max ref) o_w / sum_w 2^(ref_w - max ref) sum_w.
// No key block is skipped: a masked key's probability underflows to exactly zero, and a wave whose blocks are
// all masked gets weight zero, so rows past a sequence's length (stale but finite in the compact-row pass) never
// reach a result.  K / V of a head are fetched once per query block, which only a short batch can afford.
template <int NW>
__global__ __launch_bounds__(NW * 64, 4) void attention_split_kernel(
    const unsigned char* __restrict__ q, const unsigned char* __restrict__ k,
    const unsigned char* __restrict__ v, const float* __restrict__ maskadd,
    unsigned char* __restrict__ ctx, int heads, int S, int Sp, float scale_log2e, int ctx_packed,
    const int* __restrict__ cu, int first_only) {
    constexpr int OSTRIDE = 68;                          // floats per query row of a partial context
    constexpr int OBYTES = 32 * OSTRIDE * 4;             // two V blocks (8 KiB) first, the partial context later
    constexpr int WBYTES = OBYTES + 256;                 // + the mask values of the two key blocks in flight
    __shared__ __attribute__((aligned(16))) unsigned char sW[NW * WBYTES];
    __shared__ float sRef[NW][32], sSum[NW][32];
    typedef __attribute__((address_space(3))) void* lds_ptr_t;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g = lane >> 5;
    const int h = blockIdx.x, b = blockIdx.y, q0 = blockIdx.z * 32;
    const int qlen = cu ? cu[b + 1] - cu[b] : S;
    if (q0 >= qlen) return;                              // the whole workgroup: no barrier has been met
    const int nblk = Sp >> 5;
    const size_t bh = (size_t)b * heads + h;
    const unsigned char* qb = q + bh * S * 128;
    const unsigned char* kb = k + bh * S * 128;
    unsigned char* myV = sW + wave * WBYTES;
    unsigned char* myM = myV + OBYTES;
    // V rows and mask values go from memory into this wave's LDS without passing through registers
    const __amdgpu_buffer_rsrc_t vres = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(v + bh * S * 128), 0, S * 128, 0x00020000);
    const __amdgpu_buffer_rsrc_t mres = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(maskadd + (size_t)b * Sp), 0, Sp * 4, 0x00020000);

    uint4 qf[4];
    {
        int qrow = q0 + l32;
        qrow = qrow < qlen ? qrow : qlen - 1;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            qf[kk] = *reinterpret_cast<const uint4*>(qb + (size_t)qrow * 128 + (2 * kk + g) * 16);
    }
    f32x16_t o[2];
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[db][e] = 0.0f;
    float run_max = -INFINITY, run_sum = 0.0f;
    // where my 8-byte piece of a transposing read lies in a V block (see attention_lds_kernel)
    int vpiece[2];
    {
        const int i16 = l32 & 15, prow = 4 * g + (i16 >> 2), psw = (prow >> 1) & 3;
#pragma unroll
        for (int db = 0; db < 2; ++db)
            vpiece[db] = prow * 128 + (((2 * db + (l32 >> 4)) ^ psw) << 5) + (i16 & 3) * 8;
    }

    for (int kb0 = wave; kb0 < nblk; kb0 += 2 * NW) {
        const int nb = (kb0 + NW < nblk) ? 2 : 1;
        uint4 kf[2][4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (j < nb) {
                const int k0 = (kb0 + j * NW) * 32;
                int krow = k0 + l32;
                krow = krow < S ? krow : S - 1;          // rows S .. Sp-1 do not exist; their mask term is -inf
#pragma unroll
                for (int kk = 0; kk < 4; ++kk)
                    kf[j][kk] = *reinterpret_cast<const uint4*>(kb + (size_t)krow * 128 + (2 * kk + g) * 16);
                // LDS slot s = 64 i + lane of the block holds the 16-byte chunk ch of row s >> 3, where the slot's place
                // in the row is ch with its 32-byte block permuted by the row bits (the layout of the kernel above)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int sl = lane + 64 * i, row = sl >> 3, pos = sl & 7;
                    const int ch = ((((pos >> 1) ^ ((row >> 1) & 3)) << 1) | (pos & 1));
                    int vrow = k0 + row;
                    vrow = vrow < S ? vrow : S - 1;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(vres, (lds_ptr_t)(myV + j * 4096 + i * 1024), 16, vrow * 128 + ch * 16, 0, 0, 0);
                }
            }
        }
        // mask term of key l32 of block kb0 (lanes 0 .. 31) and of block kb0 + NW (lanes 32 .. 63; beyond the row: zero)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(mres, (lds_ptr_t)myM, 4, ((kb0 + g * NW) * 32 + l32) * 4, 0, 0, 0);
        // Everything requested above is one round trip; nothing below may read this wave's LDS before it is over (the
        // transposing reads are not ordered behind the memory-to-LDS loads by the compiler).
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (j < nb) {
                f32x16_t sc;
#pragma unroll
                for (int e = 0; e < 16; ++e) sc[e] = 0.0f;
#pragma unroll
                for (int kk = 0; kk < 4; ++kk)
                    sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf[j][kk]),
                                                                 __builtin_bit_cast(bf16x8_t, qf[kk]), sc, 0, 0, 0);
                float blk_max = -INFINITY;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const f32x4_t m4 = *reinterpret_cast<const f32x4_t*>(myM + j * 128 + (8 * jj + 4 * g) * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float t = fmaf(sc[4 * jj + e], scale_log2e, m4[e] * 1.4426950408889634f);
                        sc[4 * jj + e] = t;
                        blk_max = fmaxf(blk_max, t);
                    }
                }
                blk_max = half_swap_max(blk_max);
                if (__ballot(blk_max > run_max + 20.0f) != 0ull) {
                    const float new_max = fmaxf(run_max, blk_max);
                    const float alpha = __builtin_amdgcn_exp2f(run_max - new_max);
                    run_sum *= alpha;
                    run_max = new_max;
#pragma unroll
                    for (int db = 0; db < 2; ++db)
#pragma unroll
                        for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
                }
                float blk_sum = 0.0f;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float pv = __builtin_amdgcn_exp2f(sc[e] - run_max);
                    sc[e] = pv;
                    blk_sum += pv;
                }
                blk_sum = half_swap_sum(blk_sum);
                run_sum += blk_sum;
#pragma unroll
                for (int f = 0; f < 2; ++f) {
                    bf16x8_t pf;
#pragma unroll
                    for (int e = 0; e < 8; ++e) pf[e] = (__bf16)sc[8 * f + e];
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        const unsigned char* piece = myV + j * 4096 + vpiece[db] + 16 * f * 128;
                        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            reinterpret_cast<__attribute__((address_space(3))) s16x4_t*>((__attribute__((address_space(3))) unsigned char*)piece));
                        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            reinterpret_cast<__attribute__((address_space(3))) s16x4_t*>((__attribute__((address_space(3))) unsigned char*)(piece + 8 * 128)));
                        const s16x8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf), pf, o[db], 0, 0, 0);
                    }
                }
            }
        }
        // the next round's memory-to-LDS loads stay behind this round's LDS reads
        asm volatile("" ::: "memory");
    }

    // ---- the partials meet: wave w's context as [query][feature] over its V space ----
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    {
        float* myO = reinterpret_cast<float*>(myV);
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4_t w4 = {o[db][4 * j], o[db][4 * j + 1], o[db][4 * j + 2], o[db][4 * j + 3]};
                *reinterpret_cast<f32x4_t*>(myO + l32 * OSTRIDE + 32 * db + 8 * j + 4 * g) = w4;
            }
        if (g == 0) { sRef[wave][l32] = run_max; sSum[wave][l32] = run_sum; }
    }
    __syncthreads();
    constexpr int FPT = 32 / NW;                 // features per thread: 8 (16 bytes of bf16) or 4
    constexpr int GQ = 64 / FPT;                 // threads per query
    const int qi = tid / GQ, fg = tid % GQ;
    const int qrow = q0 + qi;
    if (qrow >= qlen || (first_only && qrow != 0)) return;
    const int nw = nblk < NW ? nblk : NW;        // waves that held a key block
    float top = -INFINITY;
    for (int w = 0; w < nw; ++w) top = fmaxf(top, sRef[w][qi]);
    float den = 0.0f, acc[FPT];
#pragma unroll
    for (int e = 0; e < FPT; ++e) acc[e] = 0.0f;
    for (int w = 0; w < nw; ++w) {
        const float wgt = __builtin_amdgcn_exp2f(sRef[w][qi] - top);
        den = fmaf(wgt, sSum[w][qi], den);
        const float* src = reinterpret_cast<const float*>(sW + w * WBYTES) + qi * OSTRIDE + fg * FPT;
#pragma unroll
        for (int e = 0; e < FPT; e += 4) {
            const f32x4_t x4 = *reinterpret_cast<const f32x4_t*>(src + e);
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[e + c] = fmaf(wgt, x4[c], acc[e + c]);
        }
    }
    const float inv = 1.0f / den;
    const size_t hidden = (size_t)heads * 64;
    const size_t row = first_only ? (size_t)b : (cu ? (size_t)cu[b] : (size_t)b * S) + qrow;
    const int kbyte = (h * 64 + fg * FPT) * 2;
    unsigned char* dst = ctx_packed ? ctx + packed_offset((int)row, kbyte, (int)hidden * 2 / 64) : ctx + row * hidden * 2 + kbyte;
#pragma unroll
    for (int e = 0; e < FPT; e += 4) {
        const bf16x4_t w4 = {(__bf16)(acc[e] * inv), (__bf16)(acc[e + 1] * inv), (__bf16)(acc[e + 2] * inv), (__bf16)(acc[e + 3] * inv)};
        *reinterpret_cast<bf16x4_t*>(dst + e * 2) = w4;
    }
}

}  // namespace

bool launch_attention(const void* q, const void* k, const void* vt, const float* maskadd, void* ctx,
                      bool ctx_packed, int B, int heads, int S, int Sp, float scale, int elt, hipStream_t stream,
                      const int* cu, bool v_rowmajor, bool first_only, int variant) {
    const int fo = first_only ? 1 : 0;
    if (variant < kAttnAuto || variant > kAttnSplitKeys || (variant > kAttnPerHead && !(v_rowmajor && elt == kBF16 && S <= 512))) {
        set_error("attention: the key-split variants need bf16 operands, S <= 512 and V as [B, heads, S, 64]");
        return false;
    }
    if (ctx_packed && elt != kBF16) { set_error("attention: only a bf16 context can be packed"); return false; }
    const int cp = ctx_packed ? 1 : 0;
    if (elt != kBF16 && elt != kF32) { set_error("attention: bad operand type"); return false; }
    if (B <= 0 || heads <= 0 || S <= 0) { set_error("attention: empty problem"); return false; }
    if (!(scale > 0.0f)) { set_error("attention: scale must be positive"); return false; }
    if (Sp % 32 != 0 || Sp < S || Sp - S >= 32) {
        set_error("attention: Sp must be S rounded up to a multiple of 32");
        return false;
    }
    if (B > 65535 || heads > 65535) { set_error("attention: grid too large"); return false; }
    if (!q || !k || !vt || !maskadd || !ctx) { set_error("attention: null operand"); return false; }
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(vt) |
         reinterpret_cast<uintptr_t>(maskadd) | reinterpret_cast<uintptr_t>(ctx)) & 15) {
        set_error("attention: operands must be 16-byte aligned");
        return false;
    }
    const unsigned char* qc = static_cast<const unsigned char*>(q);
    const unsigned char* kc = static_cast<const unsigned char*>(k);
    const unsigned char* vc = static_cast<const unsigned char*>(vt);
    unsigned char* cc = static_cast<unsigned char*>(ctx);
    if (elt == kBF16 && S <= 512 && v_rowmajor &&
        (variant == kAttnSplitKeys || (variant == kAttnAuto && (long)B * heads * ((S + 31) / 32) <= kAttnSplitMaxWorkgroups))) {
        const dim3 grid(heads, B, first_only ? 1 : (S + 31) / 32);
        if (grid.z > 65535) { set_error("attention: grid too large"); return false; }
        hipLaunchKernelGGL(attention_split_kernel<4>, grid, dim3(256), 0, stream, qc, kc, vc, maskadd, cc, heads, S, Sp,
                           scale * 1.4426950408889634f, cp, cu, fo);
        CUBERT_HIP_OK(hipGetLastError());
        return true;
    }
    if (elt == kBF16 && S <= 512) {
        const int vstride = round_up(Sp * 2, 256) + 8;
        const size_t lds = (size_t)Sp * 128 + (v_rowmajor ? (size_t)Sp * 128 : 64 * (size_t)vstride) + (size_t)Sp * 4 + 64;
        // More than 64 KiB of dynamic LDS has to be allowed once per device.
        // (Several host threads, one model each, may get here together: the flag is atomic and
        // setting the attribute twice is harmless.)
        static std::atomic<bool> allowed[64];
        int dev = 0;
        CUBERT_HIP_OK(hipGetDevice(&dev));
        if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {
            CUBERT_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_lds_kernel<false>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            CUBERT_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_lds_kernel<true>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);
        }
        if (v_rowmajor)
            hipLaunchKernelGGL(attention_lds_kernel<true>, dim3(heads, B), dim3(2 * Sp), lds, stream, qc, kc, vc, maskadd,
                               cc, heads, S, Sp, vstride, scale * 1.4426950408889634f, cp, cu, fo);
        else
            hipLaunchKernelGGL(attention_lds_kernel<false>, dim3(heads, B), dim3(2 * Sp), lds, stream, qc, kc, vc, maskadd,
                               cc, heads, S, Sp, vstride, scale * 1.4426950408889634f, cp, cu, fo);
        CUBERT_HIP_OK(hipGetLastError());
        return true;
    }
    if (v_rowmajor) { set_error("attention: a row-major V needs bf16 operands and S <= 512"); return false; }
    dim3 grid(first_only ? 1 : (S + 127) / 128, heads, B), block(256);
    if (elt == kBF16)
        hipLaunchKernelGGL(attention_kernel<kBF16>, grid, block, 0, stream, qc, kc, vc, maskadd, cc, heads, S, Sp, scale, cp, cu, fo);
    else
        hipLaunchKernelGGL(attention_kernel<kF32>, grid, block, 0, stream, qc, kc, vc, maskadd, cc, heads, S, Sp, scale, cp, cu, fo);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

}  // namespace cubert
