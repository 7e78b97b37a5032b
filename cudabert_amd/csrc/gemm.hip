// MFMA GEMM for gfx950 (MI355X):  Y = epilogue(X * W^T + bias).
//
// Both operands are K-contiguous ([rows, K]); a workgroup of four wave64s
// computes a BT x BT macro tile (BT features x BT tokens), each wave a
// (BT/2) x (BT/2) quadrant built from 32x32 MFMA blocks.  Per K step a slab of
// 128 bytes per row (64 bf16 / 32 f32) of both operands is loaded straight
// from global memory into LDS (buffer_load ... lds, one barrier per step): two
// LDS stages for the 256 and 128 tiles, four for the 64 tile, whose steps are so
// short that a single step of prefetch leaves every step waiting a full memory
// latency.
//
// LDS image of an operand tile: two sub-blocks (the two 64-byte halves of the
// K slab), each BT rows x 64 bytes; a row is four 16-byte chunks and chunk c
// of row r sits in slot c ^ ((r >> 2) & 3) (packed_swizzle), which spreads the
// 16-byte fragment reads of 8 or 16 consecutive rows over all banks.  This is
// also the on-device "packed" operand layout (common.h): a packed operand is
// stored as 16 KiB blocks of 256 rows x 64 bytes that already are this image,
// so loading a tile is a plain contiguous copy; an unpacked (row-major)
// operand is gathered into the same image by choosing which chunk each lane
// fetches.
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
//
// The 256 tile in bf16 has a hand-scheduled twin (gemm_bf16_256.hip); this
// file is the general kernel (any tile, f32, odd step counts).
#include "gemm_common.h"

namespace cubert {

bool launch_gemm_bf16_t256(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream);
bool launch_gemm_bf16_t256x128(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream);
bool launch_gemm_bf16_t128(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream);
bool launch_gemm_bf16_t256x128_deep(const gemm_detail::GemmDev& d, int out_elt, int epilogue, hipStream_t stream);
int gemm_pick_tile(int M, int N, int K, int elt);
int gemm_ln_pick_tile(int M, int N, int K, int elt);

namespace {

using namespace gemm_detail;

template <int ELT, int OUT, int EPI, int BT, int NS>
__global__ __launch_bounds__(256) void gemm_kernel(const GemmDev p) {
    constexpr int ES = (ELT == kBF16) ? 2 : 4;       // operand element size
    constexpr int NB = BT / 64;                      // 32x32 blocks per wave and dimension
    constexpr int GROUPS = BT / 32;                  // loads each wave issues per operand tile and step
    constexpr int SUB = BT * 64;                     // one sub-block (64-byte half of the K slab)
    constexpr int TILE_BYTES = 2 * SUB;              // one operand tile in LDS
    constexpr int SBDIV = BT / 16;                   // 16-row groups per sub-block
    constexpr int BK = 128 / ES;                     // K elements per step

    // NS = LDS stages: two, or four for the 64 tile of a launch with few workgroups (64 KiB; with
    // many workgroups the four resident ones that two stages allow hide the latency better).
    static_assert(NS == 2 || (NS == 4 && BT == 64), "four stages only fit the 64 tile");
    constexpr int LPT = 2 * GROUPS;                  // loads a wave issues per step
    // s_waitcnt vmcnt(n) with n = the loads of the NS - 2 youngest tiles: the next tile has landed
    constexpr int WAIT_N = LPT * (NS - 2);
    constexpr int WAIT_IMM = 0x0F70 | (WAIT_N & 15) | ((WAIT_N >> 4) << 14);

    // Separate LDS objects (not one array indexed by stage): the compiler
    // then knows that the asynchronous global->LDS loads filling one buffer
    // cannot alias the fragment reads of another and does not serialise them.
    __shared__ __attribute__((aligned(1024))) unsigned char lds0[2 * TILE_BYTES];   // W tile, then X tile
    __shared__ __attribute__((aligned(1024))) unsigned char lds1[2 * TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) unsigned char lds2[NS == 4 ? 2 * TILE_BYTES : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds3[NS == 4 ? 2 * TILE_BYTES : 16];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // wave-uniform: keeps LDS bases scalar
    const int wn = wave >> 1, wm = wave & 1;
    const int l32 = lane & 31, g = lane >> 5;

    int tile_n, tile_m;
    tile_of_block(blockIdx.x, p.tiles_n * p.tiles_m, p.tiles_n, p.xn_parts, &tile_n, &tile_m);
    const int n0 = tile_n * BT, m0 = tile_m * BT;

    // ---- global -> LDS, asynchronous, no registers in between ----
    // One buffer_load ... lds instruction moves 64 lanes x 16 bytes = 16 tile rows
    // of one sub-block to 1 KiB of consecutive LDS (lane l lands at base + 16 l).
    // The wave's i-th load handles load number q = wave + 4 i of the tile:
    // sub-block q / SBDIV, 16-row group q % SBDIV.
    //   unpacked source: lane fetches row 16*group + l/4 and the chunk that belongs
    //     into LDS slot l%4, i.e. chunk (l%4) ^ swz(row); rows outside the matrix
    //     read as zero through the buffer descriptor's bounds check (which covers
    //     the lane offset only, so the row part lives there and just the K offset,
    //     always in range, goes into the scalar offset);
    //   packed source: the 1 KiB is contiguous in memory.
    const int KB = p.K * ES / 64;                    // 64-byte blocks per packed row
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char*>(p.W), 0,
        p.w_packed ? (int)packed_bytes(p.N, p.K * ES) : (int)((size_t)p.N * p.K * ES), 0x00020000);
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char*>(p.X), 0,
        p.x_packed ? (int)packed_bytes(p.M, p.K * ES) : (int)((((size_t)p.M - 1) * p.ldx + p.K) * ES), 0x00020000);
    const int w_rowb = p.K * ES, x_rowb = p.ldx * ES;
    const int dc = (lane & 3) ^ packed_swizzle(lane >> 2);     // row groups start at multiples of 16: only the lane matters
    const int w_base = p.w_packed ? ((n0 >> 8) * KB * 16384 + (n0 & 255) * 64 + wave * 1024 + lane * 16)
                                  : ((n0 + 16 * wave + (lane >> 2)) * w_rowb + (dc << 4));
    const int x_base = p.x_packed ? ((m0 >> 8) * KB * 16384 + (m0 & 255) * 64 + wave * 1024 + lane * 16)
                                  : ((m0 + 16 * wave + (lane >> 2)) * x_rowb + (dc << 4));
    const int w_gs = p.w_packed ? 1024 : 16 * w_rowb, w_ss = p.w_packed ? 16384 : 64;   // group / sub-block strides
    const int x_gs = p.x_packed ? 1024 : 16 * x_rowb, x_ss = p.x_packed ? 16384 : 64;
    const int w_ks = p.w_packed ? 32768 : 128, x_ks = p.x_packed ? 32768 : 128;         // K step strides

    typedef __attribute__((address_space(3))) void* lds_ptr_t;
    // K steps of this workgroup: all of them, or (split K) the blockIdx.y-th share
    const int steps = p.K / BK;
    const int kt0 = (int)((long)steps * blockIdx.y / p.splits);
    const int KT = (int)((long)steps * (blockIdx.y + 1) / p.splits);
    // A K step past the end (odd step counts run one phantom step) fetches from
    // beyond the descriptor's range and therefore fills the tile with zeros: bit 31 of
    // the lane offset puts it past any descriptor (launch_gemm keeps operands below 2 GiB).
#define CUBERT_ISSUE_TILE(BUF, kt)                                                                          \
    do {                                                                                                    \
        const int oob = (kt) < KT ? 0 : (int)0x80000000u;                                                   \
        _Pragma("unroll") for (int i = 0; i < GROUPS; ++i) {                                                \
            const int sb = (4 * i) / SBDIV, gq = (4 * i) % SBDIV;                                       \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                       \
                wres, (lds_ptr_t)((BUF) + sb * SUB + (gq + wave) * 1024), 16,                               \
                (w_base + gq * w_gs + sb * w_ss) | oob, (kt) * w_ks, 0, 0);                                 \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                       \
                xres, (lds_ptr_t)((BUF) + TILE_BYTES + sb * SUB + (gq + wave) * 1024), 16,                  \
                (x_base + gq * x_gs + sb * x_ss) | oob, (kt) * x_ks, 0, 0);                                 \
        }                                                                                                   \
    } while (0)

    // ---- fragment read addressing ----
    // Lane (row l32, group g) of 32x32 block i reads chunk 2*(kk&1) + g of row
    // base + 32 i + l32 in sub-block kk >> 1.  swz(row) only depends on l32 (the
    // quadrant base and 32 i do not reach the bits it uses), so the byte offset is
    //   (off0 ^ ((kk & 1) << 5)) + (kk >> 1) * SUB + i * 2048.
    const int sw = packed_swizzle(l32);
    const int woff0 = (wn * (BT / 2) + l32) * 64 + ((g ^ sw) << 4);
    const int xoff0 = TILE_BYTES + (wm * (BT / 2) + l32) * 64 + ((g ^ sw) << 4);

    f32x16_t acc[NB][NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // With four stages the fragment reads are issued as inline asm on plain LDS byte addresses,
    // and waited for with an explicit lgkmcnt(0) that the fragments pass through ("+v"): a read
    // the compiler can see makes it wait for EVERY outstanding global->LDS load first, which
    // would undo the prefetch distance.  Which tile has landed is tracked by hand with the
    // vmcnt waits at the end of each step.  With two stages every load has landed at the end
    // of a step anyway and the compiler places the reads and their waits itself.
#define CUBERT_LOAD_FRAGS(BUF, kk, WF, XF)                                                                  \
    do {                                                                                                    \
        if constexpr (NS == 4) {                                                                            \
            const int cur = (int)(size_t)(__attribute__((address_space(3))) unsigned char*)(BUF);           \
            _Pragma("unroll") for (int i = 0; i < NB; ++i)                                                  \
                asm volatile("ds_read_b128 %0, %1" : "=v"(WF[i])                                            \
                             : "v"(cur + (wb ^ (((kk) & 1) << 5)) + ((kk) >> 1) * SUB + i * 2048));         \
            _Pragma("unroll") for (int j = 0; j < NB; ++j)                                                  \
                asm volatile("ds_read_b128 %0, %1" : "=v"(XF[j])                                            \
                             : "v"(cur + (xb ^ (((kk) & 1) << 5)) + ((kk) >> 1) * SUB + j * 2048));         \
        } else {                                                                                            \
            _Pragma("unroll") for (int i = 0; i < NB; ++i)                                                  \
                WF[i] = *reinterpret_cast<const u32x4_t*>((BUF) + (wb ^ (((kk) & 1) << 5)) + ((kk) >> 1) * SUB + i * 2048); \
            _Pragma("unroll") for (int j = 0; j < NB; ++j)                                                  \
                XF[j] = *reinterpret_cast<const u32x4_t*>((BUF) + (xb ^ (((kk) & 1) << 5)) + ((kk) >> 1) * SUB + j * 2048); \
        }                                                                                                   \
    } while (0)
#define CUBERT_FENCE_FRAGS(WF, XF)                                                                          \
    do {                                                                                                    \
        if constexpr (NS == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(WF[0]), "+v"(XF[0]));             \
    } while (0)

    // One K step on buffer CUR while the loads of the tile NS - 1 steps ahead fill NEXT
    // (the buffer the previous step computed on; its barrier has released it).
    // The empty asm keeps the compiler from hoisting (and then spilling) every
    // per-k-step address.
#define CUBERT_K_STEP(CUR, NEXT, kt)                                                                        \
    do {                                                                                                    \
        CUBERT_ISSUE_TILE(NEXT, (kt) + NS - 1);                                                             \
        int wb = woff0, xb = xoff0;                                                                         \
        asm volatile("" : "+v"(wb), "+v"(xb));                                                              \
        if constexpr (NS == 4) {                                                                            \
            /* One 32 x 32 block per wave: a k-slice is a single MFMA, too short to hide the next     */    \
            /* slice's fragment read behind it.  All eight reads of the step go out together and each */    \
            /* MFMA waits for its own pair only (LDS reads return in order).                          */    \
            u32x4_t wf[4][NB], xf[4][NB];                                                                   \
            _Pragma("unroll") for (int kk = 0; kk < 4; ++kk) CUBERT_LOAD_FRAGS(CUR, kk, wf[kk], xf[kk]);    \
            asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(wf[0][0]), "+v"(xf[0][0]));                          \
            mfma_chunk<ELT>(wf[0][0], xf[0][0], acc[0][0]);                                                 \
            asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(wf[1][0]), "+v"(xf[1][0]));                          \
            mfma_chunk<ELT>(wf[1][0], xf[1][0], acc[0][0]);                                                 \
            asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(wf[2][0]), "+v"(xf[2][0]));                          \
            mfma_chunk<ELT>(wf[2][0], xf[2][0], acc[0][0]);                                                 \
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wf[3][0]), "+v"(xf[3][0]));                          \
            mfma_chunk<ELT>(wf[3][0], xf[3][0], acc[0][0]);                                                 \
        } else {                                                                                            \
            u32x4_t wf[2][NB], xf[2][NB];                                                                   \
            CUBERT_LOAD_FRAGS(CUR, 0, wf[0], xf[0]);                                                        \
            CUBERT_FENCE_FRAGS(wf[0], xf[0]);                                                               \
            _Pragma("unroll") for (int kk = 0; kk < 4; ++kk) {                                              \
                if (kk < 3) CUBERT_LOAD_FRAGS(CUR, kk + 1, wf[(kk + 1) & 1], xf[(kk + 1) & 1]);             \
                _Pragma("unroll") for (int i = 0; i < NB; ++i)                                              \
                    _Pragma("unroll") for (int j = 0; j < NB; ++j)                                          \
                        mfma_chunk<ELT>(wf[kk & 1][i], xf[kk & 1][j], acc[i][j]);                           \
                if (kk < 3) CUBERT_FENCE_FRAGS(wf[(kk + 1) & 1], xf[(kk + 1) & 1]);                         \
            }                                                                                               \
        }                                                                                                   \
        __builtin_amdgcn_sched_barrier(0);  /* nothing moves across the end of the step */                  \
        __builtin_amdgcn_s_waitcnt(WAIT_IMM); /* my share of the next step's tile has landed */            \
        if constexpr (NS == 4) __builtin_amdgcn_s_barrier(); /* bare: a fenced one waits for all loads */  \
        else __syncthreads();                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                                  \
    } while (0)

    CUBERT_ISSUE_TILE(lds0, kt0);
    if constexpr (NS == 4) {
        CUBERT_ISSUE_TILE(lds1, kt0 + 1);
        CUBERT_ISSUE_TILE(lds2, kt0 + 2);
    }
    // The four-stage kernel runs launches of a few workgroups and a few K steps each, i.e. chains of round trips:
    // what the epilogue adds (bias, first residual rows) is requested now, behind the first tiles.
    constexpr bool SPLITK = (EPI == kEpiBias || EPI == kEpiBiasRes) && OUT == kF32;      // the only combinations launch_gemm splits
    constexpr bool PREFETCH = NS == 4 && BT == 64;
    f32x4_t bias[4 * NB];
    EpiPrefetch<EpiGeometry<OUT, EPI, NB, SPLITK, 4>::PB> pre;
    if constexpr (PREFETCH) {
        if constexpr (gemm_bias_at_readout<OUT, EPI>()) gemm_epilogue_prefetch<OUT, EPI, NB, SPLITK, 4>(p, n0 + wn * (BT / 2), m0 + wm * (BT / 2), l32, g, &pre);
        else gemm_load_bias<NB, SPLITK>(p, n0 + wn * (BT / 2), g, bias);
    }
    __builtin_amdgcn_s_waitcnt(WAIT_IMM);
    if constexpr (NS == 4) __builtin_amdgcn_s_barrier();
    else __syncthreads();
    if constexpr (NS == 4) {
        for (int kt = kt0; kt < KT; kt += 4) {
            CUBERT_K_STEP(lds0, lds3, kt);
            CUBERT_K_STEP(lds1, lds0, kt + 1);
            CUBERT_K_STEP(lds2, lds1, kt + 2);
            CUBERT_K_STEP(lds3, lds2, kt + 3);
        }
        // the zero tiles fetched past the end may still be landing in lds0, the epilogue's staging area
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    } else {
        for (int kt = kt0; kt < KT; kt += 2) {
            CUBERT_K_STEP(lds0, lds1, kt);
            CUBERT_K_STEP(lds1, lds0, kt + 1);
        }
    }
#undef CUBERT_ISSUE_TILE
#undef CUBERT_LOAD_FRAGS
#undef CUBERT_FENCE_FRAGS
#undef CUBERT_K_STEP

    // (the larger tiles fetch their bias here rather than before the loop: no registers to spare there)
    if constexpr (!PREFETCH && !gemm_bias_at_readout<OUT, EPI>()) gemm_load_bias<NB, SPLITK>(p, n0 + wn * (BT / 2), g, bias);
    // every wave is past the last step's barrier: the tiles are dead, lds0 is free for staging
    gemm_epilogue<OUT, EPI, NB, NB, SPLITK, 4, true>(p, acc, bias, n0 + wn * (BT / 2), m0 + wm * (BT / 2), l32, g, lds0 + wave * (BT * 64),
                                                     PREFETCH && gemm_bias_at_readout<OUT, EPI>() ? &pre : nullptr);
}

template <int ELT, int OUT, int EPI, int BT, int NS = 2>
bool launch_one(const GemmDev& d, hipStream_t stream) {
    hipLaunchKernelGGL((gemm_kernel<ELT, OUT, EPI, BT, NS>), dim3(d.tiles_n * d.tiles_m, d.splits), dim3(256), 0, stream, d);
    CUBERT_HIP_OK(hipGetLastError());
    return true;
}

template <int ELT, int OUT, int EPI>
bool launch_tile(const GemmDev& d, int bt, hipStream_t stream) {
    switch (bt) {
        case 64:
            // few workgroups: nothing else on the CU hides the memory latency, so prefetch deeper
            if ((long)d.tiles_n * d.tiles_m * d.splits <= 512) return launch_one<ELT, OUT, EPI, 64, 4>(d, stream);
            return launch_one<ELT, OUT, EPI, 64>(d, stream);
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
        case kEpiQKVMap: return launch_tile<ELT, OUT, kEpiQKVMap>(d, bt, stream);
        case kEpiBiasRes:
            if constexpr (OUT == kF32) return launch_tile<ELT, OUT, kEpiBiasRes>(d, bt, stream);
            break;
    }
    set_error("gemm: unknown epilogue");
    return false;
}

}  // namespace

namespace {
// Workspace of the LayerNorm epilogue: flag words, two counters per band of rows (a fixed number of
// bands, so that launches with different M agree on where the counters are), then (sum, M2 about the slot mean)
// for every row and every 128-feature slot (at most 8).
constexpr size_t kLnMaxBands = 16384;
size_t ln_stats_offset() { return ((gemm_detail::kLnCntFirst + 2 * kLnMaxBands) * sizeof(int) + 255) / 256 * 256; }
}  // namespace

size_t gemm_ln_workspace_bytes(size_t M) { return ln_stats_offset() + ((M + 255) / 256 * 256) * 8 * sizeof(unsigned long long); }

namespace {
bool ln_shape_ok(int N, int K, int elt) { return elt == kBF16 && N > 0 && N % 256 == 0 && N <= 1024 && K % 32 == 0 && K >= 64; }
}  // namespace

bool gemm_ln_workspace_force_expiry(void* ln_ws) {
    if (!ln_ws) { set_error("gemm: null workspace"); return false; }
    const int limit = 1, stuck = -1000000;
    int* w = static_cast<int*>(ln_ws);
    CUBERT_HIP_OK(hipMemcpy(w + 1, &limit, sizeof(int), hipMemcpyHostToDevice));
    CUBERT_HIP_OK(hipMemcpy(w + gemm_detail::kLnCntFirst, &stuck, sizeof(int), hipMemcpyHostToDevice));
    return true;
}

// Tile of a GEMM with the LayerNorm in its epilogue, 0 if the separate kernels are the better choice.
// Measured on MI355X (N = 768 and 1024, K = N and 4 N): from about 6000 rows on the fused kernel beats
// GEMM + LayerNorm launch.  Inside a forward pass (two half-batches on two streams) the 256 x 256 tile wins
// once its tiles cover half of the CUs (152 and 200 tiles: +7 % on the pass over the 256 x 128 tile), below
// that the 256 x 128 tile, two workgroups per CU and half as coarse (96 tiles: +3 %).
int gemm_ln_pick_tile(int M, int N, int K, int elt) {
    if (M < 6144 || !ln_shape_ok(N, K, elt)) return 0;
    const long tiles256 = (long)((M + 255) / 256) * (N / 256);
    return (K % 128 == 0 && tiles256 >= 128) ? 256 : kTile256x128;
}

bool gemm_ln_supported(int M, int N, int K, int elt) { return gemm_ln_pick_tile(M, N, K, elt) != 0; }

int gemm_pick_tile(int M, int N, int K, int elt) {
    auto tiles = [&](int bt) { return (long)((M + bt - 1) / bt) * ((N + bt - 1) / bt); };
    auto rounds = [](long wgs, long slots) { return (double)((wgs + slots - 1) / slots); };
    if (elt != kBF16) {
        // float32 operands: a 128 tile keeps two workgroups on a CU, which the compiler-scheduled
        // loop needs more than the larger tile's operand reuse (measured 20 % faster than 256).
        return tiles(128) >= 512 ? 128 : 64;
    }
    // bf16: estimated time = rounds over the chip x time of one workgroup, with per-step costs
    // measured on MI355X (microseconds): the hand-scheduled 256 tile (one workgroup per CU)
    // 9 + 0.75 per 32 k; the hand-scheduled 256 x 128 tile (two per CU, which overlap instead of
    // running in rounds) 4.5 + 0.98 per 32 k (1.06 for K > 1536, where its shorter prefetch
    // distance shows); the 128 tile (two per CU) 5 + 1.2 per 64 k; the
    // 64 tile (four per CU) 4 + 0.9 per 64 k.
    const double c128 = rounds(tiles(128), 512) * (5.0 + 1.2 * K / 64.0);
    const double c64 = rounds(tiles(64), 1024) * (4.0 + 0.9 * K / 64.0);
    double best = c128;
    int bt = 128;
    if (c64 < best) { best = c64; bt = 64; }
    if (K % 128 == 0) {
        const double c256 = rounds(tiles(256), 256) * (9.0 + 0.75 * K / 32.0);
        if (c256 <= best) { best = c256; bt = 256; }
    }
    {
        const double wgs = (double)((M + 127) / 128) * ((N + 255) / 256);
        const double c384 = (wgs > 512.0 ? wgs / 512.0 : 1.0) * (4.5 + (K > 1536 ? 1.06 : 0.98) * K / 32.0);
        if (c384 < best) bt = kTile256x128;
    }
    return bt;
}

// Tile and split count for a problem (tile as in GemmParams::tile, never 0).  max_splits > 1: the caller can take the
// result as that many partial sums (float32 result, plain bias epilogue; see GemmParams::splits).
//
// Below kPlanSmallRows rows of bf16 operands the launch does not fill the chip for long and what counts is how the
// workgroups spread over the 256 CUs.  Estimated time (microseconds, constants measured on MI355X with launches of
// a few hundred to a few thousand rows of the four linears of BERT-large) = launch + result traffic + T * g, where T is the time of a
// workgroup that has its CU to itself (a constant plus a cost per half-step of 32 k), and g says how the launch
// stretches when a CU gets w > 1 workgroups on average: g = 1 + (w - 1 + q) * rho; rho is what one more workgroup on a CU
// costs relative to a lone one (1: nothing is gained from sharing a CU, the 128 x 128 tile saturates the LDS on its
// own) and q allows for the uneven hand-out of coarse tiles.  From kPlanSmallRows rows on, and for float32 operands,
// gemm_pick_tile decides (its costs were measured inside whole forward passes at the power limit) and K is not split.
constexpr int kPlanSmallRows = 6144;

namespace {
// Best (tile, splits) with min_splits <= splits <= max_splits (powers of two times min_splits).
GemmPlan plan_small(int M, int N, int K, int min_splits, int max_splits, bool f32_result, bool gelu) {
    // launch: before the first workgroup runs; fixed + per_hs * half-steps: a workgroup alone on its CU (deep_k: what a
    // half-step costs more when K > 2048 and the weights stream from memory); rho, q: see above; out: weight of the
    // result traffic (bytes / 4 TB/s).  Least-squares fit (5 % mean error) to launches of the four linears of BERT-large
    // at 400 .. 6400 rows that cycle through 40 weight matrices, so that weights come from memory as in a forward pass.
    struct Cand { int tile, bm, bn; double launch, fixed, per_hs, rho, q, out, deep_k; bool splits, k128; };
    static const Cand cands[] = {
        {64, 64, 64, 2.80, 0.20, 0.129, 0.77, 0.37, 0.01, 0.02, true, false},
        {kTile128Hand, 128, 128, 2.37, 2.81, 0.283, 0.61, 0.16, 0.28, 0.14, true, false},
        {kTile256x128, 128, 256, 8.00, 0.95, 0.260, 1.21, 0.45, 0.86, 0.46, false, false},
        {kTile256x128Deep, 128, 256, 6.25, 1.33, 0.263, 1.50, 0.62, 0.86, 0.43, false, true},
        {256, 256, 256, 8.00, 3.43, 0.448, 1.15, 0.85, 0.97, 0.11, false, true},
    };
    GemmPlan best{64, min_splits};
    double best_cost = 1e30;
    for (const Cand& c : cands) {
        if ((!c.splits && min_splits > 1) || (c.k128 && K % 128 != 0)) continue;
        for (int sp = min_splits; sp <= (c.splits ? max_splits : 1) && sp <= 16; sp *= 2) {
            if (sp > min_splits && K / sp < 128) break;             // at least four half-steps per share
            const double wgs = (double)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn) * sp;
            const double w = wgs / 256.0;
            const double g = w <= 1.0 ? 1.0 : 1.0 + (w - 1.0 + c.q) * c.rho;
            const double T = c.fixed + c.per_hs * (K / 32.0 / sp) * (K > 2048 ? 1.0 + c.deep_k : 1.0) + (sp > 1 ? 0.6 : 0.0) +
                             (gelu ? 0.8 : 0.0);
            const double out_us = (double)M * N * (f32_result ? 4.0 : 2.0) * sp / 4.0e6;
            // the consumer of split results reads every part again
            const double cost = c.launch + c.out * out_us * (sp > 1 ? 1.5 : 1.0) + T * g;
            if (cost < best_cost) { best_cost = cost; best = GemmPlan{c.tile, sp}; }
        }
    }
    return best;
}
}  // namespace

GemmPlan gemm_plan(int M, int N, int K, int elt, int max_splits, bool f32_result, bool gelu) {
    GemmPlan best{gemm_pick_tile(M, N, K, elt), 1};
    if (elt != kBF16 || M >= kPlanSmallRows || K % 64 != 0) {
        if (max_splits > 1) {
            // float32 operands: the rule the short batches were tuned with (64 x 64 tiles, at most 512 workgroups)
            const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64);
            int sp = 1;
            while (sp * 2 <= max_splits && tiles * sp < 512 && K / (sp * 2) >= 256) sp *= 2;
            best.splits = sp;
            if (sp > 1 && best.tile == 256) best.tile = 128;      // the 256 x 256 kernel does not split
        }
        return best;
    }
    return plan_small(M, N, K, 1, max_splits > 1 ? max_splits : 1, f32_result, gelu);
}

bool launch_gemm(const GemmParams& p, hipStream_t stream) {
    const int es = (p.elt == kBF16) ? 2 : 4;
    const int bk = 128 / es;
    if (p.elt != kBF16 && p.elt != kF32) { set_error("gemm: bad operand type"); return false; }
    if (p.M <= 0 || p.N <= 0 || p.K <= 0) { set_error("gemm: empty problem"); return false; }
    if (p.xcd_partition != -1 && p.xcd_partition != 0 && p.xcd_partition != 2 && p.xcd_partition != 4) { set_error("gemm: the XCD partition is 0, 2 or 4"); return false; }
    if (p.K % bk != 0) { set_error("gemm: K must be a multiple of " + std::to_string(bk)); return false; }
    if (p.N % 4 != 0) { set_error("gemm: N must be a multiple of 4"); return false; }
    if (p.out_elt == kBF16 && p.N % 8 != 0) { set_error("gemm: N must be a multiple of 8 for bf16 results"); return false; }
    if (!p.x_packed && (p.ldx < p.K || (p.ldx * es) % 16 != 0)) { set_error("gemm: bad ldx"); return false; }
    if (p.x_packed && p.ldx != p.K) { set_error("gemm: a packed X has no row stride"); return false; }
    if (!p.X || !p.W || !p.bias) { set_error("gemm: null operand"); return false; }
    if (((size_t)p.M + 256) * (p.x_packed ? p.K : p.ldx) * es >= (1ull << 31) ||
        ((size_t)p.N + 256) * p.K * es >= (1ull << 31)) {
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
    d.x_packed = p.x_packed; d.w_packed = p.w_packed; d.y_packed = p.y_packed;
    int out = p.out_elt;
    int epi = (p.epilogue == kEpiQKV && p.rowmap) ? (int)kEpiQKVMap : p.epilogue;
    if (p.epilogue == kEpiQKVMap || p.epilogue == kEpiBiasRes || p.epilogue == kEpiBiasResLN) { set_error("gemm: unknown epilogue"); return false; }
    if (p.residual) {
        if (p.epilogue != kEpiBias || out != kF32 || p.y_packed || p.N % 4 != 0 ||
            (reinterpret_cast<uintptr_t>(p.residual) & 15)) {
            set_error("gemm: a residual needs the plain bias epilogue, a float32 row-major result, N a multiple of 4 and 16-byte alignment");
            return false;
        }
        epi = kEpiBiasRes;
        d.R = p.residual;
    }
    if (p.ln_gamma) {
        if (!p.residual || !p.ln_beta || !p.ln_ws || p.splits > 1 || !ln_shape_ok(p.N, p.K, p.elt) ||
            ((size_t)p.M + 256) * p.N * 4 >= (1ull << 31) || (size_t)(p.M + 127) / 128 > kLnMaxBands ||
            (p.tile ? (p.tile != 256 && p.tile != kTile256x128) || (p.tile == 256 && p.K % 128 != 0)
                    : !gemm_ln_supported(p.M, p.N, p.K, p.elt)) ||
            ((reinterpret_cast<uintptr_t>(p.ln_gamma) | reinterpret_cast<uintptr_t>(p.ln_beta) |
              reinterpret_cast<uintptr_t>(p.ln_xb) | reinterpret_cast<uintptr_t>(p.ln_ws)) & 15)) {
            set_error("gemm: the LayerNorm epilogue needs a residual, bf16 operands, N a multiple of 256 up to 1024, the "
                      "256 or 256x128 tile, no split K, a workspace and 16-byte aligned gamma / beta / copy");
            return false;
        }
        epi = kEpiBiasResLN;
        d.ln_gamma = p.ln_gamma;
        d.ln_beta = p.ln_beta;
        d.ln_xb = static_cast<unsigned char*>(p.ln_xb);
        d.ln_xb_packed = p.ln_xb_packed ? 1 : 0;
        d.ln_bands = (int)kLnMaxBands;
        d.ln_cnt = static_cast<int*>(p.ln_ws);
        d.ln_stats = reinterpret_cast<unsigned long long*>(static_cast<unsigned char*>(p.ln_ws) + ln_stats_offset());
    }
    if (p.epilogue == kEpiQKV) {
        if (!p.q || !p.k || !p.vt || p.S <= 0 || p.heads <= 0 || p.N != 3 * p.heads * 64 ||
            (!p.rowmap && p.M % p.S != 0) || p.Sp < p.S || p.Sp % 4 != 0) {
            set_error("gemm: bad QKV epilogue arguments");
            return false;
        }
        d.q = static_cast<unsigned char*>(p.q);
        d.k = static_cast<unsigned char*>(p.k);
        d.vt = static_cast<unsigned char*>(p.vt);
        d.v_rowmajor = p.v_rowmajor ? 1 : 0;
        d.S = p.S; d.Sp = p.Sp; d.heads = p.heads; d.hidden = p.heads * 64;
        d.rowmap = p.rowmap;
        d.y_packed = 0;
        out = p.elt;
    } else {
        if (!p.Y || (reinterpret_cast<uintptr_t>(p.Y) & 15)) { set_error("gemm: bad Y"); return false; }
        if (out != kBF16 && out != kF32) { set_error("gemm: bad output type"); return false; }
        if (p.y_packed && (out != kBF16 || p.N % 32 != 0)) {
            set_error("gemm: a packed Y must be bf16 with N a multiple of 32");
            return false;
        }
    }
    d.splits = p.splits > 0 ? p.splits : 1;
    if (d.splits > 1) {
        if ((epi != kEpiBias && epi != kEpiBiasRes) || out != kF32 || p.y_packed || d.splits > p.K / bk) {
            set_error("gemm: split K needs the plain bias epilogue, a float32 result and at least one K step per split");
            return false;
        }
    }
    int bt = p.tile;
    if (!bt) {
        // the caller has settled on the split count; the tile follows
        if (p.elt == kBF16 && p.M < kPlanSmallRows && p.K % 64 == 0)
            bt = plan_small(p.M, p.N, p.K, d.splits, d.splits, out == kF32, epi == kEpiBiasGelu).tile;
        else
            bt = gemm_pick_tile(p.M, p.N, p.K, p.elt);
    }
    if (epi == kEpiBiasResLN && !p.tile) bt = gemm_ln_pick_tile(p.M, p.N, p.K, p.elt);
    if (d.splits > 1 && (bt == 256 || bt == kTile256x128 || bt == kTile256x128Deep) && !p.tile) bt = 128;      // those kernels do not split
    if (epi == kEpiBiasResLN && p.compiler_scheduled) { set_error("gemm: the LayerNorm epilogue has no compiler-scheduled kernel"); return false; }
    if (bt == kTile256x128 || bt == kTile256x128Deep) {
        if (p.elt != kBF16 || d.splits != 1) { set_error("gemm: the 256x128 tile is bf16 only and does not split K"); return false; }
        d.tiles_n = (p.N + 255) / 256;
        d.tiles_m = (p.M + 127) / 128;
        d.xn_parts = gemm_pick_partition((double)p.M * p.K * es, (double)p.N * p.K * es, d.tiles_n, d.tiles_m, 8);
        if (p.xcd_partition >= 0) d.xn_parts = p.xcd_partition;
        if (bt == kTile256x128Deep) {
            if (epi == kEpiBiasResLN) { set_error("gemm: the one-per-CU 256x128 tile has no LayerNorm epilogue"); return false; }
            return launch_gemm_bf16_t256x128_deep(d, out, epi, stream);
        }
        return launch_gemm_bf16_t256x128(d, out, epi, stream);
    }
    if (bt == kTile128Hand) {
        if (p.elt != kBF16) { set_error("gemm: the hand-scheduled 128 tile is bf16 only"); return false; }
        d.tiles_n = (p.N + 127) / 128;
        d.tiles_m = (p.M + 127) / 128;
        d.xn_parts = gemm_pick_partition((double)p.M * p.K * es, (double)p.N * p.K * es, d.tiles_n, d.tiles_m, 8);
        if (p.xcd_partition >= 0) d.xn_parts = p.xcd_partition;
        return launch_gemm_bf16_t128(d, out, epi, stream);
    }
    d.tiles_n = (p.N + bt - 1) / bt;
    d.tiles_m = (p.M + bt - 1) / bt;
    d.xn_parts = gemm_pick_partition((double)p.M * p.K * es, (double)p.N * p.K * es, d.tiles_n, d.tiles_m, 4);
    if (p.xcd_partition >= 0) d.xn_parts = p.xcd_partition;
    if (p.elt == kBF16) {
        // 256 tile with a multiple of four half-steps: the hand-scheduled kernel
        if (bt == 256 && p.K % 128 == 0 && !p.compiler_scheduled && d.splits == 1)
            return launch_gemm_bf16_t256(d, out, epi, stream);
        return out == kBF16 ? launch_epi<kBF16, kBF16>(d, epi, bt, stream)
                            : launch_epi<kBF16, kF32>(d, epi, bt, stream);
    }
    if (out != kF32) { set_error("gemm: f32 operands require f32 output"); return false; }
    return launch_epi<kF32, kF32>(d, epi, bt, stream);
}

}  // namespace cubert
