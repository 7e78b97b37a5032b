// Host-callable launchers for the gfx950 kernels.  Every launcher validates
// the operand shapes its kernel and grid assume before launching and returns
// false (with the error text set) instead of launching on a mismatch.
//
// Element types: `elt` selects the GEMM/attention operand type of a tensor --
// 0 = float32, 1 = bfloat16 (stored as uint16).  Accumulation, LayerNorm and
// softmax statistics are always float32.
#pragma once
#include "common.h"

namespace cubert {

// ---------------------------------------------------------------- GEMM -----
// Y[m, n] = epilogue( sum_k X[m, k] * W[n, k] + bias[n] )
//   X: [M, K] row-major with row stride ldx (elements), operand type `elt`
//   W: [N, K] row-major (the on-disk [in,out] kernel transposed at load time)
//   K must be a multiple of 128 bytes worth of elements (64 bf16 / 32 f32).
// Replaces the cuBLAS calls + bias broadcast-fill of the reference
// (cuda_bert/ops/linear.cu:91-148, 241-319; ops/matmul.cu:3-99).
enum GemmEpilogue : int {
    kEpiBias = 0,      // Y = acc + bias
    kEpiBiasGelu = 1,  // Y = gelu_erf(acc + bias)       (ops/elementwise.cu:37-42 fused)
    kEpiBiasTanh = 2,  // Y = tanh(acc + bias)           (ops/elementwise.cu:56-61 fused)
    kEpiQKV = 3,       // scatter into per-head Q, K and transposed V (see below)
    kEpiQKVMap = 4,    // the same on compact rows: row m is token rowmap[m] (chosen by launch_gemm when rowmap is set)
    kEpiBiasRes = 5,   // Y = acc + bias + R, float32 row-major (chosen by launch_gemm when residual is set)
    kEpiBiasResLN = 6, // Y = LayerNorm(acc + bias + R) (chosen by launch_gemm when ln_gamma is set)
};

// Unpadded ("compact") rows: only the valid tokens of every sequence are stored,
// sequence after sequence.  rowmap[r] = b * S + s of compact row r; cu[b] = first
// compact row of sequence b, cu[B] = number of rows.  Both live in device memory.
struct Compact {
    const int* rowmap = nullptr;
    const int* cu = nullptr;
    int rows = 0;
};

constexpr int kTile256x128 = 384;     // GemmParams::tile value of the 256 features x 128 tokens kernel
constexpr int kTile256x128Deep = 385; // ... of the 256 x 128 kernel with one workgroup per CU and the deeper pipeline (K % 128 == 0)
constexpr int kTile128Hand = 192;     // ... of the hand-scheduled 128 x 128 kernel (bf16, three workgroups per CU, splits K)

struct GemmParams {
    const void* X = nullptr;
    const void* W = nullptr;
    const float* bias = nullptr;
    void* Y = nullptr;        // [M, N] row-major, type out_elt (unused for kEpiQKV)
    int M = 0, N = 0, K = 0;
    int ldx = 0;              // row stride of X in elements (>= K)
    int elt = kBF16;          // operand type of X and W
    int out_elt = kBF16;      // type of Y
    int epilogue = kEpiBias;
    // kEpiQKV: N == 3*hidden.  Feature n -> (which = n / hidden, head, dd).
    // Token m -> (b = m / S, s = m % S).  Outputs, all of operand type `elt`:
    //   q  [B, heads, S, 64]      k  [B, heads, S, 64]     vt [B, heads, 64, Sp]
    void* q = nullptr;
    void* k = nullptr;
    void* vt = nullptr;
    bool v_rowmajor = false;  // kEpiQKV: V leaves like q and k, [B, heads, S, 64], instead of transposed (bf16 attention with S <= 512 transposes on its LDS reads)
    int S = 0, Sp = 0, heads = 0;
    const int* rowmap = nullptr;   // kEpiQKV on compact rows: row m is token rowmap[m] = b * S + s
    // kEpiBias with a float32 row-major Y: [M, N] float32 added to the result (the residual branch of
    // the layer, so that the LayerNorm after it reads one operand).  With split K it goes into partial 0.
    const float* residual = nullptr;
    // kEpiBias with a residual and ln_gamma set: the LayerNorm that follows the linear runs in the
    // epilogue.  Y (float32 row-major, may be the residual buffer itself) receives
    // LayerNorm(acc + bias + R) * gamma + beta over each row of N features, ln_xb (optional) a bf16
    // copy of it (row-major, or packed with ln_xb_packed).  bf16 operands, the 256 x 256 or 256 x 128
    // tile, N a multiple of 256 up to 1024, no split K.  The N / 256 workgroups that hold one band
    // of rows exchange their partial row sums through ln_ws: gemm_ln_workspace_bytes(M) bytes of
    // device memory that are all zero before the first launch (each launch leaves the words it
    // counts with at zero again), used by one launch at a time.
    const float* ln_gamma = nullptr;
    const float* ln_beta = nullptr;
    void* ln_xb = nullptr;
    bool ln_xb_packed = false;
    void* ln_ws = nullptr;
    int tile = 0;             // 0 = choose; otherwise 64, 128 or 256 (square macro tile), kTile256x128 or kTile128Hand
    // Split K (kEpiBias, float32 Y): `splits` workgroups share a tile, each reduces its share of K and
    // writes its partial result to Y + z * M * N; the bias goes into partial 0.  The consumer adds
    // them up (launch_add_layernorm's y_parts).  Y must hold splits * M * N floats.
    int splits = 1;
    bool compiler_scheduled = false;   // 256 tile: use the generic kernel, not the hand-scheduled one
    // Packed operand layout (common.h): X / W read from it, Y (bf16, plain epilogues) written in it.
    bool x_packed = false, w_packed = false, y_packed = false;
    int xcd_partition = -1;   // how the eight XCDs divide the tile grid (see tile_of_block): -1 = estimate and choose, 0 = contiguous
                              // runs of the tile sequence, 2 / 4 = 4 x 2 / 2 x 4 cells (for measurements)
};
bool launch_gemm(const GemmParams& p, hipStream_t stream);
// The tile (a GemmParams::tile value, never 0) and split count launch_gemm's cost model prefers for a problem.
// max_splits > 1: the caller can take a float32 result as up to that many partial sums (a power of two is chosen).
// f32_result / gelu: the launch will write float32 / use the GELU epilogue.
struct GemmPlan { int tile; int splits; };
GemmPlan gemm_plan(int M, int N, int K, int elt, int max_splits, bool f32_result, bool gelu);
// Workspace of a GEMM with the LayerNorm in its epilogue (GemmParams::ln_ws) for up to M rows.
size_t gemm_ln_workspace_bytes(size_t M);
// Test aid: puts a workspace into a state in which the workgroups of row band 0 can never see their band complete
// (arrival counter far below zero) and give up after a single poll, so that the bounded wait expires -- every kernel
// still runs to its end -- and the error word gets raised.  Synchronous.
bool gemm_ln_workspace_force_expiry(void* ln_ws);
// True if launch_gemm can run the LayerNorm of a [M, N] float32 result in the epilogue of a
// bf16 GEMM with reduction length K.
bool gemm_ln_supported(int M, int N, int K, int elt);

// ----------------------------------------------------------- attention -----
// Fused QK^T * scale + mask -> softmax -> P V for head dim 64.
//   q, k [B, heads, S, 64], vt [B, heads, 64, Sp], maskadd [B, Sp] float
//   (0 valid, -10000 masked, -inf for the padding columns S..Sp-1),
//   ctx [B*S, heads*64] of type `elt`.
// Replaces Query_Key / op_SoftMax / Prob_Value of the reference
// (cuda_bert/ops/batch_matmul.cu:48-83,107-141; ops/softmax.cu:86-143)
// without materialising the [B,S,heads,S] score tensor.
// ctx_packed (bf16 only): write ctx in the packed GEMM-operand layout (common.h).
bool launch_attention(const void* q, const void* k, const void* vt, const float* maskadd,
                      void* ctx, bool ctx_packed, int B, int heads, int S, int Sp, float scale, int elt,
                      hipStream_t stream, const int* cu = nullptr, bool v_rowmajor = false, bool first_only = false,
                      int variant = kAttnAuto);
// v_rowmajor (bf16, S <= 512 only): `vt` holds V as [B, heads, S, 64] like k.
// variant (v_rowmajor only): kAttnPerHead = one workgroup per (batch, head); kAttnSplitKeys = one workgroup per
// (batch, head, 32 queries) whose four waves share the keys: the short-batch kernel; kAttnAuto picks by the number of such workgroups.
// The variants agree to the last bit or two of the bf16 context, not bit for bit.
// first_only: only the context of every sequence's first token is produced, as row b of ctx [B, heads*64] (same bits
// as row b * S of the full result).

// ----------------------------------------------------------- LayerNorm -----
// x <- LayerNorm(x + y) * gamma + beta   over rows of length H, in place on the
// float32 residual stream x; when xb != nullptr a bf16 copy of the result is
// written as the next GEMM's operand.  y has type y_elt (may be nullptr: plain
// LayerNorm).  eps = 1e-12 inside the square root, biased variance
// (cuda_bert/ops/layernorm.cu:136-182; modeling.py:168-172).
// xb_packed: write the copy in the packed GEMM-operand layout (common.h).
// add_x = false: x <- LayerNorm(y): y is already the sum with the residual stream (a GEMM with
// GemmParams::residual produced it) and x is only written.
bool launch_add_layernorm(float* x, const void* y, int y_elt, const float* gamma,
                          const float* beta, bf16_t* xb, bool xb_packed, int rows, int H,
                          hipStream_t stream, int y_parts = 1, bool add_x = true);

// --------------------------------------------------- embedding + LN --------
// x[t] = LayerNorm(word[ids[t]] + pos[t % S] + type[seg[t]]); also writes the
// additive attention mask row maskadd[b, 0..Sp) (see launch_attention).  mask
// may be nullptr (all positions valid).  ids/seg are clamped into range.
// (cuda_bert/ops/embedding.cu:3-58; utils/bert.cu:94-97 for the positions.)
bool launch_embed_layernorm(const int* ids, const int* seg, const int* mask, const float* word,
                            const float* pos, const float* type, const float* gamma,
                            const float* beta, float* x, bf16_t* xb, bool xb_packed, float* maskadd,
                            int B, int S, int Sp, int H, int vocab, int type_vocab, hipStream_t stream,
                            const Compact* compact = nullptr);

// ------------------------------------------------ scale+mask+softmax -------
// In place over materialised scores [B, rows_per_batch, S] (float32 or bf16):
// p = softmax(scores * scale + (1 - mask[b, :]) * -10000) along the last axis.
// Stand-alone counterpart of cuApplySoftmax (cuda_bert/ops/softmax.cu:86-143).
bool launch_mask_softmax(void* scores, int elt, const int* mask, int B, int rows_per_batch, int S,
                         float scale, hipStream_t stream);

// ------------------------------------------------------ classifier ---------
// probs[b, :] = softmax(pooled[b, :] @ kernel[H, C] + bias[C]), C <= 8
// (apps/finetune.py:16-24; the commented-out Cuda_Classify, cuda_bert.cu:72-89).
bool launch_classifier(const float* pooled, const float* kernel, const float* bias, float* probs,
                       int B, int H, int C, hipStream_t stream);

// ------------------------------------------------------------ pooler -------
// pooled[b, :] = tanh(x[b * S, :] @ W^T + bias): first-token gather + dense +
// tanh in one kernel; x is the float32 sequence output [B*S, H], W [H, H]
// row-major ([out, in]) of type w_elt (cuda_bert/ops/elementwise.cu:5-32, 56-70 and
// the pooler op_Linear of cuda_bert/utils/bert.cu:238-247; modeling.py:347-353).
bool launch_pooler(const float* x, const void* W, int w_elt, const float* bias, float* pooled, int B, int S, int H,
                   hipStream_t stream, const int* cu = nullptr);

// out[b, :] = x[first row of sequence b, :] (row b * S, or cu[b] on compact rows): the residual rows of a last
// layer that is only computed for the first tokens.
bool launch_gather_first_rows(const float* x, const int* cu, float* out, int B, int S, int H, hipStream_t stream);

// Compact rows -> padded [B, S, H] float32 (zeros on the positions past a sequence's length).
bool launch_unpad_rows(const float* xc, const int* cu, float* out, int B, int S, int H, hipStream_t stream);

// ------------------------------------------------------ load helpers -------
// dst[n, k] = convert(src[k, n])  : on-disk [in,out] float32 -> [out,in] operand type,
// row-major or (bf16) packed; in the packed case dst is the whole operand and the
// tensor's rows land at row0 .. row0 + N - 1 of it.
bool launch_transpose_convert(const float* src, void* dst, int K, int N, int elt, bool packed, int row0,
                              hipStream_t stream);
bool launch_fill_f32(float* dst, float value, size_t n, hipStream_t stream);

// Looks up, for the current device, the address of the scratch array of the allocation-free
// split-K GEMM (cubert_op_gemm_splitk_noalloc), so that later calls need no symbol lookup.
bool noalloc_setup_current_device();

}  // namespace cubert
