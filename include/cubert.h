/* C ABI of libcudaBERT.so, the MI355X (gfx950) BERT encoder inference engine.
 *
 * The first five entry points are exactly what the reference's ctypes binding
 * loads (cuda_bert/pybert.py:12-38) and what cuda_model.py's Cuda_BERT calls;
 * they keep the reference's names, argument order and meaning
 * (cuda_bert/cuda_bert.cu:24-181).  Everything after them is additive.
 *
 * All `int*` inputs are C-contiguous int32 [batchsize, seq_length].  A model
 * handle is not thread-safe (as in the reference); use one per host thread.
 */
#ifndef CUBERT_H_
#define CUBERT_H_

#include <stdbool.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------
 * Reference-compatible entry points
 * ---------------------------------------------------------------------- */

/* Device pointers returned by Cuda_Inference (cuda_bert/utils/common.h:173-177):
 * tensor = sequence output [B, S, hidden] float32, pooled_output = [B, hidden]
 * float32.  Valid until the next call on the same model. */
typedef struct Retval {
    float* tensor;
    float* pooled_output;
} Retval;

/* Replaces init_model (cuda_bert/cuda_bert.cu:26-33).  `large` selects
 * BERT-large (24 x 1024 x 16 heads x 4096) or BERT-base (12 x 768 x 12 x 3072)
 * as in cuda_bert/utils/manager.cu:8-15; `num_gpu` is the device ordinal;
 * (max_batchsize, max_seq_length) size the activation memory, (0, 0) gives the
 * reference's default capacity of 200*512 tokens; `dir` is the .npy weight
 * directory ("" -> model_npy/base_uncased or model_npy/large_uncased).
 * Precision and graph use come from the environment: CUBERT_PRECISION=fp32
 * (default) | bf16, CUBERT_GRAPH_MAX_TOKENS (default 8192, 0 disables graphs).
 * fp32 mode agrees with the reference model to 1e-3 max-abs.  bf16 mode stores
 * the Linear kernels and the GEMM operands in bfloat16 (fp32 accumulation,
 * residual stream, statistics and softmax): against the float32 model on the
 * same checkpoint it is within 3e-2 on both outputs when the checkpoint's
 * Linear kernels are bfloat16-representable, and for the 12-layer model in
 * any case; on a 24-layer checkpoint that is not, the [B,S,H] sequence output
 * is within about 4e-2 (pooled output 2e-2), of which 0.026-0.035 is the
 * storage rounding of the weights alone, whatever computes on them.
 * Returns NULL on failure (the reference exits the process); the reason is
 * available from cubert_last_error(). */
void* init_model(bool large, int num_gpu, int max_batchsize, int max_seq_length, char* dir);

/* Replaces release_model (cuda_bert/cuda_bert.cu:34-37). */
void release_model(void* model);

/* Replaces Cuda_Bert (cuda_bert/cuda_bert.cu:55-70): runs the encoder on host
 * inputs and writes batchsize*hidden float32 pooled outputs to the host buffer
 * `output`; synchronous.  attention_mask may be NULL (no masking).  On an
 * invalid call (shape over capacity, id out of range, device failure) it
 * prints the reason to stderr and terminates the process with
 * exit(EXIT_FAILURE), which is what the reference does through its asserts
 * and checkCudaErrors (cuda_bert/utils/manager.cu:100-108, common.h:58-65).
 * Callers that want an error code use cubert_encode instead.
 * Since the caller receives only [B, hidden], the last encoder layer is computed for the first token of every
 * sequence only (keys and values still of every token): the pooled output has the bits of the full pass, the
 * device-side sequence buffer (cubert_seq_ptr) is not defined after such a call.  The same holds for
 * Cuda_Classify and cubert_encode with seq_out == NULL; CUBERT_FIRST_TOKEN_LAST_LAYER=0 at init turns it off. */
void Cuda_Bert(void* model, float* output, int* words, int* token_types, int batchsize,
               int seq_length, int* attention_mask);

/* Replaces Cuda_Inference (cuda_bert/cuda_bert.cu:40-53): same forward pass,
 * asynchronous, returns device pointers.  Call cubert_sync (or any later
 * synchronous entry point) before reading them from another stream. */
Retval Cuda_Inference(void* model, int* words, int* token_types, int batchsize, int seq_length,
                      int* masks);

/* The entry point the reference left commented out (cuda_bert/cuda_bert.cu:72-89; its binding
 * cuda_bert/pybert.py:40-42): encoder + classifier head, batchsize*num_classes float32
 * probabilities softmax(pooled @ classifier_kernel + bias) to the host buffer `output`
 * (the head of apps/finetune.py:16-44, which keeps the last column).  Needs
 * classifier_kernel.npy / classifier_bias.npy in the weight directory; num_classes must
 * match them.  Synchronous; terminates the process on an invalid call like Cuda_Bert. */
void Cuda_Classify(void* model, float* output, int* words, int* token_types, int batchsize,
                   int seq_length, int num_classes, int* attention_mask);

/* Replaces test (cuda_bert/cuda_bert.cu:91-180; cuda_bert.cuh:4-5): loads the
 * default weight directory, tiles the reference's 11-token seed input to
 * (batchsize, seq_length), runs 10 warm-up and nIter timed iterations of
 * forward + pooled-output copy and prints the 99th-percentile latency and the
 * throughput in batches per second. */
void test(int batchsize, int seq_length, int nIter, bool large, int num_gpu);

/* ------------------------------------------------------------------------
 * Additive entry points (no counterpart in the reference unless noted)
 * ---------------------------------------------------------------------- */

/* Text of the last error raised on the calling thread ("" if none). */
const char* cubert_last_error(void);

typedef struct cubert_config {
    int hidden, layers, heads, intermediate; /* head dim (hidden/heads) must be 64 */
    int precision;                           /* 0 = float32, 1 = bfloat16 operands / float32 accumulate */
    int graph_max_tokens;                    /* hipGraph replay for batches up to this many tokens; 0 = off */
} cubert_config;

/* init_model with explicit dimensions and precision. */
void* init_model_ex(const cubert_config* cfg, int num_gpu, int max_batchsize, int max_seq_length,
                    const char* dir);

/* Host-only validation of a weight directory against cfg (names, dtypes,
 * shapes); touches no GPU.  Returns 0 if init_model_ex would accept it. */
int cubert_check_weight_dir(const cubert_config* cfg, const char* dir);

/* Cuda_Bert with an error code instead of process exit.  Any of pooled_out
 * [B, hidden], seq_out [B, S, hidden] and cls_out [B, num_classes] may be NULL.
 * cls_out is the fine-tune head softmax(pooled @ classifier_kernel + bias) --
 * the reference's commented-out Cuda_Classify (cuda_bert/cuda_bert.cu:72-89)
 * and apps/finetune.py:16-44 run on the device.  Returns 0 on success. */
int cubert_encode(void* model, const int* words, const int* token_types, const int* attention_mask,
                  int batchsize, int seq_length, float* pooled_out, float* seq_out, float* cls_out);

/* Forward pass on inputs that already live in device memory; asynchronous on
 * the model's stream.  Returns 0 on success. */
int cubert_forward_device(void* model, const int* d_words, const int* d_token_types,
                          const int* d_attention_mask, int batchsize, int seq_length);
int cubert_sync(void* model);

/* Unpadded forward pass (goes beyond the reference, which pads every batch to its
 * longest line, utils.py:3-13): only the first lengths[b] (1..seq_length) tokens of
 * every sequence are computed, as if the attention mask were 1 on exactly those.
 * d_words / d_token_types are device [B, S] as above; `lengths` is HOST memory [B].
 * The pooled output and the sequence output on the valid positions are bit-identical
 * to cubert_forward_device with the corresponding prefix mask; the sequence output is
 * zero on the padding positions (the padded pass computes values there that no caller
 * uses).  The host-input entry points take this path by themselves when every mask row
 * is a non-empty prefix of ones and
 *   CUBERT_VARLEN=1:      always (Cuda_Bert, Cuda_Classify, Cuda_Inference, cubert_encode);
 *   CUBERT_VARLEN unset:  only for calls that return no sequence output (Cuda_Bert,
 *                         Cuda_Classify, cubert_encode with seq_out == NULL), on batches above
 *                         the hipGraph limit with at least 5 % padding -- the results such a
 *                         call returns are bit-identical either way;
 *   CUBERT_VARLEN=0:      never.
 * Returns 0 on success. */
int cubert_forward_device_lens(void* model, const int* d_words, const int* d_token_types,
                               const int* lengths, int batchsize, int seq_length);

/* Enqueues the fine-tune head on the pooled output of the last forward pass
 * (softmax(pooled @ classifier_kernel + bias), apps/finetune.py:16-44; the
 * reference's commented-out classify_inference, cuda_bert/utils/bert.cu:254-265).
 * Result: cubert_cls_ptr, device [B, num_classes] float32. */
int cubert_classify(void* model);
float* cubert_cls_ptr(void* model);

/* One eager forward pass on device inputs with a hipEvent before every kernel;
 * phase_ms[8] receives milliseconds summed per phase in the order: embedding,
 * QKV GEMM, attention, attention-output GEMM, residual+LayerNorm (both per
 * layer), FFN-in GEMM, FFN-out GEMM, pooler.  Synchronous. */
int cubert_profile_device(void* model, const int* d_words, const int* d_token_types,
                          const int* d_attention_mask, int batchsize, int seq_length, float* phase_ms);

/* Introspection. */
float* cubert_seq_ptr(void* model);       /* device, [B, S, hidden] float32 */
float* cubert_pooled_ptr(void* model);    /* device, [B, hidden] float32 */
void* cubert_stream(void* model);         /* hipStream_t the model enqueues on */
int cubert_hidden_size(void* model);
int cubert_num_classes(void* model);
int cubert_precision(void* model);
int cubert_graphs_cached(void* model);
/* How often a pass of this model was repeated with the LayerNorms as kernels of their own.  The bf16 GEMMs before the
 * LayerNorms of large batches normalise in their epilogue: the workgroups that share a row wait for each other, for a
 * bounded time.  If that wait ever expires (the chip shared with another process in a way that keeps partners from being
 * resident together), the next synchronising call notices, repeats the pass from the inputs still on the device with
 * separate LayerNorm kernels -- the results are the same bits -- keeps this model on those kernels, and counts it here.
 * No reference counterpart: cuda_bert/ops/layernorm.cu:136-206 is always a kernel of its own.
 * (CUBERT_FUSE_LAYERNORM=0 at init never fuses.) */
int cubert_ln_fallbacks(void* model);
/* Test aid for the above: leaves the model's LayerNorm-epilogue workspaces in a state in which the next pass that uses
 * them cannot see row band 0 complete and gives up after one poll.  Every kernel still runs to its end.  Returns 0. */
int cubert_debug_force_ln_timeout(void* model);
long cubert_capacity_tokens(void* model);

/* ---- single kernels on caller-owned device memory (parity tests, roofline
 * timing).  `stream` is a hipStream_t (NULL = default stream); elt: 0 float32,
 * 1 bfloat16.  All return 0 on success. ---- */

/* Layout flags of the GEMM entry points.  A "packed" operand is stored as
 * 16 KiB blocks of 256 rows x 64 bytes in the order the kernels' LDS tiles use
 * (cubert_packed_bytes / cubert_packed_offset give size and element address);
 * in bf16 mode the engine keeps weights and GEMM-input activations this way. */
#define CUBERT_X_PACKED 1           /* activation operand X is packed */
#define CUBERT_W_PACKED 2           /* weight operand W is packed */
#define CUBERT_Y_PACKED 4           /* write Y packed (bf16 output only) */
#define CUBERT_COMPILER_SCHEDULED 8 /* 256 tile: general kernel instead of the hand-scheduled one */
#define CUBERT_LN_NO_RESIDUAL 16    /* cubert_op_add_layernorm: y already contains the residual stream */
#define CUBERT_V_ROWMAJOR 32        /* cubert_op_gemm_qkv / cubert_op_attention (bf16, S <= 512): the `vt` argument holds V as
                                       [B, heads, S, 64] like k instead of transposed */
/* cubert_op_attention with CUBERT_V_ROWMAJOR: which kernel.  0 (no flag) = by batch size; 1 = one workgroup per
 * (batch, head); 2 = one workgroup per (batch, head, 32 queries) whose four waves share the keys (short batches). */
#define CUBERT_ATTN_VARIANT(n) (((n) & 3) << 20)
/* Split K (cubert_op_gemm, epilogue 0, float32 Y): n workgroups share a tile, each reduces 1/n of K
 * and writes its partial sum to Y + i * M * N (the bias is in partial 0); Y holds n * M * N floats and
 * the consumer adds the parts (cubert_op_add_layernorm takes the count in the same flag bits). */
/* For measurements: how the eight XCDs (each with its own L2) divide the tile grid of a GEMM: n = 0 contiguous runs of the
 * tile sequence (an XCD owns a band of token rows), 2 or 4: a 4 x 2 / 2 x 4 partition (an XCD keeps half / a quarter of the
 * weight rows).  Without the flag the library estimates the traffic of each and takes the smallest. */
#define CUBERT_XCD_PARTITION(n) ((((n) + 1) & 0xf) << 16)
#define CUBERT_SPLITS(n) (((n) & 0xff) << 8)
#define CUBERT_SPLITS_OF(flags) (((flags) >> 8) & 0xff)
size_t cubert_packed_bytes(size_t rows, size_t row_bytes);
size_t cubert_packed_offset(int row, int byte_in_row, int row_bytes);

/* Y[M,N] = epilogue(X[M,K] (row stride ldx) * W[N,K]^T + bias[N]);
 * epilogue 0 bias, 1 bias+GELU(erf), 2 bias+tanh.  tile 0 = automatic.
 * Replaces op_Linear::forward (cuda_bert/ops/linear.cu:91-148) + op_Gelu /
 * op_Tanh (ops/elementwise.cu:37-70). */
int cubert_op_gemm(const void* X, const void* W, const float* bias, void* Y, int M, int N, int K,
                   int ldx, int elt, int out_elt, int epilogue, int tile, int flags, void* stream);

/* Y[M,N] (float32) = X * W^T + bias + R[M,N] (float32): the linear before a LayerNorm with the
 * residual add of cuApplyLayerNorm (cuda_bert/ops/layernorm.cu:152-158) moved into its epilogue.
 * With CUBERT_SPLITS(n) the residual and the bias are in partial 0. */
int cubert_op_gemm_residual(const void* X, const void* W, const float* bias, const float* R, float* Y,
                            int M, int N, int K, int ldx, int elt, int tile, int flags, void* stream);

/* The same linear with the LayerNorm that follows it in the epilogue as well (cuApplyLayerNorm,
 * cuda_bert/ops/layernorm.cu:136-206, after op_Linear::forward, ops/linear.cu:91-148):
 *   Y[M,N] (float32, may be R itself) = LayerNorm(X * W^T + bias + R) * gamma + beta   per row,
 * eps 1e-12 inside the square root, biased variance; xb (optional) receives a bf16 copy of Y, row-major
 * or (CUBERT_Y_PACKED) in the packed operand layout.  bf16 operands, tile 256 or 384 (0 = automatic,
 * which needs a problem large enough for one of them), N a multiple of 256 up to 1024, no split K.
 * The N / 256 workgroups that hold the same rows exchange partial row sums through `workspace`:
 * cubert_gemm_layernorm_workspace_bytes(M) bytes of device memory, all zero before the first launch
 * (a launch leaves it ready for the next one), used by one launch at a time.  A workgroup that waits
 * for its partners longer than a bounded number of polls gives up and sets the first int of the
 * workspace to 1 (the second int, if positive, replaces the built-in poll limit). */
size_t cubert_gemm_layernorm_workspace_bytes(int M);
int cubert_op_gemm_residual_layernorm(const void* X, const void* W, const float* bias, const float* R,
                                      const float* gamma, const float* beta, float* Y, void* xb, void* workspace,
                                      int M, int N, int K, int ldx, int tile, int flags, void* stream);

/* Allocation-free split-K GEMM.  No counterpart in the reference: it is for callers that cannot
 * allocate device memory -- code under hipGraph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Y[M,N] (float32) = X * W^T + bias, K shared by `splits` (1..16) workgroups per tile,
 * i.e. cubert_op_gemm with epilogue 0, a float32 Y and CUBERT_SPLITS(splits), except that the partial
 * sums live in a device array built into the library (cubert_noalloc_scratch_bytes() = 16 MiB per GPU,
 * held until the process ends) and are added up on the device, part 0 first: Y holds M*N floats.
 * The call makes no hipMalloc / hipFree.  splits * M * N * 4 bytes above the array's size are refused
 * with an error.  All calls on one GPU share that GPU's array, so calls that overlap in time on one
 * GPU race; calls on one stream are ordered and need no clearing in between.  The first call on a
 * device (or creating a model on it) looks the array's address up: make it outside graph capture.
 * flags: CUBERT_X_PACKED | CUBERT_W_PACKED. */
int cubert_op_gemm_splitk_noalloc(const void* X, const void* W, const float* bias, float* Y, int M, int N,
                                  int K, int ldx, int elt, int splits, int tile, int flags, void* stream);
size_t cubert_noalloc_scratch_bytes(void);

/* Fused QKV projection (op_BatchedLinear::forward, cuda_bert/ops/linear.cu:241-319):
 * X[B*S, hidden] * Wqkv[3*hidden, hidden]^T + bias -> q,k [B,heads,S,64],
 * vt [B,heads,64,Sp] with Sp = S rounded up to 32 (CUBERT_V_ROWMAJOR: V as [B,heads,S,64] in the same buffer). */
int cubert_op_gemm_qkv(const void* X, const void* W, const float* bias, void* q, void* k, void* vt,
                       int B, int S, int heads, int elt, int tile, int flags, void* stream);

/* Fused attention (Query_Key + op_SoftMax + Prob_Value,
 * cuda_bert/ops/batch_matmul.cu:48-141, ops/softmax.cu:86-143). */
int cubert_op_attention(const void* q, const void* k, const void* vt, const float* maskadd,
                        void* ctx, int B, int heads, int S, float scale, int elt, int flags,
                        void* stream); /* flags: CUBERT_Y_PACKED writes ctx packed (bf16); CUBERT_V_ROWMAJOR */

/* x <- LayerNorm(x + y); optional bf16 copy xb (op_LayerNorm::forward,
 * cuda_bert/ops/layernorm.cu:136-206). */
int cubert_op_add_layernorm(float* x, const void* y, int y_elt, const float* gamma,
                            const float* beta, void* xb, int rows, int hidden, int flags,
                            void* stream); /* flags: CUBERT_Y_PACKED writes xb packed;
                                              CUBERT_LN_NO_RESIDUAL: x <- LayerNorm(y), x is only written */

/* Embedding gather + add + LayerNorm + additive mask rows (Embedding::forward,
 * cuda_bert/ops/embedding.cu:3-58). */
int cubert_op_embed_layernorm(const int* ids, const int* seg, const int* mask, const float* word,
                              const float* pos, const float* type, const float* gamma,
                              const float* beta, float* x, void* xb, float* maskadd, int B, int S,
                              int hidden, int vocab, int type_vocab, int flags, void* stream);

/* pooled[b, :] = tanh(x[b * S, :] @ W^T + bias): first-token gather, dense and
 * tanh in one kernel (copy_pooler + op_Linear + op_Tanh, cuda_bert/utils/bert.cu:238-247;
 * ops/elementwise.cu:5-32, 56-70).  x float32 [B*S, hidden], W [hidden, hidden]
 * row-major ([out, in]) of type w_elt. */
int cubert_op_pooler(const float* x, const void* W, const float* bias, float* pooled, int B, int S,
                     int hidden, int w_elt, void* stream);

/* In-place scale + mask + softmax over materialised scores [B, rows_per_batch, S]
 * (cuApplySoftmax, cuda_bert/ops/softmax.cu:86-143). */
int cubert_op_mask_softmax(void* scores, int elt, const int* mask, int B, int rows_per_batch,
                           int S, float scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CUBERT_H_ */
