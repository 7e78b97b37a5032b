// The encoder model: device-resident weights, a static activation plan and the
// forward schedule.  Counterpart of `class bert` + `global_handle` of the
// reference (cuda_bert/utils/bert.cu:4-252, utils/manager.cu:4-109).
//
// Differences that matter to callers: all device memory is allocated once at
// construction (weights in one block, activations in one block sized for the
// token capacity), every buffer address is a pure function of the model, there
// are no host synchronisations inside the forward pass, and small batches are
// replayed from a hipGraph captured per (batch, seq) shape.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "common.h"

namespace cubert {

struct Compact;      // kernels.h

struct ModelOptions {
    Dims dims;
    int precision = kF32;      // operand type of the GEMMs and attention
    int gpu = 0;
    int max_batch = 0;         // (0, 0): default capacity of 200*512 tokens
    int max_seq = 0;
    int split_parts = 2;           // number of parts (1..4) a large batch is cut into
    int split_min_tokens = 14336;  // passes over at least this many token rows run as two halves on two streams (0: never);
                                   // the C API's default follows the precision
    bool fuse_residual = true;     // residual add in the epilogue of the GEMM before each LayerNorm
    bool fuse_layernorm = true;    // ... and the LayerNorm itself, where the GEMM kernel supports it (bf16, large batches)
    bool v_rowmajor = true;        // bf16, S <= 512: V is stored [B, heads, S, 64] like K; attention transposes on its LDS reads
    int attn_split_workgroups = kAttnSplitMaxWorkgroups;   // bf16, S <= 512, row-major V: batches of up to this many
                                   // (batch, head, 32 queries) blocks run the attention kernel that splits a head's keys
                                   // over a workgroup's waves (0: never)
    bool split_k = true;           // short batches: split K of the hidden-wide GEMMs (changes the summation order)
    int varlen = -1;               // host-input calls with prefix masks compute only the valid tokens: 1 always,
                                   // 0 never, -1 when the caller asks for no sequence output (see forward_host)
    int graph_max_tokens = 8192;   // capture a hipGraph for batches up to this many tokens (0: never)
    bool first_token_last_layer = true;   // calls that hand back no sequence output compute the last layer for the first
                                          // token of every sequence only (everything the pooler reads)
    int graph_cache = 64;          // instantiated hipGraphs kept per model (least recently used is dropped)
    std::string dir;
};

struct LayerDev {
    void *w_qkv, *w_ao, *w_in, *w_out;            // [out, in] in the operand type
    float *b_qkv, *b_ao, *b_in, *b_out;
    float *g1, *be1, *g2, *be2;
};

class Model {
  public:
    static Model* create(const ModelOptions& opt);     // nullptr + error text on failure
    ~Model();

    // Host inputs [B, S] int32 (mask may be nullptr).  Asynchronous.
    // need_seq: the caller will read the sequence output (else only pooled / classifier results).
    bool forward_host(const int* ids, const int* seg, const int* mask, int B, int S, bool need_seq = true);
    // Inputs already in device memory.  Asynchronous on stream().
    bool forward_device(const int* d_ids, const int* d_seg, const int* d_mask, int B, int S);
    // Unpadded forward: only the first h_lens[b] >= 1 tokens of every sequence are computed (as if
    // the attention mask were 1 on exactly those).  Pooled output and the sequence output on
    // the valid positions equal forward_device's bit for bit; the padding positions of the
    // sequence output are zero.  h_lens is host memory.  Asynchronous after the metadata upload.
    bool forward_device_lens(const int* d_ids, const int* d_seg, const int* h_lens, int B, int S);
    // softmax(pooled @ classifier_kernel + bias) for the last forward -> cls_probs().
    bool classify();
    // One eager forward pass with a hipEvent before every launch; fills
    // phase_ms[kNumPhases] with the summed time per phase (milliseconds).
    enum Phase { kPhEmbed = 0, kPhQKV, kPhAttention, kPhAttnOut, kPhLayerNorm, kPhFFNIn, kPhFFNOut, kPhPooler,
                 kNumPhases };
    bool profile_device(const int* d_ids, const int* d_seg, const int* d_mask, int B, int S, float* phase_ms);
    bool sync();
    bool copy_out(float* host_out, const float* dev, size_t floats);   // D2H + sync (again after a repeated pass)
    bool copy_pooled(float* host_out);                 // D2H + sync, B*hidden floats
    bool copy_seq(float* host_out);                    // D2H + sync, B*S*hidden floats
    bool copy_cls(float* host_out);                    // D2H + sync, B*num_classes floats

    float* seq_ptr() const { return last_compact_ ? seqpad_ : x32_; }
    float* pooled_ptr() const { return pooled_; }
    float* cls_ptr() const { return cls_; }
    hipStream_t stream() const { return stream_; }
    const Dims& dims() const { return opt_.dims; }
    int precision() const { return opt_.precision; }
    int num_classes() const { return num_classes_; }
    long capacity_tokens() const { return cap_tokens_; }
    int last_batch() const { return B_; }
    int last_seq() const { return S_; }
    int graphs_cached() const;                         // instantiated hipGraphs held
    int ln_fallbacks() const { return ln_fallbacks_; } // passes repeated with separate LayerNorm kernels (see sync())
    bool force_ln_timeout();                           // test aid: the next pass with a LayerNorm epilogue times out
    size_t weight_bytes() const { return weight_bytes_; }
    size_t activation_bytes() const { return act_bytes_; }

  private:
    Model() = default;
    bool init(const ModelOptions& opt);
    bool check_shape(int B, int S);
    bool run(int B, int S, bool has_mask);             // graph or eager
    bool enqueue(int B, int S, bool has_mask);         // the launch sequence (one or two parts)
    bool enqueue_part(int part, int b0, int B, size_t r0, int S, bool has_mask, hipStream_t st, const Compact* cp = nullptr);
    bool run_compact(const int* h_lens, int B, int S);
    bool rerun_last();                                 // the last pass once more, eagerly, from the inputs still on the device
    bool mark(int phase);                              // profiling: event before a launch

    ModelOptions opt_;
    hipStream_t stream_ = nullptr;
    static constexpr int kMaxParts = 4;
    hipStream_t side_[kMaxParts] = {};           // streams of parts 1.. of a split batch
    hipEvent_t ev_fork_ = nullptr, ev_join_[kMaxParts] = {};
    // weights
    unsigned char* wblock_ = nullptr;
    size_t weight_bytes_ = 0;
    float *word_ = nullptr, *pos_ = nullptr, *type_ = nullptr, *emb_g_ = nullptr, *emb_b_ = nullptr;
    std::vector<LayerDev> layers_;
    void* w_pool_ = nullptr;
    float* b_pool_ = nullptr;
    float *w_cls_ = nullptr, *b_cls_ = nullptr;
    int num_classes_ = 0;
    // activations
    unsigned char* ablock_ = nullptr;
    size_t act_bytes_ = 0;
    long cap_tokens_ = 0;
    float* x32_ = nullptr;       // residual stream / sequence output [N, H] f32
    bf16_t* xb_ = nullptr;       // bf16 copy of x (bf16 mode only)
    void *q_ = nullptr, *k_ = nullptr, *vt_ = nullptr, *ctx_ = nullptr, *h_ = nullptr;
    float* y32_ = nullptr;       // attn-out / ffn-out GEMM result [N, H] f32
    float* maskadd_ = nullptr;   // [B, Sp]
    float* pooled_ = nullptr;    // [B, H]
    float* cls_ = nullptr;       // [B, C]
    int* d_in_ = nullptr;        // ids | seg | mask, cap_tokens each
    int* h_in_ = nullptr;        // pinned staging, same layout
    // unpadded passes: per part a row map (token index of every compact row) and cu (row offsets)
    static constexpr int kSplitRows = 8192;   // extra rows of y32 for the partial results of split-K GEMMs
    static constexpr int kCuStride = 1032;    // B <= 1024 per part, + 1
    int* d_meta_ = nullptr;      // rowmap (cap tokens) | cu (kMaxParts * kCuStride)
    int* h_meta_ = nullptr;      // pinned, same layout
    float* seqpad_ = nullptr;    // padded [B, S, H] sequence output of an unpadded pass
    unsigned char* ln_ws_ = nullptr;   // kMaxParts workspaces of the GEMMs that normalise in their epilogue
    size_t ln_ws_bytes_ = 0;           // size of one of them
    int ln_used_ = 0;                  // parts whose workspaces such GEMMs used since sync() last looked at their error words
    int ln_fallbacks_ = 0;             // times sync() found an error word raised and repeated the pass without the fused LayerNorm
    bool recovered_ = false;           // the last sync() repeated the pass: copies enqueued before it carry the discarded results
    bool last_has_mask_ = false, last_classified_ = false;
    std::vector<int> last_lens_;       // lengths of the last unpadded pass
    // Last layer for the first tokens only: [kMaxParts * 1024] rows each (a part's sequences at part * 1024)
    float *xc32_ = nullptr, *yc32_ = nullptr;      // residual stream / GEMM result of those rows
    bf16_t* xbc_ = nullptr;                        // bf16 copy (bf16 mode)
    void *ctxc_ = nullptr, *hc_ = nullptr;         // attention context / FFN activation of those rows
    bool first_only_ = false;                      // the pass being enqueued (and the last one run) is of that kind
    bool last_compact_ = false;
    int cur_parts_ = 1;          // parts of the pass being enqueued
    int cur_attn_ = kAttnPerHead;   // attention kernel of the pass being enqueued (decided on the whole batch)
    int B_ = 0, S_ = 0;
    // hipGraph cache: one entry per (B, S, mask) shape, captured on second sight, at most
    // opt_.graph_cache instantiated at a time (least recently used goes first).
    int max_graphs() const { return opt_.graph_cache > 0 ? opt_.graph_cache : 1; }
    struct GraphEntry {
        hipGraphExec_t exec = nullptr;
        unsigned long long last_use = 0;
        int ln_parts = 0;        // parts whose LayerNorm-epilogue workspaces the captured pass uses
    };
    std::map<unsigned long long, GraphEntry> graphs_;
    unsigned long long graph_clock_ = 0;
    bool evict_graphs(int keep);
    void forget_uncaptured_shapes();
    bool profiling_ = false;
    std::vector<hipEvent_t> prof_events_;
    std::vector<int> prof_phase_;
    size_t prof_used_ = 0;
};

}  // namespace cubert
