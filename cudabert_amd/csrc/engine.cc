#include "engine.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <iterator>

#include "kernels.h"
#include "weights.h"

namespace cubert {

namespace {

thread_local std::string g_error;

struct Arena {
    size_t off = 0;
    size_t take(size_t bytes) {
        const size_t at = off;
        off += (bytes + 255) / 256 * 256;
        return at;
    }
};

}  // namespace

void set_error(const std::string& msg) { g_error = msg; }
const char* get_error() { return g_error.c_str(); }

Model* Model::create(const ModelOptions& opt) {
    Model* m = new Model();
    if (!m->init(opt)) {
        const std::string keep = g_error;      // the destructor may issue HIP calls
        delete m;
        g_error = keep;
        return nullptr;
    }
    return m;
}

Model::~Model() {
    if (stream_) (void)hipStreamSynchronize(stream_);
    for (auto& kv : graphs_)
        if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
    for (hipEvent_t e : prof_events_) (void)hipEventDestroy(e);
    if (wblock_) (void)hipFree(wblock_);
    if (ablock_) (void)hipFree(ablock_);
    if (h_in_) (void)hipHostFree(h_in_);
    if (h_meta_) (void)hipHostFree(h_meta_);
    if (ev_fork_) (void)hipEventDestroy(ev_fork_);
    for (int i = 1; i < kMaxParts; ++i) {
        if (ev_join_[i]) (void)hipEventDestroy(ev_join_[i]);
        if (side_[i]) (void)hipStreamDestroy(side_[i]);
    }
    if (stream_) (void)hipStreamDestroy(stream_);
}

bool Model::init(const ModelOptions& opt_in) {
    opt_ = opt_in;
    Dims& D = opt_.dims;
    if (opt_.precision != kF32 && opt_.precision != kBF16) { set_error("precision must be 0 (f32) or 1 (bf16)"); return false; }
    if (D.hidden <= 0 || D.layers <= 0 || D.heads <= 0 || D.inter <= 0) { set_error("model dimensions must be positive"); return false; }
    if (D.hidden != D.heads * 64) { set_error("head dimension must be 64 (hidden == 64 * heads)"); return false; }
    if (D.hidden > 1024 || D.hidden % 64 != 0 || D.inter % 64 != 0) {
        set_error("hidden must be a multiple of 64 up to 1024 and intermediate a multiple of 64");
        return false;
    }
    if ((opt_.max_batch == 0) != (opt_.max_seq == 0) || opt_.max_batch < 0 || opt_.max_seq < 0) {
        set_error("max_batchsize and max_seq_length must both be zero or both be positive");
        return false;
    }

    // ---- host side first: nothing touches the GPU until the directory is valid ----
    WeightDir wd;
    if (!load_weight_dir(opt_.dir, &D, &wd)) return false;
    if (opt_.max_seq > D.max_pos) {
        set_error("max_seq_length " + std::to_string(opt_.max_seq) + " exceeds the position table (" +
                  std::to_string(D.max_pos) + ")");
        return false;
    }
    // Token capacity: explicit (B, S) as given, else the reference's default of
    // 200*512 tokens (cuda_bert/utils/manager.cuh:55).
    cap_tokens_ = opt_.max_batch ? (long)opt_.max_batch * opt_.max_seq : 200L * 512L;

    int ndev = 0;
    CUBERT_HIP_OK(hipGetDeviceCount(&ndev));
    if (opt_.gpu < 0 || opt_.gpu >= ndev) {
        set_error("GPU " + std::to_string(opt_.gpu) + " does not exist (" + std::to_string(ndev) + " visible)");
        return false;
    }
    CUBERT_HIP_OK(hipSetDevice(opt_.gpu));
    // best effort: the allocation-free GEMM entry point looks its scratch address up itself if this did not work
    if (!noalloc_setup_current_device()) set_error("");
    CUBERT_HIP_OK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    for (int i = 1; i < kMaxParts; ++i) {
        CUBERT_HIP_OK(hipStreamCreateWithFlags(&side_[i], hipStreamNonBlocking));
        CUBERT_HIP_OK(hipEventCreateWithFlags(&ev_join_[i], hipEventDisableTiming));
    }
    CUBERT_HIP_OK(hipEventCreateWithFlags(&ev_fork_, hipEventDisableTiming));

    const int elt = opt_.precision;
    const size_t es = elt == kBF16 ? 2 : 4;
    const size_t H = D.hidden, I = D.inter;

    // ---- weight block layout ----
    Arena wa;
    const size_t o_word = wa.take((size_t)D.vocab * H * 4), o_pos = wa.take((size_t)D.max_pos * H * 4),
                 o_type = wa.take((size_t)D.type_vocab * H * 4), o_eg = wa.take(H * 4), o_eb = wa.take(H * 4);
    auto wbytes = [&](size_t rows, size_t k) { return elt == kBF16 ? packed_bytes(rows, k * 2) : rows * k * es; };
    struct LayerOff { size_t w_qkv, w_ao, w_in, w_out, b_qkv, b_ao, b_in, b_out, g1, be1, g2, be2; };
    std::vector<LayerOff> lo(D.layers);
    for (auto& l : lo) {
        // packed operands (bf16 mode) pad their rows to a multiple of 256
        l.w_qkv = wa.take(wbytes(3 * H, H)); l.w_ao = wa.take(wbytes(H, H));
        l.w_in = wa.take(wbytes(I, H)); l.w_out = wa.take(wbytes(H, I));
        l.b_qkv = wa.take(3 * H * 4); l.b_ao = wa.take(H * 4); l.b_in = wa.take(I * 4); l.b_out = wa.take(H * 4);
        l.g1 = wa.take(H * 4); l.be1 = wa.take(H * 4); l.g2 = wa.take(H * 4); l.be2 = wa.take(H * 4);
    }
    const size_t o_wp = wa.take(H * H * es), o_bp = wa.take(H * 4);
    num_classes_ = wd.num_classes;
    const size_t o_wc = wa.take((size_t)(num_classes_ ? num_classes_ : 1) * H * 4), o_bc = wa.take(8 * 4);
    const size_t stage_floats = std::max(H * I, H * H);
    const size_t o_stage = wa.take(stage_floats * 4);
    weight_bytes_ = wa.off;
    CUBERT_HIP_OK(hipMalloc(reinterpret_cast<void**>(&wblock_), weight_bytes_));

    auto up = [&](size_t off, const NpyArray* a) -> bool {
        CUBERT_HIP_OK(hipMemcpy(wblock_ + off, a->data.data(), a->data.size() * 4, hipMemcpyHostToDevice));
        return true;
    };
    // [in, out] float32 on disk -> [out, in] operand type on device
    float* stage = reinterpret_cast<float*>(wblock_ + o_stage);
    // bf16 mode keeps GEMM operands in the packed layout (common.h); the pooler
    // weight stays row-major (its kernel is a plain dot product).
    const bool packed = elt == kBF16;
    bool pack_this = true;
    // `row0`: first output row of this tensor inside the destination matrix (the
    // Q, K and V kernels are stacked into one [3H, H] operand).
    auto up_t = [&](size_t off, const NpyArray* a, int row0 = 0) -> bool {
        const int K = (int)a->shape[0], N = (int)a->shape[1];
        CUBERT_HIP_OK(hipMemcpyAsync(stage, a->data.data(), a->data.size() * 4, hipMemcpyHostToDevice, stream_));
        const bool pk = packed && pack_this;
        unsigned char* dst = wblock_ + off + (pk ? 0 : (size_t)row0 * K * es);
        if (!launch_transpose_convert(stage, dst, K, N, elt, pk, pk ? row0 : 0, stream_)) return false;
        CUBERT_HIP_OK(hipStreamSynchronize(stream_));      // the staging buffer is reused
        return true;
    };
    if (!up(o_word, wd.word) || !up(o_pos, wd.pos) || !up(o_type, wd.type) || !up(o_eg, wd.emb_g) || !up(o_eb, wd.emb_b))
        return false;
    word_ = reinterpret_cast<float*>(wblock_ + o_word);
    pos_ = reinterpret_cast<float*>(wblock_ + o_pos);
    type_ = reinterpret_cast<float*>(wblock_ + o_type);
    emb_g_ = reinterpret_cast<float*>(wblock_ + o_eg);
    emb_b_ = reinterpret_cast<float*>(wblock_ + o_eb);
    layers_.resize(D.layers);
    for (int i = 0; i < D.layers; ++i) {
        const LayerTensors& T = wd.layers[i];
        const LayerOff& l = lo[i];
        // Q, K, V stacked along the output axis: rows [0,H) query, [H,2H) key, [2H,3H) value
        // (the reference concatenates them too, cuda_bert/ops/linear.cu:60-88).
        if (!up_t(l.w_qkv, T.q_k, 0) || !up_t(l.w_qkv, T.k_k, (int)H) || !up_t(l.w_qkv, T.v_k, 2 * (int)H) ||
            !up_t(l.w_ao, T.ao_k) || !up_t(l.w_in, T.in_k) || !up_t(l.w_out, T.out_k))
            return false;
        if (!up(l.b_qkv, T.q_b) || !up(l.b_qkv + H * 4, T.k_b) || !up(l.b_qkv + 2 * H * 4, T.v_b) ||
            !up(l.b_ao, T.ao_b) || !up(l.b_in, T.in_b) || !up(l.b_out, T.out_b) || !up(l.g1, T.ao_g) ||
            !up(l.be1, T.ao_be) || !up(l.g2, T.out_g) || !up(l.be2, T.out_be))
            return false;
        LayerDev& L = layers_[i];
        L.w_qkv = wblock_ + l.w_qkv; L.w_ao = wblock_ + l.w_ao; L.w_in = wblock_ + l.w_in; L.w_out = wblock_ + l.w_out;
        L.b_qkv = reinterpret_cast<float*>(wblock_ + l.b_qkv); L.b_ao = reinterpret_cast<float*>(wblock_ + l.b_ao);
        L.b_in = reinterpret_cast<float*>(wblock_ + l.b_in); L.b_out = reinterpret_cast<float*>(wblock_ + l.b_out);
        L.g1 = reinterpret_cast<float*>(wblock_ + l.g1); L.be1 = reinterpret_cast<float*>(wblock_ + l.be1);
        L.g2 = reinterpret_cast<float*>(wblock_ + l.g2); L.be2 = reinterpret_cast<float*>(wblock_ + l.be2);
    }
    pack_this = false;
    if (!up_t(o_wp, wd.pool_k) || !up(o_bp, wd.pool_b)) return false;
    w_pool_ = wblock_ + o_wp;
    b_pool_ = reinterpret_cast<float*>(wblock_ + o_bp);
    if (num_classes_) {
        if (!up(o_wc, wd.cls_k) || !up(o_bc, wd.cls_b)) return false;
        w_cls_ = reinterpret_cast<float*>(wblock_ + o_wc);
        b_cls_ = reinterpret_cast<float*>(wblock_ + o_bc);
    }

    // ---- activation block: one allocation, addresses fixed for the model's life ----
    // B <= 1024 and every sequence is padded by < 32 key columns in vt/maskadd.
    // Packed operands pad rows to 256; a batch split over several streams has one such region per part.
    const size_t N = ((size_t)cap_tokens_ + 255) / 256 * 256 + 256 * (kMaxParts - 1);
    const size_t Npad = N + 32 * 1024;
    Arena aa;
    const size_t o_x32 = aa.take(N * H * 4);
    const size_t o_xb = elt == kBF16 ? aa.take(N * H * 2) : 0;
    const size_t o_q = aa.take((N + 64) * H * es), o_k = aa.take((N + 64) * H * es);
    const size_t o_vt = aa.take(Npad * H * es), o_ctx = aa.take(N * H * es);
    const size_t o_h = aa.take(N * I * es), o_y = aa.take((N + kSplitRows) * H * 4);
    const size_t o_mask = aa.take(Npad * 4), o_pool = aa.take((size_t)1024 * H * 4), o_cls = aa.take(1024 * 8 * 4);
    const size_t o_in = aa.take(3 * N * 4);
    const size_t meta_ints = N + (size_t)kMaxParts * kCuStride;
    const size_t o_meta = aa.take(meta_ints * 4), o_seqpad = aa.take(N * H * 4);
    ln_ws_bytes_ = (gemm_ln_workspace_bytes(N) + 255) / 256 * 256;
    const size_t o_lnws = aa.take(ln_ws_bytes_ * kMaxParts);
    const size_t NC = (size_t)kMaxParts * 1024;       // first-token rows: B <= 1024 per part, parts 1024 rows apart
    const size_t o_xc = aa.take(NC * H * 4), o_yc = aa.take(NC * H * 4), o_xbc = elt == kBF16 ? aa.take(NC * H * 2) : 0;
    const size_t o_ctxc = aa.take(NC * H * es), o_hc = aa.take(NC * I * es);
    act_bytes_ = aa.off;
    size_t free_b = 0, total_b = 0;
    CUBERT_HIP_OK(hipMemGetInfo(&free_b, &total_b));
    if (act_bytes_ > free_b) {
        set_error("activation plan needs " + std::to_string(act_bytes_ >> 20) + " MiB but only " +
                  std::to_string(free_b >> 20) + " MiB of device memory are free");
        return false;
    }
    CUBERT_HIP_OK(hipMalloc(reinterpret_cast<void**>(&ablock_), act_bytes_));
    // K rows past a sequence end and V^T padding columns are read (and then
    // masked out); they must hold finite numbers, so start from all zeros.
    CUBERT_HIP_OK(hipMemsetAsync(ablock_, 0, act_bytes_, stream_));
    x32_ = reinterpret_cast<float*>(ablock_ + o_x32);
    xb_ = elt == kBF16 ? reinterpret_cast<bf16_t*>(ablock_ + o_xb) : nullptr;
    q_ = ablock_ + o_q; k_ = ablock_ + o_k; vt_ = ablock_ + o_vt; ctx_ = ablock_ + o_ctx; h_ = ablock_ + o_h;
    y32_ = reinterpret_cast<float*>(ablock_ + o_y);
    maskadd_ = reinterpret_cast<float*>(ablock_ + o_mask);
    pooled_ = reinterpret_cast<float*>(ablock_ + o_pool);
    cls_ = reinterpret_cast<float*>(ablock_ + o_cls);
    d_in_ = reinterpret_cast<int*>(ablock_ + o_in);
    d_meta_ = reinterpret_cast<int*>(ablock_ + o_meta);
    seqpad_ = reinterpret_cast<float*>(ablock_ + o_seqpad);
    ln_ws_ = ablock_ + o_lnws;       // all zero from the clearing above, which is what the first launch needs
    xc32_ = reinterpret_cast<float*>(ablock_ + o_xc);
    yc32_ = reinterpret_cast<float*>(ablock_ + o_yc);
    xbc_ = elt == kBF16 ? reinterpret_cast<bf16_t*>(ablock_ + o_xbc) : nullptr;
    ctxc_ = ablock_ + o_ctxc;
    hc_ = ablock_ + o_hc;
    CUBERT_HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&h_meta_), meta_ints * 4, hipHostMallocDefault));
    CUBERT_HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&h_in_), 3 * N * 4, hipHostMallocDefault));
    CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    return true;
}

bool Model::force_ln_timeout() {
    CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    for (int i = 0; i < kMaxParts; ++i)
        if (!gemm_ln_workspace_force_expiry(ln_ws_ + (size_t)i * ln_ws_bytes_)) return false;
    return true;
}

bool Model::check_shape(int B, int S) {
    // Limits inherited from the reference: B*S within the allocated capacity
    // (cuda_bert/utils/manager.cu:100-108), B <= 1024 (ops/batch_matmul.cu:60),
    // S within the position table.
    if (B <= 0 || S <= 0) { set_error("batchsize and seq_length must be positive"); return false; }
    if (B > 1024) { set_error("batchsize " + std::to_string(B) + " exceeds 1024"); return false; }
    if (S > opt_.dims.max_pos) {
        set_error("seq_length " + std::to_string(S) + " exceeds the position table (" + std::to_string(opt_.dims.max_pos) + ")");
        return false;
    }
    if ((long)B * S > cap_tokens_) {
        set_error("batchsize * seq_length = " + std::to_string((long)B * S) + " exceeds the allocated capacity of " +
                  std::to_string(cap_tokens_) + " tokens");
        return false;
    }
    return true;
}

bool Model::forward_host(const int* ids, const int* seg, const int* mask, int B, int S, bool need_seq) {
    if (!check_shape(B, S)) return false;
    if (!ids || !seg) { set_error("input_ids and token_type_ids must not be null"); return false; }
    const size_t n = (size_t)B * S, cap = (size_t)cap_tokens_;
    const Dims& D = opt_.dims;
    for (size_t i = 0; i < n; ++i) {
        if ((unsigned)ids[i] >= (unsigned)D.vocab) {
            set_error("input id " + std::to_string(ids[i]) + " at position " + std::to_string(i) + " is outside the vocabulary");
            return false;
        }
        if ((unsigned)seg[i] >= (unsigned)D.type_vocab) {
            set_error("token type " + std::to_string(seg[i]) + " at position " + std::to_string(i) + " is out of range");
            return false;
        }
    }
    // The pinned staging buffer is reused by every call: the previous upload
    // must have left it before it is overwritten.
    CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    std::memcpy(h_in_, ids, n * 4);
    std::memcpy(h_in_ + cap, seg, n * 4);
    if (mask) std::memcpy(h_in_ + 2 * cap, mask, n * 4);
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_, h_in_, n * 4, hipMemcpyHostToDevice, stream_));
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + cap, h_in_ + cap, n * 4, hipMemcpyHostToDevice, stream_));
    if (mask) CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + 2 * cap, h_in_ + 2 * cap, n * 4, hipMemcpyHostToDevice, stream_));
    // Masks that are 1 on a non-empty prefix and 0 after it allow the unpadded pass (valid tokens
    // only; same pooled output bit for bit, zeros instead of values on the padding positions of the
    // sequence output).  varlen = 1: whenever the masks allow it.  varlen = -1 (default): only when
    // the caller cannot see the sequence output, the batch is too large for hipGraph replay and at
    // least 5 % of it is padding.
    const bool too_big_for_graph = opt_.graph_max_tokens <= 0 || (long)n > opt_.graph_max_tokens;
    // The caller will not see the sequence output: the last layer only has to produce what the pooler reads.
    first_only_ = !need_seq && opt_.first_token_last_layer;
    if (mask && (opt_.varlen == 1 || (opt_.varlen < 0 && !need_seq && too_big_for_graph))) {
        std::vector<int> lens(B);
        bool prefix = true;
        size_t valid = 0;
        for (int b = 0; b < B && prefix; ++b) {
            const int* m = mask + (size_t)b * S;
            int len = 0;
            while (len < S && m[len] == 1) ++len;
            for (int s = len; s < S && prefix; ++s) prefix = m[s] == 0;
            prefix = prefix && len >= 1;
            lens[b] = len;
            valid += (size_t)len;
        }
        if (prefix && (opt_.varlen == 1 || valid * 20 <= n * 19)) return run_compact(lens.data(), B, S);
    }
    return run(B, S, mask != nullptr);
}

bool Model::forward_device_lens(const int* d_ids, const int* d_seg, const int* h_lens, int B, int S) {
    if (!check_shape(B, S)) return false;
    first_only_ = false;
    if (!d_ids || !d_seg || !h_lens) { set_error("input_ids, token_type_ids and lengths must not be null"); return false; }
    for (int b = 0; b < B; ++b)
        if (h_lens[b] < 1 || h_lens[b] > S) {
            set_error("length " + std::to_string(h_lens[b]) + " of sequence " + std::to_string(b) + " is outside 1.." + std::to_string(S));
            return false;
        }
    const size_t n = (size_t)B * S, cap = (size_t)cap_tokens_;
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_, d_ids, n * 4, hipMemcpyDeviceToDevice, stream_));
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + cap, d_seg, n * 4, hipMemcpyDeviceToDevice, stream_));
    return run_compact(h_lens, B, S);
}

// Unpadded pass: the host lays out, per part, the token index of every compact row and the
// row offset of every sequence, uploads both and enqueues the parts (never through a graph:
// the row counts change from call to call).
bool Model::run_compact(const int* lens, int B, int S) {
    B_ = B;
    S_ = S;
    last_compact_ = true;
    last_classified_ = false;
    if (lens != last_lens_.data()) last_lens_.assign(lens, lens + B);
    long tokens = 0;                  // rows this pass computes: the valid tokens
    for (int b = 0; b < B; ++b) tokens += lens[b];
    int parts = opt_.split_parts < kMaxParts ? opt_.split_parts : kMaxParts;
    if (parts > B) parts = B;
    if (parts < 1 || opt_.split_min_tokens <= 0 || tokens < opt_.split_min_tokens) parts = 1;
    // the pinned metadata of the previous call must have been consumed
    CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    const size_t cap = (size_t)cap_tokens_;
    // packed operands pad every part to 256 rows; capacity was sized for kMaxParts such regions
    Compact cp[kMaxParts];
    size_t r0[kMaxParts];
    int b0s[kMaxParts], Bs[kMaxParts];
    size_t rows_total = 0, r = 0;
    for (int i = 0, b0 = 0; i < parts; ++i) {
        const int Bi = B / parts + (i < B % parts ? 1 : 0);
        int* rowmap = h_meta_ + rows_total;
        int* cu = h_meta_ + cap + 256 * (kMaxParts - 1) + (size_t)i * kCuStride;
        int rows = 0;
        for (int b = 0; b < Bi; ++b) {
            cu[b] = rows;
            for (int s = 0; s < lens[b0 + b]; ++s) rowmap[rows++] = b * S + s;
        }
        cu[Bi] = rows;
        cp[i].rowmap = d_meta_ + rows_total;
        cp[i].cu = d_meta_ + cap + 256 * (kMaxParts - 1) + (size_t)i * kCuStride;
        cp[i].rows = rows;
        r0[i] = r;
        b0s[i] = b0;
        Bs[i] = Bi;
        rows_total += rows;
        r += (size_t)round_up(rows, 256);
        b0 += Bi;
    }
    CUBERT_HIP_OK(hipMemcpyAsync(d_meta_, h_meta_, rows_total * 4, hipMemcpyHostToDevice, stream_));
    const size_t cu_off = cap + 256 * (kMaxParts - 1);
    CUBERT_HIP_OK(hipMemcpyAsync(d_meta_ + cu_off, h_meta_ + cu_off, (size_t)parts * kCuStride * 4, hipMemcpyHostToDevice, stream_));
    cur_parts_ = parts;
    cur_attn_ = (long)B * opt_.dims.heads * ((S + 31) / 32) <= opt_.attn_split_workgroups ? kAttnSplitKeys : kAttnPerHead;
    if (parts == 1) return enqueue_part(0, 0, B, 0, S, false, stream_, &cp[0]);
    CUBERT_HIP_OK(hipEventRecord(ev_fork_, stream_));
    bool ok = true;
    for (int i = 0; i < parts; ++i) {
        hipStream_t st = i == 0 ? stream_ : side_[i];
        if (i > 0) CUBERT_HIP_OK(hipStreamWaitEvent(st, ev_fork_, 0));
        ok = ok && enqueue_part(i, b0s[i], Bs[i], r0[i], S, false, st, &cp[i]);
        if (i > 0) {
            CUBERT_HIP_OK(hipEventRecord(ev_join_[i], st));
            CUBERT_HIP_OK(hipStreamWaitEvent(stream_, ev_join_[i], 0));
        }
    }
    return ok;
}

bool Model::forward_device(const int* d_ids, const int* d_seg, const int* d_mask, int B, int S) {
    if (!check_shape(B, S)) return false;
    first_only_ = false;
    if (!d_ids || !d_seg) { set_error("input_ids and token_type_ids must not be null"); return false; }
    const size_t n = (size_t)B * S, cap = (size_t)cap_tokens_;
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_, d_ids, n * 4, hipMemcpyDeviceToDevice, stream_));
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + cap, d_seg, n * 4, hipMemcpyDeviceToDevice, stream_));
    if (d_mask) CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + 2 * cap, d_mask, n * 4, hipMemcpyDeviceToDevice, stream_));
    return run(B, S, d_mask != nullptr);
}

bool Model::run(int B, int S, bool has_mask) {
    B_ = B;
    S_ = S;
    last_compact_ = false;
    last_has_mask_ = has_mask;
    last_classified_ = false;
    const long tokens = (long)B * S;
    if (opt_.graph_max_tokens <= 0 || tokens > opt_.graph_max_tokens) return enqueue(B, S, has_mask);
    // One entry per (B, S, mask, kind of last layer) shape; the key is injective for every B <= 1024 and any S.
    const unsigned long long key = ((unsigned long long)B << 33) | ((unsigned long long)(unsigned)S << 1) | (has_mask ? 1ull : 0ull) |
                                   (first_only_ ? 1ull << 62 : 0ull);
    auto it = graphs_.find(key);
    if (it != graphs_.end() && it->second.exec) {
        it->second.last_use = ++graph_clock_;
        CUBERT_HIP_OK(hipGraphLaunch(it->second.exec, stream_));
        ln_used_ = std::max(ln_used_, it->second.ln_parts);      // sync() looks at the error words of a replayed pass too
        return true;
    }
    if (it == graphs_.end()) {
        // first sight: run eagerly (one-time kernel setup) and remember the shape
        if (graphs_.size() >= 4 * (size_t)max_graphs()) forget_uncaptured_shapes();
        graphs_[key].last_use = ++graph_clock_;
        return enqueue(B, S, has_mask);
    }
    // second sight: capture the launch sequence, then replay it.  The cache holds at most
    // max_graphs() instantiated graphs; the least recently used one makes room.
    if (!evict_graphs(max_graphs() - 1)) return false;
    GraphEntry& ge = graphs_[key];
    hipGraph_t graph = nullptr;
    CUBERT_HIP_OK(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal));
    const int ln_before = ln_used_;
    ln_used_ = 0;
    const bool ok = enqueue(B, S, has_mask);
    ge.ln_parts = ln_used_;
    ln_used_ = std::max(ln_before, ge.ln_parts);
    const std::string keep = ok ? std::string() : std::string(get_error());
    const hipError_t e = hipStreamEndCapture(stream_, &graph);
    if (!ok) { if (graph) (void)hipGraphDestroy(graph); set_error(keep); return false; }
    if (e != hipSuccess) { set_error(std::string("hipStreamEndCapture failed: ") + hipGetErrorString(e)); return false; }
    const hipError_t e2 = hipGraphInstantiate(&ge.exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e2 != hipSuccess) { ge.exec = nullptr; set_error(std::string("hipGraphInstantiate failed: ") + hipGetErrorString(e2)); return false; }
    ge.last_use = ++graph_clock_;
    CUBERT_HIP_OK(hipGraphLaunch(ge.exec, stream_));
    return true;
}

int Model::graphs_cached() const {
    int n = 0;
    for (const auto& kv : graphs_) n += kv.second.exec ? 1 : 0;
    return n;
}

// Destroys least recently used graphs until at most `keep` remain.  A graph may still be
// running on the stream, so the stream is drained first (evictions are rare).
bool Model::evict_graphs(int keep) {
    int have = graphs_cached();
    if (have <= keep) return true;
    CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    while (have > keep) {
        auto lru = graphs_.end();
        for (auto it = graphs_.begin(); it != graphs_.end(); ++it)
            if (it->second.exec && (lru == graphs_.end() || it->second.last_use < lru->second.last_use)) lru = it;
        if (lru == graphs_.end()) break;
        (void)hipGraphExecDestroy(lru->second.exec);
        graphs_.erase(lru);
        --have;
    }
    return true;
}

// Shapes seen once and never again would otherwise pile up in the map.
void Model::forget_uncaptured_shapes() {
    for (auto it = graphs_.begin(); it != graphs_.end();)
        it = it->second.exec ? std::next(it) : graphs_.erase(it);
}

// One forward pass.  A large batch is cut into parts of whole sequences that run
// the same launch sequence on separate streams: the parts are independent, and
// while one part's GEMM is in its last, partly filled round of tiles (or in a
// bandwidth-bound row kernel) another part's kernel takes the idle CUs.
bool Model::enqueue(int B, int S, bool has_mask) {
    const long tokens = (long)B * S;
    cur_attn_ = (long)B * opt_.dims.heads * ((S + 31) / 32) <= opt_.attn_split_workgroups ? kAttnSplitKeys : kAttnPerHead;
    int parts = opt_.split_parts < kMaxParts ? opt_.split_parts : kMaxParts;
    if (parts > B) parts = B;
    if (profiling_ || parts < 2 || opt_.split_min_tokens <= 0 || tokens < opt_.split_min_tokens) {
        cur_parts_ = 1;
        return enqueue_part(0, 0, B, 0, S, has_mask, stream_);
    }
    cur_parts_ = parts;
    CUBERT_HIP_OK(hipEventRecord(ev_fork_, stream_));
    bool ok = true;
    size_t r0 = 0;
    for (int i = 0, b0 = 0; i < parts; ++i) {
        const int Bi = B / parts + (i < B % parts ? 1 : 0);
        hipStream_t st = i == 0 ? stream_ : side_[i];
        if (i > 0) CUBERT_HIP_OK(hipStreamWaitEvent(st, ev_fork_, 0));
        ok = ok && enqueue_part(i, b0, Bi, r0, S, has_mask, st);
        // join even after a failed launch so that a capture in progress can be closed
        if (i > 0) {
            CUBERT_HIP_OK(hipEventRecord(ev_join_[i], st));
            CUBERT_HIP_OK(hipStreamWaitEvent(stream_, ev_join_[i], 0));
        }
        b0 += Bi;
        r0 += (size_t)round_up(Bi * S, 256);
    }
    return ok;
}

// The launch sequence for sequences [b0, b0 + B) (cuda_bert/utils/bert.cu:129-252):
// 1 + 7 * layers + 1 kernels (1 + 5 * layers + 1 when the GEMMs before the LayerNorms normalise in their
// epilogue), no host synchronisation.  `r0` is the first row of
// this part in the internal activation buffers (a multiple of 256, so that a
// packed operand starts on a block boundary); inputs and the sequence output
// are indexed by token.
bool Model::enqueue_part(int part, int b0, int B, size_t r0, int S, bool has_mask, hipStream_t st, const Compact* cp) {
    const Dims& D = opt_.dims;
    const int elt = opt_.precision;
    const size_t es = elt == kBF16 ? 2 : 4;
    // rows of this part: every token, or (unpadded pass) the valid ones only, stored from row r0
    const int H = D.hidden, I = D.inter, N = cp ? cp->rows : B * S, Sp = round_up(S, 32);
    const size_t cap = (size_t)cap_tokens_, t0 = (size_t)b0 * S;
    const int* cu = cp ? cp->cu : nullptr;
    const int *ids = d_in_ + t0, *seg = d_in_ + cap + t0, *mask = has_mask ? d_in_ + 2 * cap + t0 : nullptr;
    float* x32 = x32_ + (cp ? r0 : t0) * H;
    float* y32 = y32_ + r0 * H;
    bf16_t* xb = xb_ ? xb_ + r0 * H : nullptr;
    unsigned char* q = static_cast<unsigned char*>(q_) + t0 * H * es;
    unsigned char* k = static_cast<unsigned char*>(k_) + t0 * H * es;
    unsigned char* vt = static_cast<unsigned char*>(vt_) + (size_t)b0 * H * Sp * es;
    unsigned char* ctx = static_cast<unsigned char*>(ctx_) + r0 * H * es;
    unsigned char* h = static_cast<unsigned char*>(h_) + r0 * I * es;
    float* maskadd = maskadd_ + (size_t)b0 * Sp;
    const void* xin = elt == kBF16 ? static_cast<const void*>(xb) : static_cast<const void*>(x32);
    const float scale = 1.0f / std::sqrt(64.0f);

    // Short batches: the two GEMMs with only `hidden` output features have too few tiles for the
    // chip; they split K over several workgroups and the LayerNorm that follows adds the parts.
    // (Not for the parts of a split batch, which sit side by side in y32; the parts of K need rows of y32.)
    auto plan_for = [&](int K) {
        int max_splits = 1;
        if (cur_parts_ == 1 && opt_.split_k) {
            max_splits = 16;
            while (max_splits > 1 && (long)max_splits * N > (long)N + kSplitRows) max_splits /= 2;
        }
        return gemm_plan(N, H, K, elt, max_splits, true, false);
    };
    const GemmPlan plan_ao = plan_for(H), plan_fo = plan_for(I);
    const int sp_ao = plan_ao.splits, sp_fo = plan_fo.splits;
    // the attn-out / FFN-out GEMMs add the residual stream in their epilogue, so LayerNorm reads one operand
    const bool fuse_res = opt_.fuse_residual;
    // ... and, where the GEMM kernel can, normalise there as well: x32 and its bf16 copy come straight out of
    // the GEMM and the LayerNorm launch disappears.  (Not with split K, whose parts the LayerNorm kernel adds.)
    const bool ln_ao = fuse_res && opt_.fuse_layernorm && sp_ao == 1 && gemm_ln_supported(N, H, H, elt);
    const bool ln_fo = fuse_res && opt_.fuse_layernorm && sp_fo == 1 && gemm_ln_supported(N, H, I, elt);
    void* ln_ws = ln_ws_ + (size_t)part * ln_ws_bytes_;
    if (ln_ao || ln_fo) ln_used_ = std::max(ln_used_, part + 1);

    if (!mark(kPhEmbed)) return false;
    const bool pk = elt == kBF16;           // packed GEMM operands (weights were packed at load)
    if (!launch_embed_layernorm(ids, seg, mask, word_, pos_, type_, emb_g_, emb_b_, x32, xb, pk, maskadd, B, S, Sp,
                                H, D.vocab, D.type_vocab, st, cp))
        return false;
    for (int i = 0; i < D.layers; ++i) {
        const LayerDev& L = layers_[i];
        GemmParams g;
        g.elt = elt;
        // QKV projection, scattered per head (V transposed, unless the attention kernel that follows
        // transposes on its own LDS reads)
        const bool vrow = opt_.v_rowmajor && elt == kBF16 && S <= 512;
        g.X = xin; g.ldx = H; g.W = L.w_qkv; g.bias = L.b_qkv; g.M = N; g.N = 3 * H; g.K = H;
        g.epilogue = kEpiQKV; g.q = q; g.k = k; g.vt = vt; g.S = S; g.Sp = Sp; g.heads = D.heads;
        g.v_rowmajor = vrow;
        g.rowmap = cp ? cp->rowmap : nullptr;
        g.x_packed = g.w_packed = pk;
        if (!mark(kPhQKV) || !launch_gemm(g, st)) return false;
        // The last layer of a pass whose caller gets no sequence output: keys and values are needed of every token,
        // everything after them only of the first token of each sequence, which is all the pooler reads.  Its B rows
        // go through the same kernels as row b * S of the full pass would (K is never split for them, and every
        // kernel treats a row the same whatever else is in the launch), so the pooled output keeps its bits.
        const bool first = first_only_ && i == D.layers - 1 && sp_ao == 1 && sp_fo == 1;
        if (!mark(kPhAttention)) return false;
        if (first) {
            const size_t c0 = (size_t)part * 1024;
            float* xc = xc32_ + c0 * H;
            float* yc = yc32_ + c0 * H;
            bf16_t* xbc = xbc_ ? xbc_ + c0 * H : nullptr;
            unsigned char* ctxc = static_cast<unsigned char*>(ctxc_) + c0 * H * es;
            unsigned char* hc = static_cast<unsigned char*>(hc_) + c0 * I * es;
            const void* xcin = elt == kBF16 ? static_cast<const void*>(xbc) : static_cast<const void*>(xc);
            if (!launch_attention(q, k, vt, maskadd, ctxc, pk, B, D.heads, S, Sp, scale, elt, st, cu, vrow, true, vrow ? cur_attn_ : kAttnAuto)) return false;
            if (!launch_gather_first_rows(x32, cu, xc, B, S, H, st)) return false;
            g = GemmParams();
            g.elt = elt; g.out_elt = kF32; g.X = ctxc; g.ldx = H; g.W = L.w_ao; g.bias = L.b_ao; g.Y = yc;
            g.M = B; g.N = H; g.K = H; g.epilogue = kEpiBias; g.x_packed = g.w_packed = pk;
            g.residual = fuse_res ? xc : nullptr;
            if (!mark(kPhAttnOut) || !launch_gemm(g, st)) return false;
            if (!mark(kPhLayerNorm)) return false;
            if (!launch_add_layernorm(xc, yc, kF32, L.g1, L.be1, xbc, pk, B, H, st, 1, !fuse_res)) return false;
            g = GemmParams();
            g.elt = elt; g.out_elt = elt; g.X = xcin; g.ldx = H; g.W = L.w_in; g.bias = L.b_in; g.Y = hc;
            g.M = B; g.N = I; g.K = H; g.epilogue = kEpiBiasGelu; g.x_packed = g.w_packed = g.y_packed = pk;
            if (!mark(kPhFFNIn) || !launch_gemm(g, st)) return false;
            g = GemmParams();
            g.elt = elt; g.out_elt = kF32; g.X = hc; g.ldx = I; g.W = L.w_out; g.bias = L.b_out; g.Y = yc;
            g.M = B; g.N = H; g.K = I; g.epilogue = kEpiBias; g.x_packed = g.w_packed = pk;
            g.residual = fuse_res ? xc : nullptr;
            if (!mark(kPhFFNOut) || !launch_gemm(g, st)) return false;
            if (!mark(kPhLayerNorm)) return false;
            if (!launch_add_layernorm(xc, yc, kF32, L.g2, L.be2, nullptr, false, B, H, st, 1, !fuse_res)) return false;
            if (!mark(kPhPooler)) return false;
            return launch_pooler(xc, w_pool_, elt, b_pool_, pooled_ + (size_t)b0 * H, B, 1, H, st, nullptr);
        }
        if (!launch_attention(q, k, vt, maskadd, ctx, pk, B, D.heads, S, Sp, scale, elt, st, cu, vrow, false, vrow ? cur_attn_ : kAttnAuto)) return false;
        // attention output projection -> f32, then residual add + LayerNorm
        g = GemmParams();
        g.elt = elt; g.out_elt = kF32; g.X = ctx; g.ldx = H; g.W = L.w_ao; g.bias = L.b_ao; g.Y = y32;
        g.M = N; g.N = H; g.K = H; g.epilogue = kEpiBias; g.x_packed = g.w_packed = pk; g.splits = sp_ao;
        g.residual = fuse_res ? x32 : nullptr;
        g.tile = plan_ao.tile;
        if (ln_ao) { g.tile = 0; g.Y = x32; g.ln_gamma = L.g1; g.ln_beta = L.be1; g.ln_xb = xb; g.ln_xb_packed = pk; g.ln_ws = ln_ws; }
        if (!mark(kPhAttnOut) || !launch_gemm(g, st)) return false;
        if (!mark(kPhLayerNorm)) return false;
        if (!ln_ao && !launch_add_layernorm(x32, y32, kF32, L.g1, L.be1, xb, pk, N, H, st, sp_ao, !fuse_res)) return false;
        // feed-forward
        g = GemmParams();
        g.elt = elt; g.out_elt = elt; g.X = xin; g.ldx = H; g.W = L.w_in; g.bias = L.b_in; g.Y = h;
        g.M = N; g.N = I; g.K = H; g.epilogue = kEpiBiasGelu; g.x_packed = g.w_packed = g.y_packed = pk;
        if (!mark(kPhFFNIn) || !launch_gemm(g, st)) return false;
        g = GemmParams();
        g.elt = elt; g.out_elt = kF32; g.X = h; g.ldx = I; g.W = L.w_out; g.bias = L.b_out; g.Y = y32;
        g.M = N; g.N = H; g.K = I; g.epilogue = kEpiBias; g.x_packed = g.w_packed = pk; g.splits = sp_fo;
        g.residual = fuse_res ? x32 : nullptr;
        g.tile = plan_fo.tile;
        if (ln_fo) { g.tile = 0; g.Y = x32; g.ln_gamma = L.g2; g.ln_beta = L.be2; g.ln_xb = xb; g.ln_xb_packed = pk; g.ln_ws = ln_ws; }
        if (!mark(kPhFFNOut) || !launch_gemm(g, st)) return false;
        if (!mark(kPhLayerNorm)) return false;
        if (!ln_fo && !launch_add_layernorm(x32, y32, kF32, L.g2, L.be2, xb, pk, N, H, st, sp_fo, !fuse_res)) return false;
    }
    // pooler: first-token gather + dense + tanh on the float32 sequence output
    if (!mark(kPhPooler)) return false;
    if (!launch_pooler(x32, w_pool_, elt, b_pool_, pooled_ + (size_t)b0 * H, B, S, H, st, cu)) return false;
    // unpadded pass: the caller still gets a padded [B, S, H] sequence output
    return cp ? launch_unpad_rows(x32, cu, seqpad_ + t0 * H, B, S, H, st) : true;
}

bool Model::mark(int phase) {
    if (!profiling_) return true;
    if (prof_used_ == prof_events_.size()) {
        hipEvent_t e;
        CUBERT_HIP_OK(hipEventCreate(&e));
        prof_events_.push_back(e);
    }
    CUBERT_HIP_OK(hipEventRecord(prof_events_[prof_used_], stream_));
    if (phase >= 0) prof_phase_.push_back(phase);
    ++prof_used_;
    return true;
}

bool Model::profile_device(const int* d_ids, const int* d_seg, const int* d_mask, int B, int S, float* phase_ms) {
    if (!phase_ms) { set_error("profile: null output"); return false; }
    if (!check_shape(B, S)) return false;
    if (!d_ids || !d_seg) { set_error("input_ids and token_type_ids must not be null"); return false; }
    const size_t n = (size_t)B * S, cap = (size_t)cap_tokens_;
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_, d_ids, n * 4, hipMemcpyDeviceToDevice, stream_));
    CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + cap, d_seg, n * 4, hipMemcpyDeviceToDevice, stream_));
    if (d_mask) CUBERT_HIP_OK(hipMemcpyAsync(d_in_ + 2 * cap, d_mask, n * 4, hipMemcpyDeviceToDevice, stream_));
    B_ = B;
    S_ = S;
    first_only_ = false;
    last_compact_ = false;
    last_has_mask_ = d_mask != nullptr;
    last_classified_ = false;
    profiling_ = true;
    prof_used_ = 0;
    prof_phase_.clear();
    bool ok = enqueue(B, S, d_mask != nullptr);
    ok = ok && mark(-1);                       // closing event
    profiling_ = false;
    if (!ok) return false;
    if (!sync()) return false;
    for (int i = 0; i < kNumPhases; ++i) phase_ms[i] = 0.0f;
    for (size_t i = 0; i + 1 < prof_used_; ++i) {
        float ms = 0.0f;
        CUBERT_HIP_OK(hipEventElapsedTime(&ms, prof_events_[i], prof_events_[i + 1]));
        phase_ms[prof_phase_[i]] += ms;
    }
    return true;
}

bool Model::classify() {
    if (!num_classes_) { set_error("the weight directory holds no classifier_kernel / classifier_bias"); return false; }
    if (B_ <= 0) { set_error("classify() needs a preceding forward pass"); return false; }
    last_classified_ = true;
    return launch_classifier(pooled_, w_cls_, b_cls_, cls_, B_, opt_.dims.hidden, num_classes_, stream_);
}

// The last pass once more, launch by launch, from the inputs (and, for an unpadded pass, the lengths) it left behind.
bool Model::rerun_last() {
    const bool classified = last_classified_;
    bool ok;
    if (last_compact_) {
        ok = run_compact(last_lens_.data(), B_, S_);
    } else {
        last_classified_ = false;
        ok = enqueue(B_, S_, last_has_mask_);
    }
    return ok && (!classified || classify());
}

bool Model::sync() {
    CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    recovered_ = false;
    if (ln_used_ > 0) {
        // A workgroup of a GEMM that normalises in its epilogue gives up after a bounded wait for its
        // partners and raises word 0 of its workspace; the results of that pass are then not valid.
        // Every used part is looked at (and put back to zero) before anything else happens.
        const int parts = ln_used_;
        ln_used_ = 0;
        bool raised = false;
        for (int i = 0; i < parts; ++i) {
            int flag = 0;
            CUBERT_HIP_OK(hipMemcpy(&flag, ln_ws_ + (size_t)i * ln_ws_bytes_, sizeof(int), hipMemcpyDeviceToHost));
            if (flag != 0) {
                CUBERT_HIP_OK(hipMemset(ln_ws_ + (size_t)i * ln_ws_bytes_, 0, ln_ws_bytes_));
                raised = true;
            }
        }
        if (raised) {
            // Nothing is lost: the inputs of the pass are still on the device.  The pass is repeated with the
            // LayerNorms as kernels of their own (which wait for nobody), this model keeps them that way, and
            // the graphs captured with the fused kernels go.
            opt_.fuse_layernorm = false;
            ++ln_fallbacks_;
            if (!evict_graphs(0)) return false;
            graphs_.clear();
            if (!rerun_last()) return false;
            CUBERT_HIP_OK(hipStreamSynchronize(stream_));
            recovered_ = true;
        }
    }
    return true;
}

bool Model::copy_out(float* out, const float* dev, size_t floats) {
    CUBERT_HIP_OK(hipMemcpyAsync(out, dev, floats * 4, hipMemcpyDeviceToHost, stream_));
    if (!sync()) return false;
    if (recovered_) {       // the copy above ran before the pass was repeated
        CUBERT_HIP_OK(hipMemcpyAsync(out, dev, floats * 4, hipMemcpyDeviceToHost, stream_));
        CUBERT_HIP_OK(hipStreamSynchronize(stream_));
    }
    return true;
}

bool Model::copy_pooled(float* out) {
    if (!out || B_ <= 0) { set_error("no result to copy"); return false; }
    return copy_out(out, pooled_, (size_t)B_ * opt_.dims.hidden);
}

bool Model::copy_seq(float* out) {
    if (!out || B_ <= 0) { set_error("no result to copy"); return false; }
    return copy_out(out, seq_ptr(), (size_t)B_ * S_ * opt_.dims.hidden);
}

bool Model::copy_cls(float* out) {
    if (!out || B_ <= 0 || !num_classes_) { set_error("no result to copy"); return false; }
    return copy_out(out, cls_, (size_t)B_ * num_classes_);
}

}  // namespace cubert
