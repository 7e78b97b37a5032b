"""The benchmark configurations at their full size, through the C ABI, against the CPU oracle.

Configuration 0 (BERT-base b8 s128) and the bf16 half of configuration 2 (BERT-large b128
s200) are in test_gpu_model.py; this file holds configuration 1 (BERT-base b128 s128, both
precisions), configuration 2 in float32, configuration 3 (BERT-large, batch 1 and 8, s200,
all valid, replayed from a hipGraph, with and without split K) and configuration 4
(BERT-large b64 s512, skewed lengths), plus what a bf16 run of an unrounded float32
checkpoint agrees to.

Tolerances: max-abs 1e-3 (float32 operands) and 3e-2 (bfloat16 operands) on the sequence and
the pooled output.  The bf16 figure is asserted with both sides holding the same weights
(Linear kernels made bfloat16-representable); RAW_BF16_TOL is the measured bound when the
engine has to round an arbitrary float32 checkpoint to bfloat16 storage first.
"""
import ctypes

import numpy as np
import pytest
import torch

from cudabert_amd import synth
from cudabert_amd import weights as W
from oracle import bert_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16 = 0, 1
TOL = {F32: 1e-3, BF16: 3e-2}
# bf16 mode on a float32 checkpoint whose weights are NOT bfloat16-representable, against the
# float32 oracle on the unrounded weights: (sequence output, pooled output).  Rounding the
# Linear kernels to 8 mantissa bits perturbs every layer's output by about 2^-9 relative,
# whatever the engine does afterwards.  Measured on MI355X: BERT-base (12 layers) 0.024 / 0.010,
# inside the 3e-2 tolerance; BERT-large (24 layers) 0.036 / 0.015 on the first four sequences of
# configuration 2, of which 0.017 / 0.009 is the engine's own arithmetic (the second assert of
# the test) -- the sequence output of the 24-layer model is the one figure that 3e-2 does not
# cover when the storage rounding is counted in, and it is held to 5e-2 here.
RAW_BF16_TOL = {"base": (3e-2, 3e-2), "large": (5e-2, 3e-2)}


@pytest.fixture(scope="module")
def pb():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from cudabert_amd import pybert
    return pybert


def load(pb, dims, wdir, precision, maxB, maxS, graph=0):
    return pb.load_model_ex(wdir, dims.hidden, dims.layers, dims.heads, dims.inter, precision=precision,
                            max_batchsize=maxB, max_seq_length=maxS, graph_max_tokens=graph)


def err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - b).max())


def device_results(pb, m, B, S, H):
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    pooled = np.empty((B, H), np.float32)
    seq = np.empty((B, S, H), np.float32)
    pb.check(pb.lib.cubert_sync(m))
    assert hip.hipMemcpy(pooled.ctypes.data, pb.lib.cubert_pooled_ptr(m), pooled.nbytes, 2) == 0
    assert hip.hipMemcpy(seq.ctypes.data, pb.lib.cubert_seq_ptr(m), seq.nbytes, 2) == 0
    return pooled, seq


# ------------------------------------------------------------------ configuration 1 ----

@pytest.mark.parametrize("precision", [F32, BF16])
def test_cfg1_base_b128_s128_full_batch(pb, base_ckpt, precision):
    """BERT-base, batch 128, seq 128, lengths U[64, 128], padding pruned to the batch maximum."""
    exact = precision == BF16
    ids, seg, mask = synth.config_inputs(1)
    B, S = ids.shape
    assert B == 128 and S <= 128
    m = load(pb, W.BASE, base_ckpt.dir(exact), precision, B, S)
    try:
        pooled, seq, cls = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
        probs_only = np.zeros((B, 2), np.float32)           # pooled-only call (last layer for the first tokens only)
        pb.classify(m, probs_only, ids, seg, B, S, 2, mask)
    finally:
        pb.unload_model(m)
    assert np.array_equal(probs_only, cls)
    n = 4
    npy = base_ckpt.npy(exact)
    seq_ref, pooled_ref = O.forward_torch(npy, W.BASE.heads, ids[:n], seg[:n], mask[:n])
    print("cfg1 precision %d max-abs: seq %.3g pooled %.3g" % (precision, err(seq[:n], seq_ref), err(pooled[:n], pooled_ref)))
    assert err(seq[:n], seq_ref) < TOL[precision]
    assert err(pooled[:n], pooled_ref) < TOL[precision]
    assert err(cls[:n], O.classifier_head(npy, pooled_ref)) < TOL[precision]
    assert np.isfinite(seq).all() and np.isfinite(pooled).all()
    assert np.allclose(cls.sum(1), 1.0, atol=1e-5)


# ------------------------------------------------------------------ configuration 2 ----

def test_cfg2_large_b128_s200_fp32(pb, large_ckpt):
    """The headline shape in the reference's own arithmetic (float32 operands)."""
    D = W.LARGE
    ids, seg, mask = synth.config_inputs(2)
    B, S = ids.shape
    m = load(pb, D, large_ckpt.raw, F32, B, S)
    try:
        pooled, seq, cls = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
    finally:
        pb.unload_model(m)
    n = 3
    seq_ref, pooled_ref = O.forward_torch(large_ckpt.npy_raw, D.heads, ids[:n], seg[:n], mask[:n])
    print("cfg2 fp32 max-abs: seq %.3g pooled %.3g" % (err(seq[:n], seq_ref), err(pooled[:n], pooled_ref)))
    assert err(seq[:n], seq_ref) < TOL[F32]
    assert err(pooled[:n], pooled_ref) < TOL[F32]
    assert err(cls[:n], O.classifier_head(large_ckpt.npy_raw, pooled_ref)) < TOL[F32]
    assert np.isfinite(seq).all()


@pytest.mark.parametrize("which", ["base", "large"])
def test_bf16_mode_on_an_unrounded_fp32_checkpoint(pb, base_ckpt, large_ckpt, which):
    """bf16 mode fed the raw seeded float32 checkpoint (what bench.py runs), against the float32
    oracle on the same unrounded weights: configuration 0 (BERT-base) and the first sequences
    of configuration 2 (BERT-large).  Both sides hold 'the same seeded weights', but the engine
    stores its Linear kernels in bfloat16, so this error contains the storage rounding as well;
    the engine's own arithmetic is held to 3e-2 by the tests on bfloat16-representable weights."""
    ck, D, cfg, n = (base_ckpt, W.BASE, 0, 8) if which == "base" else (large_ckpt, W.LARGE, 2, 4)
    ids, seg, mask = synth.config_inputs(cfg)
    B, S = ids.shape
    m = load(pb, D, ck.raw, BF16, B, S)
    try:
        pooled, seq, _ = pb.encode(m, ids, seg, mask, want_seq=True)
        pooled_only = np.ones((B, D.hidden), np.float32)    # Cuda_Bert on the same batch (cfg2: two stream parts, unpadded)
        pb.bert(m, pooled_only, ids, seg, B, S, mask)
    finally:
        pb.unload_model(m)
    if which == "large":        # (the short batch of configuration 0 splits K by its row count, which differs between the two calls)
        assert np.array_equal(pooled_only, pooled)
    seq_ref, pooled_ref = O.forward_torch(ck.npy_raw, D.heads, ids[:n], seg[:n], mask[:n])
    e_seq, e_pool = err(seq[:n], seq_ref), err(pooled[:n], pooled_ref)
    rms = float(np.sqrt(np.mean((seq[:n] - seq_ref) ** 2)))
    print("bf16 on the raw %s checkpoint: max-abs seq %.4g pooled %.4g, rms seq %.4g" % (which, e_seq, e_pool, rms))
    assert e_seq < RAW_BF16_TOL[which][0] and e_pool < RAW_BF16_TOL[which][1]
    # the same run against the float32 model on the ROUNDED weights: the engine's own share
    seq_x, pooled_x = O.forward_torch(ck.npy_bf16x, D.heads, ids[:n], seg[:n], mask[:n])
    print("   against the oracle on bf16-representable weights: seq %.4g pooled %.4g" % (err(seq[:n], seq_x), err(pooled[:n], pooled_x)))
    assert err(seq[:n], seq_x) < TOL[BF16] and err(pooled[:n], pooled_x) < TOL[BF16]


# ------------------------------------------------------------------ configuration 3 ----

def test_cfg3_large_latency_regime_graph_and_split_k(pb, large_ckpt, monkeypatch):
    """BERT-large, batch 1 and batch 8, seq 200, every position valid, bf16: the first call runs
    eagerly, the second captures the whole pass into a hipGraph, later calls replay it.  The
    hidden-wide GEMMs split K and the LayerNorm after them adds the partial sums; the same
    batches with CUBERT_SPLIT_K=0 must agree within tolerance."""
    D = W.LARGE
    S = 200
    npy = large_ckpt.npy_bf16x
    m = load(pb, D, large_ckpt.bf16x, BF16, 8, S, graph=8192)
    monkeypatch.setenv("CUBERT_SPLIT_K", "0")
    m_nosplit = load(pb, D, large_ckpt.bf16x, BF16, 8, S, graph=8192)
    try:
        for B in (1, 8):
            ids, seg, mask = synth.make_inputs(B, S, [S] * B, seed=20244 + B)
            seq_ref, pooled_ref = O.forward_torch(npy, D.heads, ids, seg, mask)
            first = None
            for call in range(4):          # eager, capture + launch, replay, replay
                pooled, seq, cls = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
                assert err(seq, seq_ref) < TOL[BF16], (B, call, err(seq, seq_ref))
                assert err(pooled, pooled_ref) < TOL[BF16], (B, call)
                assert err(cls, O.classifier_head(npy, pooled_ref)) < TOL[BF16]
                if first is None:
                    first = (pooled, seq)
                    print("cfg3 B=%d max-abs: seq %.3g pooled %.3g" % (B, err(seq, seq_ref), err(pooled, pooled_ref)))
                else:                       # a replay runs the same kernels on the same addresses
                    assert np.array_equal(pooled, first[0]) and np.array_equal(seq, first[1]), (B, call)
            assert pb.lib.cubert_graphs_cached(m) == (1 if B == 1 else 2)
            for call in range(3):
                pooled0, seq0, _ = pb.encode(m_nosplit, ids, seg, mask, want_seq=True)
            assert err(seq0, seq_ref) < TOL[BF16] and err(pooled0, pooled_ref) < TOL[BF16]
            # Split K only regroups float32 sums, but one flipped bfloat16 rounding early on sends the
            # rest of the pass down another rounding path: two bf16 runs agree with each other no
            # better than each of them agrees with the oracle.
            print("cfg3 B=%d split K on vs off: seq %.3g pooled %.3g" % (B, err(seq0, first[1]), err(pooled0, first[0])))
            assert err(seq0, first[1]) < TOL[BF16] and err(pooled0, first[0]) < TOL[BF16], (B, err(seq0, first[1]))
        assert pb.lib.cubert_graphs_cached(m_nosplit) == 2
    finally:
        pb.unload_model(m)
        pb.unload_model(m_nosplit)


def test_layernorm_in_gemm_epilogue_inside_a_captured_graph(pb, base_ckpt):
    """A batch just below the hipGraph limit (32 x 200 = 6400 tokens) is large enough for the GEMMs that
    normalise in their epilogue: their workgroups count themselves in and out on words of a workspace that
    every launch has to leave at zero, replays of the captured graph included.  Eager, capture, replays: the
    same bits each time, the first sequences within tolerance of the oracle."""
    D = W.BASE
    B, S = 32, 200
    lens = np.random.default_rng(3).integers(60, S + 1, size=B)
    lens[0] = S
    ids, seg, mask = synth.make_inputs(B, S, list(lens), seed=77)
    m = load(pb, D, base_ckpt.bf16x, BF16, B, S, graph=8192)
    try:
        first = None
        for call in range(5):
            pooled, seq, _ = pb.encode(m, ids, seg, mask, want_seq=True)
            if first is None:
                first = (pooled, seq)
            else:
                assert np.array_equal(pooled, first[0]) and np.array_equal(seq, first[1]), call
        assert pb.lib.cubert_graphs_cached(m) == 1
    finally:
        pb.unload_model(m)
    n = 2
    seq_ref, pooled_ref = O.forward_torch(base_ckpt.npy_bf16x, D.heads, ids[:n], seg[:n], mask[:n])
    assert err(first[1][:n], seq_ref) < TOL[BF16] and err(first[0][:n], pooled_ref) < TOL[BF16]


def test_layernorm_epilogue_timeout_is_recovered_not_fatal(pb, base_ckpt, monkeypatch):
    """The workgroups of a GEMM that normalises in its epilogue wait for their partners for a bounded time.  When that
    wait expires (forced here from the host: band 0 can never complete and the poll limit is one; every kernel still
    ends normally), the next synchronising call repeats the pass with separate LayerNorm kernels, keeps the model on
    them and counts it; the caller gets the bits of a model that never fused.  Seen on an eager pass and on the replay
    of a captured graph (whose launch never passes through the code that enqueues kernels)."""
    D = W.BASE
    B, S = 33, 200
    lens = np.random.default_rng(5).integers(190, S + 1, size=B)       # >= 6144 valid tokens: the unpadded pass fuses too
    lens[0] = S
    ids, seg, mask = synth.make_inputs(B, S, list(lens), seed=78)
    monkeypatch.setenv("CUBERT_FUSE_LAYERNORM", "0")
    m = load(pb, D, base_ckpt.bf16x, BF16, B, S, graph=0)
    try:
        want = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
        assert pb.lib.cubert_ln_fallbacks(m) == 0
    finally:
        pb.unload_model(m)
    monkeypatch.delenv("CUBERT_FUSE_LAYERNORM")

    def same(got):
        return all(np.array_equal(a, b) for a, b in zip(got, want))

    for graph, warm in ((0, 1), (8192, 3)):        # 3 calls: eager, capture, replay
        m = load(pb, D, base_ckpt.bf16x, BF16, B, S, graph=graph)
        try:
            for _ in range(warm):
                assert same(pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True))       # fused: the same bits anyway
            assert pb.lib.cubert_ln_fallbacks(m) == 0 and pb.lib.cubert_graphs_cached(m) == (1 if graph else 0)
            pb.check(pb.lib.cubert_debug_force_ln_timeout(m))
            assert same(pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)), graph
            assert pb.lib.cubert_ln_fallbacks(m) == 1
            assert pb.lib.cubert_graphs_cached(m) == 0          # graphs with the fused kernels are gone
            for _ in range(3):                                   # and the model carries on (capturing anew)
                assert same(pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True))
            assert pb.lib.cubert_ln_fallbacks(m) == 1
            # pooled-only host call: takes the unpadded pass, which is repeated the same way
            out = np.zeros((B, D.hidden), np.float32)
            pb.bert(m, out, ids, seg, B, S, mask)
            assert np.array_equal(out, want[0])
        finally:
            pb.unload_model(m)
    # the unpadded pass (two stream parts above 14336 rows; here one) times out and is repeated too
    monkeypatch.setenv("CUBERT_VARLEN", "1")
    m = load(pb, D, base_ckpt.bf16x, BF16, B, S, graph=0)
    try:
        pb.check(pb.lib.cubert_debug_force_ln_timeout(m))
        pooled, seq, cls = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
        valid = mask.astype(bool)
        assert pb.lib.cubert_ln_fallbacks(m) == 1
        assert np.array_equal(pooled, want[0]) and np.array_equal(cls, want[2]) and np.array_equal(seq[valid], want[1][valid])
    finally:
        pb.unload_model(m)


# ------------------------------------------------------------------ configuration 4 ----

def test_cfg4_large_b64_s512_skewed(pb, large_ckpt):
    """BERT-large, batch 64, seq 512, 70 % short / 30 % long sequences, bf16: the attention kernel
    with 1024-thread workgroups and the whole head in LDS over 24 layers.  The longest and the
    shortest sequence against the oracle (padded and unpadded pass), and the size-independent
    properties on the full batch."""
    D = W.LARGE
    npy = large_ckpt.npy_bf16x
    ids, seg, mask = synth.config_inputs(4)
    B, S = ids.shape
    lens = np.ascontiguousarray(mask.sum(1).astype(np.int32))
    assert B == 64 and S > 384 and lens.min() <= 128
    m = load(pb, D, large_ckpt.bf16x, BF16, B, S)
    try:
        pooled, seq, cls = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
        perm = np.random.default_rng(4).permutation(B)
        pooled_p, seq_p, _ = pb.encode(m, ids[perm], seg[perm], mask[perm], want_seq=True)
        d = [torch.from_numpy(a).cuda() for a in (ids, seg)]
        torch.cuda.synchronize()
        pb.check(pb.lib.cubert_forward_device_lens(m, d[0].data_ptr(), d[1].data_ptr(), lens.ctypes.data, B, S))
        pooled_u, seq_u = device_results(pb, m, B, S, D.hidden)
        # pooled-only host call: valid tokens only, last layer for the first tokens only -- the same bits
        pooled_only = np.ones((B, D.hidden), np.float32)
        pb.bert(m, pooled_only, ids, seg, B, S, mask)
    finally:
        pb.unload_model(m)
    assert np.array_equal(pooled_only, pooled)
    assert np.isfinite(seq).all() and np.allclose(cls.sum(1), 1.0, atol=1e-5)
    assert np.array_equal(pooled_p, pooled[perm]) and np.array_equal(seq_p, seq[perm])
    valid = mask.astype(bool)
    assert np.array_equal(pooled_u, pooled)
    assert np.array_equal(seq_u[valid], seq[valid]) and (seq_u[~valid] == 0).all()
    rows = [int(lens.argmax()), int(lens.argmin())]
    seq_ref, pooled_ref = O.forward_torch(npy, D.heads, ids[rows], seg[rows], mask[rows])
    print("cfg4 rows %s (lengths %s) max-abs: seq %.3g pooled %.3g" % (rows, lens[rows], err(seq[rows], seq_ref), err(pooled[rows], pooled_ref)))
    assert err(seq[rows], seq_ref) < TOL[BF16] and err(pooled[rows], pooled_ref) < TOL[BF16]
    assert err(cls[rows], O.classifier_head(npy, pooled_ref)) < TOL[BF16]
    # the unpadded pass directly against the oracle, on the positions it computes
    for i, r in enumerate(rows):
        assert err(seq_u[r, :lens[r]], seq_ref[i, :lens[r]]) < TOL[BF16]
    assert err(pooled_u[rows], pooled_ref) < TOL[BF16]


# ------------------------------------------------- unpadded pass against the oracle ----

@pytest.mark.parametrize("precision", [F32, BF16])
def test_unpadded_pass_against_the_oracle(pb, tmp_path, precision):
    """cubert_forward_device_lens computes only the valid tokens; what it returns is compared with
    the oracle itself (not with the padded pass): valid positions and pooled output within
    tolerance, padding positions zero."""
    D = W.TINY
    state = W.bf16_representable(W.synth_state(D, seed=11, degenerate=False))
    wdir = W.export_npy_dir(state, str(tmp_path / "w"))
    npy = W.to_npy_layout(state)
    B, S = 6, 61
    lens = np.array([61, 1, 32, 33, 7, 60], np.int32)
    ids, seg, mask = synth.make_inputs(B, S, list(lens), vocab=D.vocab, seed=12, prune=False)
    seq_ref, pooled_ref = O.forward_torch(npy, D.heads, ids, seg, mask)
    m = load(pb, D, wdir, precision, B, S)
    try:
        d = [torch.from_numpy(a).cuda() for a in (ids, seg)]
        torch.cuda.synchronize()
        for _ in range(2):
            pb.check(pb.lib.cubert_forward_device_lens(m, d[0].data_ptr(), d[1].data_ptr(), lens.ctypes.data, B, S))
            pooled, seq = device_results(pb, m, B, S, D.hidden)
            valid = mask.astype(bool)
            assert err(seq[valid], seq_ref[valid]) < TOL[precision]
            assert err(pooled, pooled_ref) < TOL[precision]
            assert (seq[~valid] == 0).all()
    finally:
        pb.unload_model(m)


def test_pooled_only_host_calls_compute_valid_tokens_only(pb, tmp_path, monkeypatch):
    """Cuda_Bert / Cuda_Classify return no sequence output, so on a ragged batch they take the
    unpadded pass by themselves; what they return equals the padded pass bit for bit.  A call
    that asks for the sequence output stays on the padded pass (values on the padding positions
    as the PyTorch model defines them)."""
    D = W.TINY
    state = W.bf16_representable(W.synth_state(D, seed=21, degenerate=False))
    wdir = W.export_npy_dir(state, str(tmp_path / "w"))
    npy = W.to_npy_layout(state)
    B, S = 5, 40
    ids, seg, mask = synth.make_inputs(B, S, [40, 3, 17, 1, 22], vocab=D.vocab, seed=3, prune=False)
    seq_ref, pooled_ref = O.forward_torch(npy, D.heads, ids, seg, mask)
    monkeypatch.setenv("CUBERT_SPLIT_K", "0")      # split K would group the sums by the row count
    monkeypatch.setenv("CUBERT_FIRST_TOKEN_LAST_LAYER", "0")     # this test reads the sequence buffer such calls leave behind
    for precision in (F32, BF16):
        m = load(pb, D, wdir, precision, B, S)
        try:
            pooled_full, seq_full, cls_full = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
            assert err(seq_full, seq_ref) < TOL[precision]          # padded pass: every position defined
            out = np.ones((B, D.hidden), np.float32)
            pb.bert(m, out, ids, seg, B, S, mask)
            assert np.array_equal(out, pooled_full)
            # the sequence buffer of that call holds zeros on the padding: the unpadded pass ran
            _, seq_dev = device_results(pb, m, B, S, D.hidden)
            valid = mask.astype(bool)
            assert (seq_dev[~valid] == 0).all() and np.array_equal(seq_dev[valid], seq_full[valid])
            probs = np.zeros((B, 2), np.float32)
            pb.classify(m, probs, ids, seg, B, S, 2, mask)
            assert np.array_equal(probs, cls_full)
            # all-valid batches and masks with holes stay on the padded pass
            holed = mask.copy()
            holed[0, 5] = 0
            pb.bert(m, out, ids, seg, B, S, holed)
            _, seq_dev = device_results(pb, m, B, S, D.hidden)
            assert (seq_dev[~valid] != 0).any()
        finally:
            pb.unload_model(m)


@pytest.mark.parametrize("precision", [F32, BF16])
def test_pooled_only_calls_compute_the_last_layer_for_first_tokens_only(pb, tmp_path, monkeypatch, precision):
    """Cuda_Bert / Cuda_Classify / cubert_encode(seq_out = NULL) hand back [B, hidden] (cuda_bert/cuda_bert.cu:55-70):
    after the last layer's keys and values only the first token of every sequence matters.  Those B rows run through
    the same kernels as row b * S of the full pass, so the results are the full pass's bit for bit: padded pass,
    unpadded pass, eager and replayed from a graph, one stream and two."""
    D = W.TINY
    state = W.bf16_representable(W.synth_state(D, seed=22, degenerate=False))
    wdir = W.export_npy_dir(state, str(tmp_path / "w"))
    B, S = 6, 40
    ids, seg, mask = synth.make_inputs(B, S, [40, 3, 17, 1, 22, 40], vocab=D.vocab, seed=4, prune=False)
    monkeypatch.setenv("CUBERT_SPLIT_K", "0")      # split K would group the sums by the row count
    monkeypatch.setenv("CUBERT_FIRST_TOKEN_LAST_LAYER", "0")
    m = load(pb, D, wdir, precision, B, S)
    try:
        pooled_full, _, cls_full = pb.encode(m, ids, seg, mask, want_seq=True, want_cls=True)
    finally:
        pb.unload_model(m)
    monkeypatch.delenv("CUBERT_FIRST_TOKEN_LAST_LAYER")
    for varlen in ("0", "1"):
        for split_min, graph in (("0", 0), ("1", 0), ("0", 4096), ("1", 4096)):
            monkeypatch.setenv("CUBERT_VARLEN", varlen)
            monkeypatch.setenv("CUBERT_SPLIT_MIN_TOKENS", split_min)
            m = load(pb, D, wdir, precision, B, S, graph=graph)
            try:
                for rep in range(3 if graph else 1):
                    out = np.ones((B, D.hidden), np.float32)
                    pb.bert(m, out, ids, seg, B, S, mask)
                    assert np.array_equal(out, pooled_full), (varlen, split_min, graph, rep)
                    probs = np.zeros((B, 2), np.float32)
                    pb.classify(m, probs, ids, seg, B, S, 2, mask)
                    assert np.array_equal(probs, cls_full)
                    # a call that wants the sequence output in between gets the full pass
                    pooled2, seq2, _ = pb.encode(m, ids, seg, mask, want_seq=True)
                    assert np.array_equal(pooled2, pooled_full) and np.isfinite(seq2).all()
                # no mask at all: every position valid
                out2, _, _ = pb.encode(m, ids, seg, None)          # seq_out == NULL: a pooled-only call
                pooled3, _, _ = pb.encode(m, ids, seg, None, want_seq=True)
                assert np.array_equal(out2, pooled3)
            finally:
                pb.unload_model(m)


# ------------------------------------------------------------------ hipGraph cache ----

def test_graph_cache_keeps_shapes_apart_beyond_1024_positions(pb, tmp_path):
    """(B=1, S=1500) and (B=2, S=476) must not share a captured graph (a key of the form
    (B * 1024 + S) would give both the same slot)."""
    D = W.BertDims(hidden=128, layers=2, heads=2, inter=512, vocab=97, max_pos=1536)
    state = W.synth_state(D, seed=5, degenerate=False)
    wdir = W.export_npy_dir(state, str(tmp_path / "w"))
    npy = W.to_npy_layout(state)
    m = load(pb, D, wdir, F32, 2, 1500, graph=4096)
    try:
        cases = []
        for B, S in ((1, 1500), (2, 476)):
            ids, seg, mask = synth.make_inputs(B, S, [S - 3 * b for b in range(B)], vocab=D.vocab, seed=S, prune=False)
            cases.append((ids, seg, mask) + O.forward_torch(npy, D.heads, ids, seg, mask))
        for rep in range(3):              # eager, capture, replay -- alternating between the shapes
            for ids, seg, mask, seq_ref, pooled_ref in cases:
                pooled, seq, _ = pb.encode(m, ids, seg, mask, want_seq=True)
                assert err(seq, seq_ref) < TOL[F32], (rep, ids.shape)
                assert err(pooled, pooled_ref) < TOL[F32], (rep, ids.shape)
        assert pb.lib.cubert_graphs_cached(m) == 2
    finally:
        pb.unload_model(m)


def test_graph_cache_evicts_least_recently_used(pb, tmp_path, monkeypatch):
    D = W.TINY
    state = W.synth_state(D, seed=6, degenerate=False)
    wdir = W.export_npy_dir(state, str(tmp_path / "w"))
    npy = W.to_npy_layout(state)
    monkeypatch.setenv("CUBERT_GRAPH_CACHE", "2")
    m = load(pb, D, wdir, F32, 4, 64, graph=4096)
    try:
        shapes = [(1, 9), (2, 17), (3, 33), (4, 64)]
        cases = {}
        for B, S in shapes:
            ids, seg, mask = synth.make_inputs(B, S, [S - b for b in range(B)], vocab=D.vocab, seed=B, prune=False)
            cases[(B, S)] = (ids, seg, mask) + O.forward_torch(npy, D.heads, ids, seg, mask)

        def run(shape):
            ids, seg, mask, seq_ref, pooled_ref = cases[shape]
            pooled, seq, _ = pb.encode(m, ids, seg, mask, want_seq=True)
            assert err(seq, seq_ref) < TOL[F32] and err(pooled, pooled_ref) < TOL[F32], shape

        for shape in shapes:              # every shape: eager, capture, replay
            for _ in range(3):
                run(shape)
            assert pb.lib.cubert_graphs_cached(m) <= 2
        assert pb.lib.cubert_graphs_cached(m) == 2
        for shape in shapes + shapes[::-1]:      # evicted shapes come back through eager and capture again
            for _ in range(2):
                run(shape)
        assert pb.lib.cubert_graphs_cached(m) == 2
    finally:
        pb.unload_model(m)


# ------------------------------------------------ the reference's benchmark entry ----

def test_reference_benchmark_entry_point_runs(pb, base_ckpt, tmp_path, monkeypatch, capfd):
    """`test(batchsize, seq_length, nIter, large, num_gpu)` (cuda_bert/cuda_bert.cu:91-180) loads the
    default weight directory relative to the working directory, runs its seed batch and prints the
    99th-percentile latency and the throughput."""
    import os
    os.makedirs(tmp_path / "model_npy")
    os.symlink(base_ckpt.raw, tmp_path / "model_npy" / "base_uncased")
    monkeypatch.chdir(tmp_path)
    pb.lib.test(2, 32, 2, False, 0)
    out = capfd.readouterr().out
    assert " Seq_length : 32" in out and " Batchsize : 2" in out and "Using Base Model" in out
    assert " 99 Latency : " in out and " Throughput: " in out
    vals = [float(x) for x in out.split("unit_test pooled[0][:10]:")[1].splitlines()[0].split()]
    # the seed batch (cuda_bert/cuda_bert.cu:94-103) through the oracle
    ids, seg, mask = pb.seed_batch(2, 32)
    _, pooled_ref = O.forward_torch(base_ckpt.npy_raw, W.BASE.heads, ids, seg, mask)
    assert err(np.array(vals), pooled_ref[0, :10]) < TOL[F32]


# ------------------------------------------------------- odd shapes through every path ----
@pytest.mark.gpu
@pytest.mark.parametrize("B,S", [(90, 161), (70, 100), (128, 60), (33, 199)])
def test_odd_shapes_reach_every_path_against_the_oracle(pb, tmp_path, monkeypatch, B, S):
    """A two-layer model of BERT-base width on batch shapes that are no multiple of any tile: 14 490
    token rows (two streams, LayerNorm in the GEMM epilogue), 7 000 and 7 680 (one stream, fused
    LayerNorm), 6 567 (about 5 400 valid rows: separate LayerNorm kernels in the unpadded pass); ragged
    lengths, one mask with holes; padded and unpadded pass against the float32 oracle, bf16."""
    import dataclasses
    dims = dataclasses.replace(W.BASE, layers=2, vocab=2000, max_pos=512)
    state = W.bf16_representable(W.synth_state(dims, seed=11, degenerate=False))
    W.export_npy_dir(state, str(tmp_path))
    npy = W.load_npy_dir(str(tmp_path))
    rng = np.random.default_rng(B * 1000 + S)
    lens = rng.integers((2 * S) // 3, S + 1, size=B)
    lens[0] = S
    ids, seg, mask = synth.make_inputs(B, S, lens, vocab=dims.vocab, seed=S, prune=False)
    if B % 2 == 0:
        mask[1, 2:5] = 0                       # not a prefix: the unpadded pass must decline and run padded
    seq_ref, pooled_ref = O.forward_torch(npy, dims.heads, ids, seg, mask)
    valid = mask.astype(bool)
    for varlen in ("0", "1"):
        monkeypatch.setenv("CUBERT_VARLEN", varlen)
        m = load(pb, dims, str(tmp_path), BF16, B, S)
        try:
            pooled, seq, _ = pb.encode(m, ids, seg, mask, want_seq=True)
        finally:
            pb.unload_model(m)
        assert np.isfinite(seq).all()
        assert np.abs(seq - seq_ref)[valid].max() < TOL[BF16], (varlen, np.abs(seq - seq_ref)[valid].max())
        assert np.abs(pooled - pooled_ref).max() < TOL[BF16], varlen
