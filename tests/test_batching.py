"""Length-bucketed batching frontend (host logic; the GPU case runs it over the engine)."""
import numpy as np
import pytest

from cudabert_amd import batching as Bt


def test_generate_splits_matches_reference_edges():
    # engine.py:225-232 with the defaults of engine.py:196-198: [0, 50, 52, ..., 180, max_seq_length]
    s = Bt.generate_splits(200)
    assert s[0] == 0 and s[1] == 50 and s[2] == 52 and s[-2] == 180 and s[-1] == 200
    assert len(s) == 1 + 66 + 1
    assert Bt.generate_splits(64, 16, 32, 8) == [0, 16, 24, 32, 64]


def line(i, length, total=40, hole=False):
    mask = np.zeros(total, np.int32)
    mask[:length] = 1
    if hole and length > 2:
        mask[1] = 0                      # the useful length is set by the LAST 1 (utils.py:46-52)
    ids = np.arange(total, dtype=np.int32) + 100 * i
    return Bt.TaggedLine(i, "line%d" % i, ids, mask, np.zeros(total, np.int32))


def test_tagged_line_length_and_trim():
    assert line(0, 7).length == 7
    assert line(0, 7, hole=True).length == 7
    assert Bt.TaggedLine(0, "", [5, 6], [0, 0], [0, 0]).length == 1
    with pytest.raises(ValueError):
        Bt.TaggedLine(0, "", [1, 2, 3], [1, 1], [0, 0])
    ids, seg, mask = Bt.optimize_batch([line(0, 7), line(1, 12), line(2, 3)])
    assert ids.shape == seg.shape == mask.shape == (3, 12) and ids.dtype == np.int32
    assert (ids[1] == np.arange(12) + 100).all() and mask[2].sum() == 3


def test_bucket_routing_and_emission_order():
    qm = Bt.QueueManager([0, 8, 16, 40], batchsize=2)
    for i, n in enumerate([3, 20, 9, 8, 16, 40, 10]):      # buckets: 0,2,1,0,1,2,1
        qm.put(line(i, n))
    # bucket 0 filled by lines 0,3; bucket 1 by 2,4; bucket 2 by 1,5; line 6 waits
    assert qm.ready() == 3
    order = []
    while (b := qm.get()) is not None:
        order.append([l.num_line for l in b.lines_list])
        assert b.tensor[0].shape[1] == max(l.length for l in b.lines_list)
    assert order == [[0, 3], [1, 5], [2, 4]]                 # earliest first line goes first
    qm.force_enqueue()
    assert [l.num_line for l in qm.get().lines_list] == [6]
    assert qm.get() is None
    with pytest.raises(ValueError):
        qm.put(line(9, 41, total=48))


def test_ordered_writer_rejects_duplicates():
    got = []
    w = Bt.OrderedWriter(lambda l: got.append(l.num_line))
    b1 = Bt.BatchPacked([line(1, 3), line(2, 3)], None); b1.set_output([0, 0])
    b0 = Bt.BatchPacked([line(0, 3)], None); b0.set_output([0])
    w.add(b1)
    assert got == [] and w.backlog == 2
    w.add(b0)
    assert got == [0, 1, 2] and w.backlog == 0
    with pytest.raises(RuntimeError):
        w.add(b0)


@pytest.mark.parametrize("alert", [1000000, 5])
def test_engine_every_line_once_in_order(alert):
    rng = np.random.default_rng(3)
    lens = rng.integers(1, 65, size=257)

    def tokenize(max_seq, text, index):
        n = int(text)
        mask = np.zeros(max_seq, np.int32); mask[:n] = 1
        ids = np.zeros(max_seq, np.int32); ids[:n] = index + 1
        return index, text, ids, mask, np.zeros(max_seq, np.int32)

    def encode(t):
        ids, seg, mask = t
        assert ids.shape == seg.shape == mask.shape and ids.shape[0] <= 16
        assert mask[:, -1].max() == 1                         # trimmed to the longest line
        return np.stack([ids[:, 0], mask.sum(1)], 1)         # (line index + 1, length)

    out = []
    eng = Bt.Engine(encode, tokenize, output=lambda data, o: (data, int(o[0]), int(o[1])), max_seq_length=64,
                    batch_size=16, start_split=8, end_split=48, split_size=8, alert_size=alert)
    eng.run((str(n) for n in lens), out.append)
    assert [o[1] for o in out] == list(range(1, 258))
    assert [o[2] for o in out] == [int(n) for n in lens]
    assert [o[0] for o in out] == [str(n) for n in lens]
    assert sum(b for b, _ in eng.batch_shapes) == 257
    if alert == 5:
        assert len(eng.batch_shapes) > 257 // 16 + 7          # the backlog limit forced early, partial batches


@pytest.mark.gpu
def test_engine_over_the_device(tmp_path):
    """The frontend over the real engine: each line's pooled output equals what the oracle gives
    for that line alone (padding and batch mates do not matter), in input order."""
    import torch
    assert torch.cuda.is_available()
    from cudabert_amd import pybert, weights as W
    from oracle import bert_oracle as O
    state = W.synth_state(W.TINY, seed=11, degenerate=False)
    wdir = str(tmp_path / "w")
    W.export_npy_dir(state, wdir)
    npy = W.load_npy_dir(wdir)
    D = W.TINY
    rng = np.random.default_rng(5)
    lens = rng.integers(2, 49, size=41)
    rows = [rng.integers(1, D.vocab, size=n) for n in lens]

    def tokenize(max_seq, text, index):
        n = lens[index]
        ids = np.zeros(max_seq, np.int32); ids[:n] = rows[index]
        mask = np.zeros(max_seq, np.int32); mask[:n] = 1
        seg = np.zeros(max_seq, np.int32); seg[n // 2:n] = 1
        return index, text, ids, mask, seg

    m = pybert.load_model_ex(wdir, D.hidden, D.layers, D.heads, D.inter, precision=0, max_batchsize=8,
                             max_seq_length=48, graph_max_tokens=4096)
    try:
        # twice over the same lines: the second time every (B, S) shape has been seen before, so
        # the engine captures it into a hipGraph and the results come from the captured pass
        for rep in range(2):
            out = []
            eng = Bt.Engine(lambda t: pybert.encode(m, t[0], t[1], t[2])[0], tokenize, max_seq_length=48, batch_size=8,
                            start_split=8, end_split=40, split_size=8)
            eng.run(("x" for _ in lens), out.append)
            assert len(out) == len(lens)
            for i, n in enumerate(lens):
                _, _, ids, mask, seg = tokenize(48, "", i)
                _, pooled_ref = O.forward_torch(npy, D.heads, ids[None, :n], seg[None, :n], mask[None, :n])
                assert np.abs(out[i] - pooled_ref[0]).max() < 1e-3, (rep, i)
        assert pybert.lib.cubert_graphs_cached(m) >= 1         # repeated (B, S) shapes were captured
    finally:
        pybert.unload_model(m)
