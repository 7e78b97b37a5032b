"""The allocation-free split-K GEMM (cubert_op_gemm_splitk_noalloc) against the existing entry
point it is a variant of: cubert_op_gemm with CUBERT_SPLITS(n), whose caller brings the buffer
for the partial sums and adds them up itself.  Same kernels, same summation order: bit-exact.
Two calls in a row share the built-in scratch array; the second one is smaller."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F32, BF16 = 0, 1


@pytest.fixture(scope="module")
def pb():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from cudabert_amd import pybert
    return pybert


def run_pair(pb, elt, M, N, K, splits, seed):
    rng = np.random.default_rng(seed)
    tdt = torch.bfloat16 if elt == BF16 else torch.float32
    X = torch.from_numpy(rng.standard_normal((M, K), dtype=np.float32)).to(tdt).cuda()
    Wt = torch.from_numpy(rng.standard_normal((N, K), dtype=np.float32) * 0.05).to(tdt).cuda()
    bias = torch.from_numpy(rng.standard_normal(N, dtype=np.float32)).cuda()
    st = torch.cuda.current_stream().cuda_stream
    # existing entry point: the caller's buffer takes the parts
    parts = torch.full((splits, M, N), float("nan"), device="cuda")
    pb.check(pb.lib.cubert_op_gemm(X.data_ptr(), Wt.data_ptr(), bias.data_ptr(), parts.data_ptr(), M, N, K, K, elt, F32,
                                   0, 0, (splits & 0xff) << 8, st))
    # allocation-free variant
    Y = torch.full((M + 1, N), float("nan"), device="cuda")        # one guard row
    pb.check(pb.lib.cubert_op_gemm_splitk_noalloc(X.data_ptr(), Wt.data_ptr(), bias.data_ptr(), Y.data_ptr(), M, N, K, K,
                                                  elt, splits, 0, 0, st))
    torch.cuda.synchronize()
    p = parts.cpu().numpy()
    want = p[0].copy()
    for z in range(1, splits):
        want = want + p[z]                 # float32 adds in the kernel's order
    got = Y.cpu().numpy()
    assert np.isnan(got[M]).all()
    assert np.array_equal(got[:M], want), (M, N, K, splits, np.abs(got[:M] - want).max())
    ref = X.float().cpu().numpy().astype(np.float64) @ Wt.float().cpu().numpy().astype(np.float64).T + bias.cpu().numpy()
    assert np.abs(got[:M] - ref).max() < 2e-3 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("elt", [BF16, F32])
def test_noalloc_split_k_gemm_two_calls_in_a_row(pb, elt):
    assert pb.lib.cubert_noalloc_scratch_bytes() == 16 << 20
    run_pair(pb, elt, 1600, 1024, 4096, 2, 1)       # batch 8 x seq 200: FFN-out of the latency regime
    run_pair(pb, elt, 200, 1024, 1024, 4, 2)        # smaller, more parts: stale partial sums must not show
    run_pair(pb, elt, 77, 128, 512, 2, 3)


def test_noalloc_refuses_what_does_not_fit(pb):
    x = torch.zeros(16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    rc = pb.lib.cubert_op_gemm_splitk_noalloc(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 25600, 1024, 4096,
                                              4096, BF16, 2, 0, 0, st)
    assert rc != 0 and "scratch" in pb.last_error()
    rc = pb.lib.cubert_op_gemm_splitk_noalloc(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 64, 64, 64, 64,
                                              BF16, 17, 0, 0, st)
    assert rc != 0 and "splits" in pb.last_error()


def test_noalloc_split_k_gemm_inside_a_captured_graph(pb):
    """What the entry point is for: two calls recorded into one hipGraph (after an eager call that looks the scratch
    address up), replayed several times with eager work in between; every replay gives the eager bits."""
    rng = np.random.default_rng(7)
    shapes = [(1600, 1024, 1024, 2), (200, 1024, 4096, 8)]
    ops = []
    for M, N, K, splits in shapes:
        X = torch.from_numpy(rng.standard_normal((M, K), dtype=np.float32)).to(torch.bfloat16).cuda()
        Wt = torch.from_numpy(rng.standard_normal((N, K), dtype=np.float32) * 0.05).to(torch.bfloat16).cuda()
        bias = torch.from_numpy(rng.standard_normal(N, dtype=np.float32)).cuda()
        ops.append((X, Wt, bias, torch.empty((M, N), device="cuda"), M, N, K, splits))

    def enqueue(st):
        for X, Wt, bias, Y, M, N, K, splits in ops:
            pb.check(pb.lib.cubert_op_gemm_splitk_noalloc(X.data_ptr(), Wt.data_ptr(), bias.data_ptr(), Y.data_ptr(), M, N, K, K,
                                                          BF16, splits, 0, 0, st))

    enqueue(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager = [op[3].clone() for op in ops]
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        g.capture_begin()
        enqueue(side.cuda_stream)
        g.capture_end()
    for rep in range(3):
        for op in ops:
            op[3].fill_(float("nan"))
        run_pair(pb, BF16, 77, 128, 512, 2, 10 + rep)      # eager work on the shared scratch between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for op, want in zip(ops, eager):
            assert torch.equal(op[3], want), rep
