"""Host-only checks of the C ABI library: it loads without a GPU, exports every
symbol include/cubert.h declares, and the weight-directory validation (names,
dtypes, shapes) rejects what it should -- all without a compute call."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from cudabert_amd import weights as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def pb():
    from cudabert_amd import pybert
    return pybert


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cubert.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^[ \t]*#.*$", "", text, flags=re.M)          # macros are not symbols
    return sorted(set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", text)))


def test_exports_every_declared_symbol(pb):
    syms = declared_symbols()
    for must in ("init_model", "release_model", "Cuda_Bert", "Cuda_Inference", "test", "cubert_encode",
                 "cubert_op_gemm", "cubert_op_attention", "cubert_op_add_layernorm", "cubert_op_mask_softmax"):
        assert must in syms
    for s in syms:
        assert hasattr(pb.lib, s), s


def test_reference_argtypes(pb):
    # cuda_bert/pybert.py:14-38
    assert pb.init_model.argtypes == [ctypes.c_bool, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_char_p]
    assert pb.init_model.restype is ctypes.c_void_p
    assert len(pb.bert.argtypes) == 7 and len(pb.inference.argtypes) == 6
    assert [f[0] for f in pb.Retval._fields_] == ["tensor", "Pooled_Output"]
    assert ctypes.sizeof(pb.Retval) == 16


@pytest.fixture()
def tiny_dir(tmp_path):
    return W.export_npy_dir(W.synth_state(W.TINY, seed=1, degenerate=False), str(tmp_path / "m"))


T = W.TINY


def chk(pb, d, dims=T):
    pb.check_weight_dir(d, dims.hidden, dims.layers, dims.heads, dims.inter)


def test_valid_dir_accepted(pb, tiny_dir):
    chk(pb, tiny_dir)
    # any file-name prefix works, as with the reference's substring lookup (load_model.cc:15-30)
    for f in os.listdir(tiny_dir):
        if f.startswith("bert_"):
            os.rename(os.path.join(tiny_dir, f), os.path.join(tiny_dir, f[len("bert_"):]))
    chk(pb, tiny_dir)


def test_missing_dir_and_empty_dir(pb, tmp_path):
    with pytest.raises(pb.CubertError, match="cannot open"):
        chk(pb, str(tmp_path / "nope"))
    os.makedirs(tmp_path / "empty")
    with pytest.raises(pb.CubertError, match="no .npy"):
        chk(pb, str(tmp_path / "empty"))


def test_missing_tensor(pb, tiny_dir):
    os.remove(os.path.join(tiny_dir, "bert_encoder_layer_1_output_dense_bias.npy"))
    with pytest.raises(pb.CubertError, match="_1_output_dense_bias"):
        chk(pb, tiny_dir)


def test_wrong_dtype(pb, tiny_dir):
    p = os.path.join(tiny_dir, "bert_pooler_dense_bias.npy")
    np.save(p, np.load(p).astype(np.float64))
    with pytest.raises(pb.CubertError, match="float32"):
        chk(pb, tiny_dir)


def test_wrong_shape_and_orientation(pb, tiny_dir):
    p = os.path.join(tiny_dir, "bert_encoder_layer_0_intermediate_dense_kernel.npy")
    np.save(p, np.ascontiguousarray(np.load(p).T))            # [out,in] instead of [in,out]
    with pytest.raises(pb.CubertError, match="intermediate_dense_kernel"):
        chk(pb, tiny_dir)


def test_fortran_order_and_truncation(pb, tiny_dir):
    p = os.path.join(tiny_dir, "bert_encoder_layer_0_output_dense_kernel.npy")
    a = np.load(p)
    np.save(p, np.asfortranarray(a))
    with pytest.raises(pb.CubertError, match="fortran"):
        chk(pb, tiny_dir)
    np.save(p, a)
    raw = open(p, "rb").read()
    open(p, "wb").write(raw[:-8])
    with pytest.raises(pb.CubertError, match="truncated"):
        chk(pb, tiny_dir)


def test_ambiguous_names(pb, tiny_dir):
    src = os.path.join(tiny_dir, "bert_pooler_dense_kernel.npy")
    np.save(os.path.join(tiny_dir, "copy_of_bert_pooler_dense_kernel.npy"), np.load(src))
    with pytest.raises(pb.CubertError, match="more than one"):
        chk(pb, tiny_dir)


def test_dimension_mismatch_and_head_dim(pb, tiny_dir):
    with pytest.raises(pb.CubertError):
        pb.check_weight_dir(tiny_dir, 256, T.layers, 4, T.inter)      # wrong hidden
    with pytest.raises(pb.CubertError, match="64"):
        pb.check_weight_dir(tiny_dir, T.hidden, T.layers, 4, T.inter)  # head dim 32
    with pytest.raises(pb.CubertError, match="_2_"):
        pb.check_weight_dir(tiny_dir, T.hidden, 3, T.heads, T.inter)   # a layer too many


def test_npy_versions(pb, tiny_dir):
    """Format 2.0 headers are accepted (the reference's reader assumed 1.0)."""
    p = os.path.join(tiny_dir, "bert_pooler_dense_bias.npy")
    a = np.load(p)
    with open(p, "wb") as f:
        np.lib.format.write_array(f, a, version=(2, 0))
    chk(pb, tiny_dir)


def test_init_model_without_gpu_reports_error(pb, tiny_dir):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(pb.CubertError):
        pb.load_model_ex(tiny_dir, T.hidden, T.layers, T.heads, T.inter)


def test_cuda_bert_exits_on_error_like_the_reference():
    """Cuda_Bert has no error return: an invalid call terminates the process
    (cuda_bert/utils/manager.cu:100-108, common.h:58-65)."""
    code = ("import numpy as np\n"
            "from cudabert_amd import pybert\n"
            "z = np.zeros((1, 4), np.int32)\n"
            "pybert.bert(None, np.zeros((1, 8), np.float32), z, z, 1, 4, z)\n"
            "print('survived')\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert r.returncode == 1 and "survived" not in r.stdout
    assert "Cuda_Bert failed" in r.stderr


def test_seed_batch(pb):
    # the stretched seed rows of the reference's benchmarks (cuda_bert/cuda_bert.cu:12-22, 94-103)
    ids, seg, mask = pb.seed_batch(2, 23)
    assert ids.shape == seg.shape == mask.shape == (2, 23) and ids.dtype == np.int32
    assert (ids[0] == ids[1]).all()
    assert list(ids[0, :10]) == pb.SEED_IDS[:10] and list(ids[0, 10:20]) == pb.SEED_IDS[:10]
    assert ids[0, -1] == pb.SEED_IDS[-1] and seg[0, -1] == 1 and mask[0, -1] == 0
    ids11, _, mask11 = pb.seed_batch(1, 11)
    assert list(ids11[0]) == pb.SEED_IDS and list(mask11[0]) == pb.SEED_MASK


def test_reference_input_helpers():
    """filling_inputs / batch_inputs / warp_inputs of cuda_bert/pybert.py:44-65, which user scripts import from the
    binding module: the seed row is stretched by cycling through all but its last entry, which stays last."""
    pb = pytest.importorskip("cudabert_amd.pybert")
    seed = list(range(100, 111))                       # 11 entries
    assert pb.filling_inputs(seed, 11) == seed
    assert pb.filling_inputs(seed, 5) == seed           # shorter requests return the row unchanged
    got = pb.filling_inputs(seed, 25)
    assert len(got) == 25 and got[-1] == 110 and got[:10] == seed[:10]
    assert got[10:24] == [100 + (i % 10) for i in range(10, 24)]
    assert seed == list(range(100, 111))                # the caller's list is untouched
    rows = pb.batch_inputs(got, 3)
    assert len(rows) == 3 and all(r == got for r in rows)
    a, b, c = pb.warp_inputs(rows, rows, rows)
    assert a.dtype == np.int32 and a.shape == (3, 25) and np.array_equal(a, b) and np.array_equal(b, c)
    ids, seg, mask = pb.seed_batch(3, 25)
    want = pb.warp_inputs(*[pb.batch_inputs(pb.filling_inputs(list(s), 25), 3) for s in (pb.SEED_IDS, pb.SEED_SEGMENTS, pb.SEED_MASK)])
    assert np.array_equal(ids, want[0]) and np.array_equal(seg, want[1]) and np.array_equal(mask, want[2])
