"""ctypes binding of ``libcudaBERT.so`` (the MI355X engine).

Mirrors the reference binding (cuda_bert/pybert.py:12-38): the same module-level
names ``load_model`` / ``unload_model`` / ``inference`` / ``bert`` with the same
argument order, so code written against the reference's ``pybert`` works when
pointed at this module.  It has no tokenizer dependency and no import-time
network access.  The library must have been built (``python -m
cudabert_amd.build``); there is no fallback when it is missing.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_bool, c_char_p, c_float, c_int, c_long, c_void_p)

import numpy
from numpy.ctypeslib import ndpointer

lib_dir = os.path.abspath(os.path.dirname(__file__))
LIB_PATH = os.path.join(lib_dir, "libcudaBERT.so")
if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `python -m cudabert_amd.build`" % LIB_PATH)
lib = ctypes.CDLL(LIB_PATH, ctypes.RTLD_GLOBAL)


class Retval(Structure):
    """Device pointers of the last forward pass (cuda_bert/utils/common.h:173-177)."""
    _fields_ = [("tensor", c_void_p), ("Pooled_Output", c_void_p)]


class Config(Structure):
    _fields_ = [("hidden", c_int), ("layers", c_int), ("heads", c_int), ("intermediate", c_int),
                ("precision", c_int), ("graph_max_tokens", c_int)]


_i32 = ndpointer(numpy.int32, flags="C_CONTIGUOUS")
_f32 = ndpointer(numpy.float32, flags="C_CONTIGUOUS")

# ---- reference-compatible surface (cuda_bert/pybert.py:14-38) ----
init_model = lib.init_model
init_model.argtypes = [c_bool, c_int, c_int, c_int, c_char_p]
init_model.restype = c_void_p

release_model = lib.release_model
release_model.argtypes = [c_void_p]
release_model.restype = None

inference = lib.Cuda_Inference
inference.argtypes = [c_void_p, _i32, _i32, c_int, c_int, _i32]
inference.restype = Retval

bert = lib.Cuda_Bert
bert.argtypes = [c_void_p, _f32, _i32, _i32, c_int, c_int, _i32]
bert.restype = None

# the binding the reference left commented out (cuda_bert/pybert.py:40-42)
classify = lib.Cuda_Classify
classify.argtypes = [c_void_p, _f32, _i32, _i32, c_int, c_int, c_int, _i32]
classify.restype = None

lib.test.argtypes = [c_int, c_int, c_int, c_bool, c_int]
lib.test.restype = None

# ---- additive surface ----
lib.cubert_last_error.argtypes = []
lib.cubert_last_error.restype = c_char_p
lib.init_model_ex.argtypes = [POINTER(Config), c_int, c_int, c_int, c_char_p]
lib.init_model_ex.restype = c_void_p
lib.cubert_check_weight_dir.argtypes = [POINTER(Config), c_char_p]
lib.cubert_check_weight_dir.restype = c_int
lib.cubert_forward_device_lens.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int]
lib.cubert_forward_device_lens.restype = c_int
lib.cubert_encode.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]
lib.cubert_encode.restype = c_int
lib.cubert_forward_device.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int]
lib.cubert_forward_device.restype = c_int
lib.cubert_classify.argtypes = [c_void_p]
lib.cubert_classify.restype = c_int
lib.cubert_cls_ptr.argtypes = [c_void_p]
lib.cubert_cls_ptr.restype = c_void_p
lib.cubert_profile_device.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, POINTER(c_float)]
lib.cubert_profile_device.restype = c_int
PHASES = ("embedding", "qkv_gemm", "attention", "attn_out_gemm", "add_layernorm", "ffn_in_gemm", "ffn_out_gemm",
          "pooler")
lib.cubert_sync.argtypes = [c_void_p]
lib.cubert_sync.restype = c_int
lib.cubert_seq_ptr.argtypes = [c_void_p]
lib.cubert_seq_ptr.restype = c_void_p
lib.cubert_pooled_ptr.argtypes = [c_void_p]
lib.cubert_pooled_ptr.restype = c_void_p
lib.cubert_stream.argtypes = [c_void_p]
lib.cubert_stream.restype = c_void_p
for _n in ("cubert_hidden_size", "cubert_num_classes", "cubert_precision", "cubert_graphs_cached", "cubert_ln_fallbacks",
           "cubert_debug_force_ln_timeout"):
    getattr(lib, _n).argtypes = [c_void_p]
    getattr(lib, _n).restype = c_int
lib.cubert_capacity_tokens.argtypes = [c_void_p]
lib.cubert_capacity_tokens.restype = c_long

X_PACKED, W_PACKED, Y_PACKED, COMPILER_SCHEDULED = 1, 2, 4, 8      # layout flags of the op entry points
lib.cubert_packed_bytes.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
lib.cubert_packed_bytes.restype = ctypes.c_size_t
lib.cubert_packed_offset.argtypes = [c_int, c_int, c_int]
lib.cubert_packed_offset.restype = ctypes.c_size_t
lib.cubert_op_gemm.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_void_p]
lib.cubert_op_gemm.restype = c_int
lib.cubert_op_gemm_residual.argtypes = [c_void_p] * 5 + [c_int] * 7 + [c_void_p]
lib.cubert_op_gemm_residual.restype = c_int
lib.cubert_gemm_layernorm_workspace_bytes.argtypes = [c_int]
lib.cubert_gemm_layernorm_workspace_bytes.restype = ctypes.c_size_t
lib.cubert_op_gemm_residual_layernorm.argtypes = [c_void_p] * 9 + [c_int] * 6 + [c_void_p]
lib.cubert_op_gemm_residual_layernorm.restype = c_int
lib.cubert_op_gemm_splitk_noalloc.argtypes = [c_void_p] * 4 + [c_int] * 8 + [c_void_p]
lib.cubert_op_gemm_splitk_noalloc.restype = c_int
lib.cubert_noalloc_scratch_bytes.argtypes = []
lib.cubert_noalloc_scratch_bytes.restype = ctypes.c_size_t
lib.cubert_op_gemm_qkv.argtypes = [c_void_p] * 6 + [c_int] * 6 + [c_void_p]
lib.cubert_op_gemm_qkv.restype = c_int
lib.cubert_op_attention.argtypes = [c_void_p] * 5 + [c_int, c_int, c_int, c_float, c_int, c_int, c_void_p]
lib.cubert_op_attention.restype = c_int
lib.cubert_op_add_layernorm.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                        c_int, c_void_p]
lib.cubert_op_add_layernorm.restype = c_int
lib.cubert_op_embed_layernorm.argtypes = [c_void_p] * 11 + [c_int] * 6 + [c_void_p]
lib.cubert_op_embed_layernorm.restype = c_int
lib.cubert_op_pooler.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
lib.cubert_op_pooler.restype = c_int
lib.cubert_op_mask_softmax.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p]
lib.cubert_op_mask_softmax.restype = c_int

F32, BF16 = 0, 1


class CubertError(RuntimeError):
    pass


def last_error() -> str:
    return lib.cubert_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise CubertError(last_error())


def load_model(is_large_model, model_dir, num_gpu=0, max_batchsize=0, max_seq_length=0):
    """Same signature as the reference's ``load_model`` (cuda_bert/pybert.py:21-26).
    Raises CubertError instead of returning a NULL handle."""
    h = init_model(bool(is_large_model), num_gpu, max_batchsize, max_seq_length,
                   bytes(model_dir, encoding="utf-8"))
    if not h:
        raise CubertError(last_error())
    return h


def load_model_ex(model_dir, hidden, layers, heads, intermediate, precision=F32, num_gpu=0,
                  max_batchsize=0, max_seq_length=0, graph_max_tokens=8192):
    cfg = Config(hidden, layers, heads, intermediate, precision, graph_max_tokens)
    h = lib.init_model_ex(ctypes.byref(cfg), num_gpu, max_batchsize, max_seq_length,
                          bytes(model_dir, encoding="utf-8"))
    if not h:
        raise CubertError(last_error())
    return h


def check_weight_dir(model_dir, hidden, layers, heads, intermediate) -> None:
    cfg = Config(hidden, layers, heads, intermediate, 0, 0)
    check(lib.cubert_check_weight_dir(ctypes.byref(cfg), bytes(model_dir, encoding="utf-8")))


def unload_model(model):
    release_model(model)


def _i32c(a):
    return numpy.ascontiguousarray(a, dtype=numpy.int32)


def encode(model, ids, seg, mask=None, want_seq=False, want_cls=False):
    """Runs the encoder; returns (pooled [B,H], seq [B,S,H] or None, cls [B,C] or None)."""
    ids, seg = _i32c(ids), _i32c(seg)
    B, S = ids.shape
    mask = None if mask is None else _i32c(mask)
    H = lib.cubert_hidden_size(model)
    pooled = numpy.empty((B, H), numpy.float32)
    seq = numpy.empty((B, S, H), numpy.float32) if want_seq else None
    cls = numpy.empty((B, lib.cubert_num_classes(model)), numpy.float32) if want_cls else None
    ptr = lambda a: None if a is None else a.ctypes.data
    check(lib.cubert_encode(model, ptr(ids), ptr(seg), ptr(mask), B, S, ptr(pooled), ptr(seq), ptr(cls)))
    return pooled, seq, cls


# ---- benchmark input of the reference (cuda_bert/pybert.py:44-100, cuda_bert/cuda_bert.cu:94-103) ----
# ids of ['who', 'was', 'jim', 'henson', '?', 'jim', '[MASK]', 'was', 'a', 'puppet', '##eer'] in the
# bert-base-uncased vocabulary, their segment ids and mask.
SEED_IDS = [2040, 2001, 3958, 27227, 1029, 3958, 103, 2001, 1037, 13997, 11510]
SEED_SEGMENTS = [0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1]
SEED_MASK = [1, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0]


def filling_inputs(words, seq_length):
    """cuda_bert/pybert.py:44-53: stretches a seed row to seq_length by cycling through all but its last entry and
    keeping the last entry at the end; a row that is already longer comes back unchanged.  Returns a new list."""
    body, last = list(words[:-1]), words[-1]
    n = len(body)
    body.extend(body[i % n] for i in range(n, seq_length - 1))
    return body + [last]


def batch_inputs(input, batchsize):
    """cuda_bert/pybert.py:55-59: the row repeated batchsize times."""
    return [input] * batchsize


def warp_inputs(indexed_tokens, segments_ids, attention_masks):
    """cuda_bert/pybert.py:61-65: the three nested lists as int32 arrays."""
    return tuple(numpy.array(a).astype(numpy.int32) for a in (indexed_tokens, segments_ids, attention_masks))


def seed_batch(batchsize, seq_length):
    """The reference benchmarks' input as int32 [batchsize, seq_length] arrays (ids, segments, mask):
    each 11-entry seed row is stretched to seq_length by cycling through its first ten entries and
    keeping its last entry in the last column, and the row is repeated batchsize times.  Equal to
    warp_inputs(*[batch_inputs(filling_inputs(seed, seq_length), batchsize) for each seed]) from 11 columns on;
    shorter requests are cut to seq_length here, where filling_inputs returns all 11 entries."""
    if seq_length < 2:
        raise ValueError("seq_length must be at least 2")
    cycle = numpy.arange(seq_length - 1) % 10

    def stretch(seed):
        seed = numpy.asarray(seed, numpy.int32)
        row = numpy.append(seed[cycle], seed[-1])
        return numpy.ascontiguousarray(numpy.broadcast_to(row, (batchsize, seq_length)))

    return stretch(SEED_IDS), stretch(SEED_SEGMENTS), stretch(SEED_MASK)


def test(is_large, model_dir, batchsize, seq_length, num_gpu=0, iters=100):
    """Mean time of an asynchronous inference call on the seed batch: what the reference's
    Python timing loop prints (cuda_bert/pybert.py:70-100), without its tokenizer download."""
    import time
    ids, seg, mask = seed_batch(batchsize, seq_length)
    model = load_model(is_large, model_dir, num_gpu=num_gpu)
    try:
        start = time.perf_counter()
        for _ in range(iters):
            inference(model, ids, seg, batchsize, seq_length, mask)
        check(lib.cubert_sync(model))
        mean = (time.perf_counter() - start) / iters
    finally:
        unload_model(model)
    print("Batchsize: {} Seq_length: {} Use_Time: {}".format(batchsize, seq_length, mean))
    return mean
