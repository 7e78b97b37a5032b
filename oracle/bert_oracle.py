"""CPU oracle for the BERT encoder forward pass.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the algorithm of the reference's PyTorch
``BertModel`` (apps/pytorch_pretrained_bert/modeling.py) -- the model the HIP
engine has to agree with.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it, and only as the checker.
The engine itself never calls into this file and has no CPU fallback.

Two independent restatements live here:

* ``forward_torch``  -- float32, ``torch`` ops on the host cores.  Used for
  full-size parity and for the CPU throughput baseline.
* ``forward_numpy64`` -- float64, plain ``numpy`` with explicit per-head loops.
  Slow; used on small cases to pin ``forward_torch``.

Pinning (tests/test_oracle.py): both restatements are checked against each
other, against the HuggingFace ``transformers`` ``BertModel`` (an independent
library implementation of the same architecture) loaded with identical
weights, against golden vectors of that library under ``tests/golden/``, and
against closed-form invariants (softmax rows sum to one, LayerNorm moments,
padding invariance, batch permutation equivariance, explicit brute-force
attention on a 1x3 example).  The reference ships no golden vectors for this
path (its only sample output needs fine-tuned weights that are not in the
tree), so none are used.

Weights are taken in the on-disk ``.npy`` layout (name -> array, Linear kernels
stored ``[in, out]``; convert_pytorch_model_to_npys.py:27-40,59-66).
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import numpy as np


# --------------------------------------------------------------------------- #
# float32 torch restatement
# --------------------------------------------------------------------------- #

def _t(npy, name):
    import torch
    return torch.from_numpy(np.ascontiguousarray(npy[name]))


def gelu_torch(x):
    """x * 0.5 * (1 + erf(x / sqrt(2)))        modeling.py:53-58"""
    import torch
    return x * 0.5 * (1.0 + torch.erf(x / math.sqrt(2.0)))


def layer_norm_torch(x, gamma, beta, eps: float = 1e-12):
    """TF-style LayerNorm, biased variance, eps inside the sqrt.
    modeling.py:168-172"""
    import torch
    u = x.mean(-1, keepdim=True)
    s = (x - u).pow(2).mean(-1, keepdim=True)
    x = (x - u) / torch.sqrt(s + eps)
    return gamma * x + beta


def embeddings_torch(npy, ids, seg):
    """word + position + token_type, then LayerNorm.   modeling.py:188-202"""
    import torch
    S = ids.shape[1]
    pos = torch.arange(S, dtype=torch.long).unsqueeze(0).expand_as(ids)
    e = (_t(npy, "bert_embeddings_word_embeddings")[ids]
         + _t(npy, "bert_embeddings_position_embeddings")[pos]
         + _t(npy, "bert_embeddings_token_type_embeddings")[seg])
    return layer_norm_torch(e, _t(npy, "bert_embeddings_LayerNorm_gamma"),
                            _t(npy, "bert_embeddings_LayerNorm_beta"))


def extended_mask_torch(mask):
    """(1 - mask) * -10000, broadcast as [B,1,1,S].    modeling.py:625-633"""
    import torch
    return (1.0 - mask.to(torch.float32)).unsqueeze(1).unsqueeze(2) * -10000.0


def self_attention_torch(x, npy, p, heads, ext_mask):
    """modeling.py:222-253."""
    import torch
    B, S, H = x.shape
    d = H // heads

    def lin(name):
        return x @ _t(npy, p + f"attention_self_{name}_kernel") + _t(npy, p + f"attention_self_{name}_bias")

    def split(t):                     # transpose_for_scores, modeling.py:222-225
        return t.view(B, S, heads, d).permute(0, 2, 1, 3)

    q, k, v = split(lin("query")), split(lin("key")), split(lin("value"))
    scores = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(d)
    scores = scores + ext_mask
    probs = torch.softmax(scores, dim=-1)
    ctx = torch.matmul(probs, v)
    return ctx.permute(0, 2, 1, 3).contiguous().view(B, S, H)


def layer_torch(x, npy, i, heads, ext_mask):
    """One BertLayer.                                  modeling.py:256-320"""
    p = f"bert_encoder_layer_{i}_"
    ctx = self_attention_torch(x, npy, p, heads, ext_mask)
    a = ctx @ _t(npy, p + "attention_output_dense_kernel") + _t(npy, p + "attention_output_dense_bias")
    x = layer_norm_torch(a + x, _t(npy, p + "attention_output_LayerNorm_gamma"),
                         _t(npy, p + "attention_output_LayerNorm_beta"))
    h = gelu_torch(x @ _t(npy, p + "intermediate_dense_kernel") + _t(npy, p + "intermediate_dense_bias"))
    o = h @ _t(npy, p + "output_dense_kernel") + _t(npy, p + "output_dense_bias")
    return layer_norm_torch(o + x, _t(npy, p + "output_LayerNorm_gamma"),
                            _t(npy, p + "output_LayerNorm_beta"))


def pooler_torch(seq, npy):
    """tanh(dense(h[:, 0]))                            modeling.py:347-353"""
    import torch
    return torch.tanh(seq[:, 0] @ _t(npy, "bert_pooler_dense_kernel") + _t(npy, "bert_pooler_dense_bias"))


def forward_torch(npy: Dict[str, np.ndarray], heads: int, ids, seg, mask=None,
                  layers: Optional[int] = None, return_stages: bool = False):
    """BertModel.forward in eval mode (modeling.py:613-647).

    ids/seg/mask: integer arrays [B,S].  Returns (sequence_output [B,S,H],
    pooled_output [B,H]) as float32 numpy arrays.
    """
    import torch
    with torch.no_grad():
        ids_t = torch.as_tensor(np.asarray(ids), dtype=torch.long)
        seg_t = torch.zeros_like(ids_t) if seg is None else torch.as_tensor(np.asarray(seg), dtype=torch.long)
        mask_t = torch.ones_like(ids_t) if mask is None else torch.as_tensor(np.asarray(mask), dtype=torch.long)
        ext = extended_mask_torch(mask_t)
        x = embeddings_torch(npy, ids_t, seg_t)
        stages = {"embedding": x.numpy().copy()} if return_stages else None
        L = layers
        if L is None:
            L = 0
            while f"bert_encoder_layer_{L}_attention_self_query_kernel" in npy:
                L += 1
        for i in range(L):
            x = layer_torch(x, npy, i, heads, ext)
            if return_stages:
                stages[f"layer{i}"] = x.numpy().copy()
        pooled = pooler_torch(x, npy)
        if return_stages:
            return x.numpy(), pooled.numpy(), stages
        return x.numpy(), pooled.numpy()


def classifier_head(npy, pooled: np.ndarray) -> np.ndarray:
    """softmax(pooled @ classifier_kernel + bias); the frontend keeps the last
    column (apps/finetune.py:16-24, 33-34, 40-44).  Returns [B, 2]."""
    z = pooled.astype(np.float64) @ npy["classifier_kernel"].astype(np.float64) + npy["classifier_bias"]
    z = z - z.max(-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(-1, keepdims=True)).astype(np.float32)


# --------------------------------------------------------------------------- #
# float64 numpy restatement, written with explicit loops over batch and head so
# that it shares no reshaping logic with the torch version above.
# --------------------------------------------------------------------------- #

def _erf64(x):
    from scipy.special import erf
    return erf(x)


def layer_norm_np(x, gamma, beta, eps=1e-12):
    u = x.mean(-1, keepdims=True)
    s = ((x - u) ** 2).mean(-1, keepdims=True)
    return gamma * ((x - u) / np.sqrt(s + eps)) + beta


def forward_numpy64(npy, heads: int, ids, seg, mask=None, layers: Optional[int] = None):
    W = {k: v.astype(np.float64) for k, v in npy.items()}
    ids = np.asarray(ids)
    B, S = ids.shape
    seg = np.zeros_like(ids) if seg is None else np.asarray(seg)
    mask = np.ones_like(ids) if mask is None else np.asarray(mask)
    H = W["bert_embeddings_word_embeddings"].shape[1]
    d = H // heads
    x = np.empty((B, S, H))
    for b in range(B):
        for t in range(S):
            x[b, t] = (W["bert_embeddings_word_embeddings"][ids[b, t]]
                       + W["bert_embeddings_position_embeddings"][t]
                       + W["bert_embeddings_token_type_embeddings"][seg[b, t]])
    x = layer_norm_np(x, W["bert_embeddings_LayerNorm_gamma"], W["bert_embeddings_LayerNorm_beta"])
    L = layers
    if L is None:
        L = 0
        while f"bert_encoder_layer_{L}_attention_self_query_kernel" in W:
            L += 1
    for i in range(L):
        p = f"bert_encoder_layer_{i}_"
        q = x @ W[p + "attention_self_query_kernel"] + W[p + "attention_self_query_bias"]
        k = x @ W[p + "attention_self_key_kernel"] + W[p + "attention_self_key_bias"]
        v = x @ W[p + "attention_self_value_kernel"] + W[p + "attention_self_value_bias"]
        ctx = np.empty_like(x)
        for b in range(B):
            addm = (1.0 - mask[b].astype(np.float64)) * -10000.0
            for h in range(heads):
                sl = slice(h * d, (h + 1) * d)
                sc = q[b, :, sl] @ k[b, :, sl].T / math.sqrt(d) + addm[None, :]
                sc = sc - sc.max(-1, keepdims=True)
                e = np.exp(sc)
                pr = e / e.sum(-1, keepdims=True)
                ctx[b, :, sl] = pr @ v[b, :, sl]
        a = ctx @ W[p + "attention_output_dense_kernel"] + W[p + "attention_output_dense_bias"]
        x = layer_norm_np(a + x, W[p + "attention_output_LayerNorm_gamma"], W[p + "attention_output_LayerNorm_beta"])
        hmid = x @ W[p + "intermediate_dense_kernel"] + W[p + "intermediate_dense_bias"]
        hmid = hmid * 0.5 * (1.0 + _erf64(hmid / math.sqrt(2.0)))
        o = hmid @ W[p + "output_dense_kernel"] + W[p + "output_dense_bias"]
        x = layer_norm_np(o + x, W[p + "output_LayerNorm_gamma"], W[p + "output_LayerNorm_beta"])
    pooled = np.tanh(x[:, 0] @ W["bert_pooler_dense_kernel"] + W["bert_pooler_dense_bias"])
    return x, pooled
