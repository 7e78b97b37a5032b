"""Synthetic BERT checkpoints and the name-keyed ``.npy`` directory layout.

The engine loads weights from a flat directory holding one float32 ``.npy``
per tensor.  File names and tensor orientation follow the reference's
checkpoint converter (convert_pytorch_model_to_npys.py:27-40 for names,
:59-66 for orientation; name.txt:1-22 lists the resulting files):

* ``LayerNorm.weight`` / ``LayerNorm.bias``  ->  ``LayerNorm_gamma`` / ``_beta``
* 2-D ``weight``  ->  ``kernel``; embeddings drop the ``_kernel`` suffix again
* ``.``  ->  ``_``
* every 2-D tensor that is not an embedding is stored transposed, ``[in, out]``

Nothing here touches the GPU; it is host-side tooling used by tests, the
benchmark and anybody who wants to export a PyTorch state dict for the engine.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, asdict
from typing import Dict

import numpy as np


@dataclass(frozen=True)
class BertDims:
    hidden: int = 768
    layers: int = 12
    heads: int = 12
    inter: int = 3072
    vocab: int = 30522
    max_pos: int = 512
    type_vocab: int = 2

    @property
    def head_dim(self) -> int:
        return self.hidden // self.heads

    def as_dict(self):
        return asdict(self)


# The two shapes the reference hard-codes (cuda_bert/utils/manager.cuh:46-50,
# manager.cu:8-15) and a tiny one for fast tests.
BASE = BertDims()
LARGE = BertDims(hidden=1024, layers=24, heads=16, inter=4096)
TINY = BertDims(hidden=128, layers=2, heads=2, inter=512, vocab=97, max_pos=64)


def synth_state(dims: BertDims, seed: int = 20240, degenerate: bool = True,
                classifier: bool = True) -> Dict[str, np.ndarray]:
    """A PyTorch-named state dict (``bert.*`` plus ``classifier.*``), float32.

    ``degenerate=True`` reproduces the stock initialisation
    (apps/pytorch_pretrained_bert/modeling.py:437-448): N(0, 0.02) Linear and
    Embedding weights, zero Linear biases, LayerNorm weight 1 / bias 0.
    ``degenerate=False`` draws biases ~N(0, 0.02), LayerNorm weight
    ~1 + N(0, 0.02) and bias ~N(0, 0.02) so that the bias and affine code
    paths are exercised.
    """
    rng = np.random.default_rng(seed)
    H, I = dims.hidden, dims.inter

    def normal(*shape):
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02))

    def bias(n):
        return np.zeros(n, np.float32) if degenerate else normal(n)

    def ln(prefix, out):
        out[prefix + ".weight"] = (np.ones(H, np.float32) if degenerate
                                   else (1.0 + normal(H)).astype(np.float32))
        out[prefix + ".bias"] = bias(H)

    sd: Dict[str, np.ndarray] = {}
    sd["bert.embeddings.word_embeddings.weight"] = normal(dims.vocab, H)
    sd["bert.embeddings.position_embeddings.weight"] = normal(dims.max_pos, H)
    sd["bert.embeddings.token_type_embeddings.weight"] = normal(dims.type_vocab, H)
    ln("bert.embeddings.LayerNorm", sd)
    for i in range(dims.layers):
        p = f"bert.encoder.layer.{i}."
        for nm in ("query", "key", "value"):
            sd[p + f"attention.self.{nm}.weight"] = normal(H, H)      # [out, in]
            sd[p + f"attention.self.{nm}.bias"] = bias(H)
        sd[p + "attention.output.dense.weight"] = normal(H, H)
        sd[p + "attention.output.dense.bias"] = bias(H)
        ln(p + "attention.output.LayerNorm", sd)
        sd[p + "intermediate.dense.weight"] = normal(I, H)
        sd[p + "intermediate.dense.bias"] = bias(I)
        sd[p + "output.dense.weight"] = normal(H, I)
        sd[p + "output.dense.bias"] = bias(H)
        ln(p + "output.LayerNorm", sd)
    sd["bert.pooler.dense.weight"] = normal(H, H)
    sd["bert.pooler.dense.bias"] = bias(H)
    if classifier:
        sd["classifier.weight"] = normal(2, H)
        sd["classifier.bias"] = bias(2)
    return sd


def bf16_representable(state: Dict[str, np.ndarray]) -> Dict[str, np.ndarray]:
    """The same checkpoint with every Linear kernel (2-D, not an embedding table) rounded to the
    nearest bfloat16 and stored as float32 again: the tensors the engine's bf16 mode keeps in
    bfloat16.  A float32 model and the bf16 engine then hold identical weights, so that a
    comparison between them measures the arithmetic and not the storage rounding."""
    import torch
    out = {}
    for name, arr in state.items():
        if arr.ndim == 2 and "embeddings" not in name:
            arr = torch.from_numpy(np.ascontiguousarray(arr)).to(torch.bfloat16).to(torch.float32).numpy()
        out[name] = arr
    return out


def convert_name(name: str, ndim: int) -> str:
    """PyTorch parameter name -> ``.npy`` base name
    (convert_pytorch_model_to_npys.py:27-40)."""
    if "LayerNorm" in name:
        name = name.replace("weight", "gamma") if "weight" in name else name.replace("bias", "beta")
    elif ndim == 2:
        name = name.replace("weight", "kernel")
    name = name.replace(".", "_")
    if "embeddings" in name and "_kernel" in name:
        name = name.replace("_kernel", "")
    return name


def to_npy_layout(state: Dict[str, np.ndarray]) -> Dict[str, np.ndarray]:
    """State dict -> {npy base name: array as stored on disk}
    (2-D non-embedding tensors transposed to ``[in, out]``,
    convert_pytorch_model_to_npys.py:59-66)."""
    out = {}
    for name, arr in state.items():
        new = convert_name(name, arr.ndim)
        a = np.asarray(arr, dtype=np.float32)
        if a.ndim == 2 and "embeddings" not in new:
            a = np.ascontiguousarray(a.T)
        out[new] = np.ascontiguousarray(a)
    return out


def export_npy_dir(state: Dict[str, np.ndarray], out_dir: str) -> str:
    os.makedirs(out_dir, exist_ok=True)
    for name, arr in to_npy_layout(state).items():
        np.save(os.path.join(out_dir, name + ".npy"), arr)
    return out_dir


def load_npy_dir(path: str) -> Dict[str, np.ndarray]:
    """Read every ``.npy`` of a weight directory (host side, for the checker)."""
    out = {}
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".npy"):
            out[fn[:-4]] = np.load(os.path.join(path, fn), allow_pickle=False)
    return out


def dims_from_npy(npy: Dict[str, np.ndarray], heads: int | None = None) -> BertDims:
    """Recover the model shape from a weight dictionary in ``.npy`` layout."""
    word = npy["bert_embeddings_word_embeddings"]
    H = word.shape[1]
    layers = 0
    while f"bert_encoder_layer_{layers}_attention_self_query_kernel" in npy:
        layers += 1
    inter = npy["bert_encoder_layer_0_intermediate_dense_kernel"].shape[1]
    return BertDims(hidden=H, layers=layers, heads=heads or H // 64, inter=inter,
                    vocab=word.shape[0],
                    max_pos=npy["bert_embeddings_position_embeddings"].shape[0],
                    type_vocab=npy["bert_embeddings_token_type_embeddings"].shape[0])


def export_checkpoint(init_checkpoint: str, output_dir: str) -> Dict[str, tuple]:
    """PyTorch checkpoint file -> weight directory; the command-line tool of the reference
    (convert_pytorch_model_to_npys.py:57-68).  The file is read with
    ``torch.load(..., weights_only=True)``: only tensors, nothing executed.  Every
    tensor of the checkpoint is written (task heads included, as the reference does);
    the engine picks the ones it needs.  Returns {file name: shape}."""
    import torch
    sd = torch.load(init_checkpoint, map_location="cpu", weights_only=True)
    if isinstance(sd, dict) and "state_dict" in sd and isinstance(sd["state_dict"], dict):
        sd = sd["state_dict"]
    state = {}
    for name, t in sd.items():
        if not torch.is_tensor(t):
            raise ValueError("checkpoint entry %r is not a tensor" % name)
        if t.is_floating_point():
            state[name] = t.detach().to(torch.float32).numpy()
    export_npy_dir(state, output_dir)
    return {n: a.shape for n, a in to_npy_layout(state).items()}


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(description="Write a PyTorch BERT checkpoint as the engine's .npy weight directory")
    ap.add_argument("--init_checkpoint", default="pytorch_model.bin", help="PyTorch checkpoint (state dict)")
    ap.add_argument("--output_dir", default="./model_npy", help="directory for the .npy files")
    ap.add_argument("--check", nargs=4, type=int, metavar=("HIDDEN", "LAYERS", "HEADS", "INTERMEDIATE"),
                    help="validate the written directory against these model dimensions (needs the built library)")
    args = ap.parse_args(argv)
    for name, shape in export_checkpoint(args.init_checkpoint, args.output_dir).items():
        print(name, " shape : ", tuple(shape))
    if args.check:
        from . import pybert
        pybert.check_weight_dir(args.output_dir, *args.check)
        print("weight directory accepted for", args.check)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
