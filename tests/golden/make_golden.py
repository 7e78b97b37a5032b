"""Writes the golden vectors under tests/golden/ (run once, in the build container).

The vectors come from the HuggingFace ``transformers`` ``BertModel`` -- an
independent library implementation of the architecture the oracle restates --
loaded with weights from this repository's seeded generator.  The reference
tree holds no golden vectors for the encoder (its sample output depends on
fine-tuned weights that are not shipped), and its Python is not imported here.

    python tests/golden/make_golden.py

Outputs (all small):
  tiny_nd_s{5,16,33}.npz   TINY dims, non-degenerate weights, ragged masks:
                           inputs, sequence output, pooled output, embedding
                           output and layer-0 output.
  base_cfg0_slice.npz      BERT-base b8 s128 (benchmark configuration 0, stock
                           initialisation, weight seed 20240): inputs, pooled
                           [8,768] and seq[:, ::16, :32].
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from cudabert_amd import weights as W          # noqa: E402
from cudabert_amd import synth                 # noqa: E402


def hf_model(state, dims):
    from transformers import BertConfig, BertModel
    cfg = BertConfig(vocab_size=dims.vocab, hidden_size=dims.hidden, num_hidden_layers=dims.layers,
                     num_attention_heads=dims.heads, intermediate_size=dims.inter,
                     max_position_embeddings=dims.max_pos, type_vocab_size=dims.type_vocab,
                     hidden_act="gelu", layer_norm_eps=1e-12, hidden_dropout_prob=0.0,
                     attention_probs_dropout_prob=0.0, attn_implementation="eager")
    m = BertModel(cfg).eval()
    sd = {k[len("bert."):]: torch.from_numpy(v) for k, v in state.items() if k.startswith("bert.")}
    missing, unexpected = m.load_state_dict(sd, strict=False)
    assert not unexpected, unexpected
    assert all("position_ids" in k or "token_type_ids" in k for k in missing), missing
    return m


def run(m, ids, seg, mask):
    with torch.no_grad():
        o = m(input_ids=torch.from_numpy(ids).long(), token_type_ids=torch.from_numpy(seg).long(),
              attention_mask=torch.from_numpy(mask).long(), output_hidden_states=True)
    return o


def main():
    torch.manual_seed(0)
    dims = W.TINY
    state = W.synth_state(dims, seed=7, degenerate=False)
    m = hf_model(state, dims)
    for S, lens in ((5, [5, 3, 1]), (16, [16, 9, 4]), (33, [20, 33, 7])):
        ids, seg, mask = synth.make_inputs(3, S, lens, vocab=dims.vocab, seed=100 + S, prune=False)
        o = run(m, ids, seg, mask)
        np.savez(os.path.join(HERE, f"tiny_nd_s{S}.npz"), ids=ids, seg=seg, mask=mask,
                 seq=o.last_hidden_state.numpy(), pooled=o.pooler_output.numpy(),
                 embedding=o.hidden_states[0].numpy(), layer0=o.hidden_states[1].numpy())
    dims = W.BASE
    state = W.synth_state(dims, seed=20240, degenerate=True)
    m = hf_model(state, dims)
    ids, seg, mask = synth.config_inputs(0)
    o = run(m, ids, seg, mask)
    np.savez(os.path.join(HERE, "base_cfg0_slice.npz"), ids=ids, seg=seg, mask=mask,
             pooled=o.pooler_output.numpy(), seq_slice=o.last_hidden_state.numpy()[:, ::16, :32])
    print("golden vectors written to", HERE)


if __name__ == "__main__":
    main()
