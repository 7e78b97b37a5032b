"""The name-keyed .npy layout written by cudabert_amd.weights."""
import os

import numpy as np

from cudabert_amd import weights as W


def test_names_match_reference_listing(tmp_path):
    # name.txt:1-22 of the reference lists the embedding and layer-0 files.
    expected = """bert_embeddings_LayerNorm_beta bert_embeddings_LayerNorm_gamma
    bert_embeddings_position_embeddings bert_embeddings_token_type_embeddings
    bert_embeddings_word_embeddings
    bert_encoder_layer_0_attention_output_dense_bias bert_encoder_layer_0_attention_output_dense_kernel
    bert_encoder_layer_0_attention_output_LayerNorm_beta bert_encoder_layer_0_attention_output_LayerNorm_gamma
    bert_encoder_layer_0_attention_self_key_bias bert_encoder_layer_0_attention_self_key_kernel
    bert_encoder_layer_0_attention_self_query_bias bert_encoder_layer_0_attention_self_query_kernel
    bert_encoder_layer_0_attention_self_value_bias bert_encoder_layer_0_attention_self_value_kernel
    bert_encoder_layer_0_intermediate_dense_bias bert_encoder_layer_0_intermediate_dense_kernel
    bert_encoder_layer_0_output_dense_bias bert_encoder_layer_0_output_dense_kernel
    bert_encoder_layer_0_output_LayerNorm_beta bert_encoder_layer_0_output_LayerNorm_gamma""".split()
    state = W.synth_state(W.TINY, seed=1)
    out = W.export_npy_dir(state, str(tmp_path / "m"))
    files = {f[:-4] for f in os.listdir(out)}
    assert set(expected) <= files
    assert {"bert_pooler_dense_kernel", "bert_pooler_dense_bias", "classifier_kernel", "classifier_bias"} <= files
    assert len(files) == 5 + 16 * W.TINY.layers + 2 + 2


def test_orientation_and_dtype(tmp_path):
    d = W.TINY
    state = W.synth_state(d, seed=1, degenerate=False)
    npy = W.load_npy_dir(W.export_npy_dir(state, str(tmp_path / "m")))
    assert all(a.dtype == np.float32 for a in npy.values())
    assert npy["bert_embeddings_word_embeddings"].shape == (d.vocab, d.hidden)       # untransposed
    assert npy["bert_encoder_layer_0_intermediate_dense_kernel"].shape == (d.hidden, d.inter)   # [in,out]
    assert npy["bert_encoder_layer_1_output_dense_kernel"].shape == (d.inter, d.hidden)
    assert npy["classifier_kernel"].shape == (d.hidden, 2)
    w = state["bert.encoder.layer.0.intermediate.dense.weight"]
    assert np.array_equal(npy["bert_encoder_layer_0_intermediate_dense_kernel"], w.T)
    assert W.dims_from_npy(npy, heads=d.heads) == d


def test_stock_init_statistics():
    sd = W.synth_state(W.TINY, seed=3, degenerate=True)
    assert not sd["bert.encoder.layer.0.output.dense.bias"].any()
    assert (sd["bert.embeddings.LayerNorm.weight"] == 1).all()
    w = sd["bert.embeddings.word_embeddings.weight"]
    assert abs(w.std() - 0.02) < 2e-3 and abs(w.mean()) < 2e-3


def test_checkpoint_exporter_cli(tmp_path):
    """A PyTorch checkpoint with the usual `bert.` prefix and pre-training heads goes through the
    command-line exporter and the library's host-side validation accepts the result."""
    import torch
    from cudabert_amd import pybert
    D = W.TINY
    state = W.synth_state(D, seed=5)
    sd = {k: torch.from_numpy(v) for k, v in state.items()}
    sd["cls.predictions.transform.dense.weight"] = torch.randn(D.hidden, D.hidden)
    sd["cls.predictions.transform.LayerNorm.weight"] = torch.ones(D.hidden)
    sd["cls.predictions.transform.LayerNorm.bias"] = torch.zeros(D.hidden)
    sd["cls.predictions.decoder.weight"] = torch.randn(D.vocab, D.hidden)
    sd["cls.seq_relationship.weight"] = torch.randn(2, D.hidden)
    sd["bert.embeddings.position_ids"] = torch.arange(D.max_pos)[None]          # integer buffer: skipped
    ck = str(tmp_path / "pytorch_model.bin")
    torch.save(sd, ck)
    out = str(tmp_path / "npy")
    assert W.main(["--init_checkpoint", ck, "--output_dir", out, "--check", str(D.hidden), str(D.layers),
                   str(D.heads), str(D.inter)]) == 0
    npy = W.load_npy_dir(out)
    assert npy["cls_predictions_decoder_kernel"].shape == (D.hidden, D.vocab)      # 2-D, not an embedding: transposed
    assert npy["cls_predictions_transform_LayerNorm_gamma"].shape == (D.hidden,)
    assert "bert_embeddings_position_ids" not in npy
    q = "bert.encoder.layer.1.attention.self.query.weight"
    assert np.array_equal(npy["bert_encoder_layer_1_attention_self_query_kernel"], state[q].T)
    assert W.dims_from_npy(npy) == D
