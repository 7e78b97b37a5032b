// Host-side loader for the name-keyed ``.npy`` weight directory.
//
// Counterpart of load_from_dir_to_GPU / look_up_tts of the reference
// (cuda_bert/utils/load_model.cc:15-37, 86-99).  Like the reference a tensor is
// identified by key substrings of its file name (e.g. "_3_output_dense_kernel",
// or {"embeddings", "word"}); unlike the reference the match is made on the
// file's base name only, must be unique, and every tensor's shape is checked
// against the model dimensions before anything is uploaded.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "common.h"
#include "npy.h"

namespace cubert {

struct LayerTensors {
    const NpyArray *q_k, *q_b, *k_k, *k_b, *v_k, *v_b;
    const NpyArray *ao_k, *ao_b, *ao_g, *ao_be;
    const NpyArray *in_k, *in_b, *out_k, *out_b, *out_g, *out_be;
};

struct WeightDir {
    std::map<std::string, NpyArray> files;      // base name (no .npy) -> array
    const NpyArray *word = nullptr, *pos = nullptr, *type = nullptr, *emb_g = nullptr, *emb_b = nullptr;
    std::vector<LayerTensors> layers;
    const NpyArray *pool_k = nullptr, *pool_b = nullptr;
    const NpyArray *cls_k = nullptr, *cls_b = nullptr;   // optional
    int num_classes = 0;
};

// Reads every *.npy of `dir`, resolves all tensors the encoder needs for
// `dims` and validates their shapes.  dims->vocab / max_pos / type_vocab are
// filled in from the embedding tables.  Returns false with the error set.
bool load_weight_dir(const std::string& dir, Dims* dims, WeightDir* out);

}  // namespace cubert
