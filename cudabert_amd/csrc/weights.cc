#include "weights.h"

#include <dirent.h>

#include <algorithm>
#include <cstring>

namespace cubert {

namespace {

const NpyArray* find_unique(const WeightDir& w, const std::vector<std::string>& keys, bool required,
                            bool* ok) {
    const NpyArray* hit = nullptr;
    std::string hit_name;
    for (const auto& kv : w.files) {
        bool all = true;
        for (const auto& k : keys)
            if (kv.first.find(k) == std::string::npos) { all = false; break; }
        if (!all) continue;
        if (hit) {
            std::string ks;
            for (const auto& k : keys) ks += " '" + k + "'";
            set_error("weight keys" + ks + " match more than one file: " + hit_name + ".npy and " + kv.first + ".npy");
            *ok = false;
            return nullptr;
        }
        hit = &kv.second;
        hit_name = kv.first;
    }
    if (!hit && required) {
        std::string ks;
        for (const auto& k : keys) ks += " '" + k + "'";
        set_error("no .npy file in the weight directory matches keys" + ks);
        *ok = false;
    }
    return hit;
}

bool check_shape(const NpyArray* a, const std::vector<size_t>& want, const std::string& what) {
    if (!a) return false;
    if (a->shape != want) {
        std::string got, exp;
        for (size_t s : a->shape) got += std::to_string(s) + ",";
        for (size_t s : want) exp += std::to_string(s) + ",";
        set_error("weight '" + what + "' has shape (" + got + ") but (" + exp + ") is required");
        return false;
    }
    return true;
}

}  // namespace

bool load_weight_dir(const std::string& dir, Dims* dims, WeightDir* out) {
    DIR* d = opendir(dir.c_str());
    if (!d) { set_error("cannot open weight directory '" + dir + "'"); return false; }
    std::vector<std::string> names;
    while (struct dirent* e = readdir(d)) {
        const size_t n = std::strlen(e->d_name);
        if (n > 4 && std::strcmp(e->d_name + n - 4, ".npy") == 0) names.emplace_back(e->d_name, n - 4);
    }
    closedir(d);
    if (names.empty()) { set_error("weight directory '" + dir + "' holds no .npy files"); return false; }
    std::sort(names.begin(), names.end());
    for (const auto& nm : names) {
        std::string err;
        NpyArray arr;
        if (!npy_load_f32(dir + "/" + nm + ".npy", &arr, &err)) { set_error(err); return false; }
        out->files.emplace(nm, std::move(arr));
    }

    const size_t H = (size_t)dims->hidden, I = (size_t)dims->inter;
    bool ok = true;
    auto need = [&](std::vector<std::string> keys) { return ok ? find_unique(*out, keys, true, &ok) : nullptr; };

    out->word = need({"embeddings", "word"});
    out->pos = need({"embeddings", "position"});
    out->type = need({"embeddings", "token_type"});
    out->emb_g = need({"embeddings_LayerNorm_gamma"});
    out->emb_b = need({"embeddings_LayerNorm_beta"});
    if (!ok) return false;
    if (out->word->shape.size() != 2 || out->word->shape[1] != H) {
        set_error("word embedding table does not have hidden size " + std::to_string(H));
        return false;
    }
    if (out->pos->shape.size() != 2 || out->type->shape.size() != 2) {
        set_error("position / token_type embedding tables must be 2-D");
        return false;
    }
    dims->vocab = (int)out->word->shape[0];
    dims->max_pos = (int)out->pos->shape[0];
    dims->type_vocab = (int)out->type->shape[0];
    if (!check_shape(out->pos, {(size_t)dims->max_pos, H}, "position_embeddings") ||
        !check_shape(out->type, {(size_t)dims->type_vocab, H}, "token_type_embeddings") ||
        !check_shape(out->emb_g, {H}, "embeddings_LayerNorm_gamma") ||
        !check_shape(out->emb_b, {H}, "embeddings_LayerNorm_beta"))
        return false;

    out->layers.resize(dims->layers);
    for (int i = 0; i < dims->layers && ok; ++i) {
        const std::string p = "_" + std::to_string(i) + "_";
        LayerTensors& L = out->layers[i];
        L.q_k = need({p + "attention_self_query_kernel"});
        L.q_b = need({p + "attention_self_query_bias"});
        L.k_k = need({p + "attention_self_key_kernel"});
        L.k_b = need({p + "attention_self_key_bias"});
        L.v_k = need({p + "attention_self_value_kernel"});
        L.v_b = need({p + "attention_self_value_bias"});
        L.ao_k = need({p + "attention_output_dense_kernel"});
        L.ao_b = need({p + "attention_output_dense_bias"});
        L.ao_g = need({p + "attention_output_LayerNorm_gamma"});
        L.ao_be = need({p + "attention_output_LayerNorm_beta"});
        L.in_k = need({p + "intermediate_dense_kernel"});
        L.in_b = need({p + "intermediate_dense_bias"});
        L.out_k = need({p + "output_dense_kernel"});
        L.out_b = need({p + "output_dense_bias"});
        L.out_g = need({p + "output_LayerNorm_gamma"});
        L.out_be = need({p + "output_LayerNorm_beta"});
        if (!ok) return false;
        const std::string li = "layer " + std::to_string(i) + " ";
        if (!check_shape(L.q_k, {H, H}, li + "query_kernel") || !check_shape(L.q_b, {H}, li + "query_bias") ||
            !check_shape(L.k_k, {H, H}, li + "key_kernel") || !check_shape(L.k_b, {H}, li + "key_bias") ||
            !check_shape(L.v_k, {H, H}, li + "value_kernel") || !check_shape(L.v_b, {H}, li + "value_bias") ||
            !check_shape(L.ao_k, {H, H}, li + "attention_output_dense_kernel") ||
            !check_shape(L.ao_b, {H}, li + "attention_output_dense_bias") ||
            !check_shape(L.ao_g, {H}, li + "attention_output_LayerNorm_gamma") ||
            !check_shape(L.ao_be, {H}, li + "attention_output_LayerNorm_beta") ||
            !check_shape(L.in_k, {H, I}, li + "intermediate_dense_kernel") ||
            !check_shape(L.in_b, {I}, li + "intermediate_dense_bias") ||
            !check_shape(L.out_k, {I, H}, li + "output_dense_kernel") ||
            !check_shape(L.out_b, {H}, li + "output_dense_bias") ||
            !check_shape(L.out_g, {H}, li + "output_LayerNorm_gamma") ||
            !check_shape(L.out_be, {H}, li + "output_LayerNorm_beta"))
            return false;
    }
    if (!ok) return false;
    out->pool_k = need({"pooler_dense_kernel"});
    out->pool_b = need({"pooler_dense_bias"});
    if (!ok) return false;
    if (!check_shape(out->pool_k, {H, H}, "pooler_dense_kernel") || !check_shape(out->pool_b, {H}, "pooler_dense_bias"))
        return false;

    // Optional fine-tune head (apps/finetune.py:33-34).
    out->cls_k = find_unique(*out, {"classifier_kernel"}, false, &ok);
    out->cls_b = find_unique(*out, {"classifier_bias"}, false, &ok);
    if (!ok) return false;
    if (out->cls_k && out->cls_b) {
        if (out->cls_k->shape.size() != 2 || out->cls_k->shape[0] != H || out->cls_k->shape[1] < 1 ||
            out->cls_k->shape[1] > 8) {
            set_error("classifier_kernel must be [hidden, C] with 1 <= C <= 8");
            return false;
        }
        if (!check_shape(out->cls_b, {out->cls_k->shape[1]}, "classifier_bias")) return false;
        out->num_classes = (int)out->cls_k->shape[1];
    } else {
        out->cls_k = out->cls_b = nullptr;
    }
    return true;
}

}  // namespace cubert
