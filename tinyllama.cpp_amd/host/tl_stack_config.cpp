// tl_stack_config.cpp — loader of the layer-list families (tl_registry.hpp): config.json -> tl_stack_config, model.safetensors
// -> tl_model_set_tensor_named. Every size and every constant that can differ between two models of a design is read from
// the file (or, for an inner size the configuration does not name, from a tensor's shape); what a design fixes is set here.
//
// Ralasun   post-norm blocks with one-plus RMS norms, an embedding norm, softmax window attention with whole-projection q/k
//           norm and value mixing, routed experts g * sigmoid(1.702 g) * (u + 1) with clamps, softmax over the chosen logits.
//   {"architecture", "width", "vocab", "norm": {"eps"}, "layers": [{"type": "attention",
//     "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"}, "v_mix"},
//     "mlp": null | {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff", "limit"}, "shared": null | {"ff", "limit"}}}]}
// Madalorn  parallel blocks behind one Dynamic Tanh norm; "attention" = sigmoid-weighted window attention whose values are
//           the keys as projected, rotary positions with a context extension, per-head unit norm, kept first keys;
//           "channel_delta" = gated delta rule with a decay per key channel; feed-forward dense or routed (softmax over all
//           experts, groups) with a gated shared expert, plain silu gated units; layers may reuse an earlier layer's tensors;
//           capped logits.
//   {"architecture", "width", "vocab", "norm": {"eps"}, "logit_softcap", "layers": [{"type": "attention" | "channel_delta",
//     "weights_of": j, "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size", "keep_first"},
//     "rot": {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}}, "conv"},
//     "mlp": null | {"kind": "dense", "ff"} | {"kind": "moe", "router": {"experts", "top", "groups": {"count", "keep"}},
//     "expert": {"ff"}, "shared": null | {"ff"}}}]}
// Sogalix   pre-norm blocks with layer norms (weight and bias), an embedding norm; three mixers: "attention" = causal softmax
//           attention over grouped key/value heads with a sink in the denominator and a query temperature that grows with the
//           logarithm of the position, no rotation; "latent_attention" = queries and keys/values through normalised latents,
//           one rotated key part shared by the heads, a gate per head, optionally on an earlier layer's cache (kv_from);
//           "general_delta" = generalized delta rule with decay exp(-e^-1/2 sigmoid(.)) and a removal rate per key channel;
//           feed-forward W_down act(W_up h) with a two-parameter activation (mlp.act).
//   {"architecture", "width", "vocab", "norm": {"eps"}, "layers": [{"type": "attention" | "latent_attention" | "general_delta",
//     "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "q_temp": {"coef", "every"}} |
//              {"heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "rot": {"base", "dims"}, "kv_from": j} |
//              {"heads", "dim"},
//     "mlp": null | {"kind": "dense", "ff"}}]}
// Potipel   pre-norm blocks with plain RMS norms; the embedding row is scaled; what each sublayer reads is h + conv(h), a causal
//           convolution over time per channel (canon.taps). Mixers: "attention" = differential attention (two score maps per
//           head over the same values, per-head q/k RMS norm, lambda from four vectors, sigmoid output gate, causal);
//           "hgrn2" = gated linear attention whose forget gate also decides what is written; "parallel" = two mixers side by
//           side, left a sliding-window attention (biases, a convolution on q, k, v, capped scores, a logarithmic distance
//           bias, a learned sink per head), right the gated delta rule with one decay per head and a silu gate, summed with
//           left_scale / right_scale. Feed-forward: a relu-gated unit, or routed experts (sigmoid scores with a correction for
//           the choice, groups ranked by their two best, weights not normalised) of the clamped 1.702-swish form. Layers may
//           reuse an earlier layer's tensors.
//   {"architecture", "width", "vocab", "norm": {"eps"}, "embedding": {"scale"}, "canon": {"taps"}, "layers": [{"type":
//     "attention" | "hgrn2" | "parallel", "weights_of": j,
//     "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "diff"} | {"heads", "dim", "vdim"} |
//              {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "conv", "mask": {"size"}},
//               "right": {"heads", "kv_heads", "dim", "vdim", "conv"}, "left_scale", "right_scale"},
//     "mlp": null | {"kind": "dense", "ff"} | {"kind": "moe", "router": {"experts", "top", "groups": {"count", "keep"}},
//     "expert": {"ff", "limit"}}}]}
#include <chrono>
#include <cmath>
#include <fstream>
#include <sstream>
#include <stdexcept>

#include "tl_json.hpp"
#include "tl_registry.hpp"
#include "tl_safetensors.hpp"

namespace tlhost {

namespace {

constexpr float kGateAlpha = 1.702f;   // Ralasun: g * sigmoid(1.702 g), fixed by the design
const float kGDeltaDecayScale = 0.60653065971263342f;  // Sogalix: decay = exp(-e^(-1/2) * sigmoid(.)), fixed by the design
constexpr int kDefaultContext = 4096;  // cache rows when the caller names no context length

void hip_check(int rc, const std::string& what) {
  if (rc != 0) throw std::runtime_error("tlhip: " + what + ": " + tl_last_error());
}

int geti(const Json& o, const char* key) { return (int)o.at(key).as_int(key); }
float getf(const Json& o, const char* key) { return (float)o.at(key).as_double(key); }
const Json* present(const Json& o, const char* key) {
  const Json* v = o.find(key);
  return (v && !v->is_null()) ? v : nullptr;
}

tl_layer_spec ralasun_layer(const Json& L, int index, const SafeTensorsFile&) {
  const std::string where = "layers[" + std::to_string(index) + "]";
  tl_layer_spec sp = {};
  const std::string& type = L.at("type").as_string("type");
  if (type != "attention") throw std::runtime_error(where + ": unknown layer type \"" + type + "\"");
  const Json& mx = L.at("mixer");
  sp.mixer = TL_MIXER_SWA;
  sp.block = TL_BLOCK_POST_NORM;
  sp.heads = geti(mx, "heads");
  sp.kv_heads = geti(mx, "kv_heads");
  sp.dim = geti(mx, "dim");
  sp.vdim = geti(mx, "vdim");
  sp.scale = getf(mx, "scale");
  const Json* mask = present(mx, "mask");
  sp.window = mask ? geti(*mask, "size") : 0;
  const Json* vm = mx.find("v_mix");
  sp.v_mix = vm && vm->truthy();
  sp.qk_norm = TL_QK_NORM_WHOLE;
  sp.act_alpha = kGateAlpha;
  sp.glu_up_add = 1.0f;
  if (const Json* ml = present(L, "mlp")) {
    const Json* kind = ml->find("kind");
    if (kind && kind->as_string("kind") != "moe")
      throw std::runtime_error(where + ": unknown feed-forward kind \"" + kind->str + "\"");
    sp.mlp = TL_MLP_MOE;
    sp.route = TL_ROUTE_TOP_LOGITS;
    sp.experts = geti(ml->at("router"), "experts");
    sp.top = geti(ml->at("router"), "top");
    sp.expert_ff = geti(ml->at("expert"), "ff");
    sp.expert_limit = getf(ml->at("expert"), "limit");
    if (const Json* sh = present(*ml, "shared")) {
      sp.shared_ff = geti(*sh, "ff");
      sp.shared_limit = getf(*sh, "limit");
    }
  }
  return sp;
}

// an inner size that only a tensor's shape gives
int tensor_rows(const SafeTensorsFile& file, const std::string& name) {
  const SafeTensor* t = file.find(name);
  if (!t || t->shape.size() != 2) throw std::runtime_error("model.safetensors: no matrix named " + name);
  return (int)t->shape[0];
}

tl_layer_spec madalorn_layer(const Json& layers, int index, const SafeTensorsFile& file) {
  const Json& L = layers.arr[index];
  const std::string where = "layers[" + std::to_string(index) + "]";
  tl_layer_spec sp = {};
  const std::string& type = L.at("type").as_string("type");
  const Json& mx = L.at("mixer");
  int src = index;
  if (const Json* wo = present(L, "weights_of")) {
    src = (int)wo->as_int("weights_of");
    if (src < 0 || src >= index) throw std::runtime_error(where + ": weights_of must name an earlier layer");
    sp.weights_of = src + 1;
    while (const Json* more = present(layers.arr[src], "weights_of")) {  // the owner of the tensors, for the sizes shapes give
      const int next = (int)more->as_int("weights_of");
      if (next < 0 || next >= src) throw std::runtime_error(where + ": weights_of must name an earlier layer");
      src = next;
    }
  }
  sp.block = TL_BLOCK_PARALLEL;
  sp.heads = geti(mx, "heads");
  sp.kv_heads = geti(mx, "kv_heads");
  sp.dim = geti(mx, "dim");
  sp.vdim = geti(mx, "vdim");
  sp.act_alpha = 1.0f;  // silu
  sp.glu_up_add = 0.0f;
  sp.expert_limit = sp.shared_limit = INFINITY;
  if (type == "attention") {
    sp.mixer = TL_MIXER_SWA;
    sp.scale = getf(mx, "scale");
    sp.attn_weight = TL_ATTN_SIGMOID;
    sp.values_are_keys = 1;
    sp.qk_norm = TL_QK_NORM_HEAD_UNIT;
    if (const Json* mask = present(mx, "mask")) {
      sp.window = geti(*mask, "size");
      if (const Json* kf = present(*mask, "keep_first")) sp.keep_first = (int)kf->as_int("keep_first");
    }
    if (const Json* rot = present(mx, "rot")) {
      sp.rot_dims = geti(*rot, "dims");
      sp.rot_base = getf(*rot, "base");
      if (const Json* sc = present(*rot, "scaling")) {
        sp.rot_factor = getf(*sc, "factor");
        sp.rot_original = getf(*sc, "original");
        sp.rot_fast = getf(*sc, "fast");
        sp.rot_slow = getf(*sc, "slow");
      }
    }
  } else if (type == "channel_delta") {
    sp.mixer = TL_MIXER_DELTA;
    sp.conv_taps = geti(mx, "conv");
    const std::string p = "l" + std::to_string(src) + ".mix.";
    sp.decay_rank = tensor_rows(file, p + "a1");
    sp.gate_rank = tensor_rows(file, p + "g1");
  } else {
    throw std::runtime_error(where + ": unknown layer type \"" + type + "\"");
  }
  if (const Json* ml = present(L, "mlp")) {
    const std::string& kind = ml->at("kind").as_string("kind");
    if (kind == "dense") {
      sp.mlp = TL_MLP_DENSE;
      sp.shared_ff = geti(*ml, "ff");
    } else if (kind == "moe") {
      sp.mlp = TL_MLP_MOE;
      sp.route = TL_ROUTE_SOFTMAX_GROUPS;
      const Json& r = ml->at("router");
      sp.experts = geti(r, "experts");
      sp.top = geti(r, "top");
      sp.route_groups = sp.route_keep = 1;
      if (const Json* g = present(r, "groups")) {
        sp.route_groups = geti(*g, "count");
        sp.route_keep = geti(*g, "keep");
      }
      sp.expert_ff = geti(ml->at("expert"), "ff");
      if (const Json* sh = present(*ml, "shared")) {
        sp.shared_ff = geti(*sh, "ff");
        sp.shared_gate = 1;
      }
    } else {
      throw std::runtime_error(where + ": unknown feed-forward kind \"" + kind + "\"");
    }
  }
  return sp;
}

tl_layer_spec sogalix_layer(const Json& layers, int index, const SafeTensorsFile& file) {
  const Json& L = layers.arr[index];
  const std::string where = "layers[" + std::to_string(index) + "]";
  tl_layer_spec sp = {};
  const std::string& type = L.at("type").as_string("type");
  const Json& mx = L.at("mixer");
  sp.block = TL_BLOCK_PRE_NORM;
  sp.heads = geti(mx, "heads");
  sp.dim = geti(mx, "dim");
  if (type == "attention") {
    sp.mixer = TL_MIXER_SWA;
    sp.kv_heads = present(mx, "kv_heads") ? geti(mx, "kv_heads") : sp.heads;  // (no entry: a key/value head per query head)
    sp.vdim = present(mx, "vdim") ? geti(mx, "vdim") : sp.dim;
    sp.scale = getf(mx, "scale");
    sp.attn_weight = TL_ATTN_SOFTMAX_SINK;  // the sink is part of the design
    if (const Json* qt = present(mx, "q_temp")) {
      sp.q_temp_coef = getf(*qt, "coef");
      sp.q_temp_every = geti(*qt, "every");
      if (sp.q_temp_every <= 0) throw std::runtime_error(where + ": q_temp.every must be positive");
    }
  } else if (type == "latent_attention") {
    sp.mixer = TL_MIXER_LATENT;
    sp.kv_heads = sp.heads;
    sp.vdim = geti(mx, "vdim");
    sp.scale = getf(mx, "scale");
    sp.rot_dim = geti(mx, "rot_dim");
    sp.q_rank = geti(mx, "q_rank");
    sp.kv_rank = geti(mx, "kv_rank");
    sp.head_gate = 1;
    if (const Json* rot = present(mx, "rot")) {
      sp.rot_dims = geti(*rot, "dims");
      sp.rot_base = getf(*rot, "base");
    }
    if (const Json* kf = present(mx, "kv_from")) {
      const int j = (int)kf->as_int("kv_from");
      if (j < 0 || j >= index) throw std::runtime_error(where + ": kv_from must name an earlier layer");
      sp.kv_from = j + 1;
    }
  } else if (type == "general_delta") {
    sp.mixer = TL_MIXER_GDELTA;
    sp.kv_heads = sp.heads;
    sp.vdim = sp.dim;
    sp.decay_scale = kGDeltaDecayScale;
    sp.decay_rank = tensor_rows(file, "l" + std::to_string(index) + ".mix.w1");
  } else {
    throw std::runtime_error(where + ": unknown layer type \"" + type + "\"");
  }
  if (const Json* ml = present(L, "mlp")) {
    const std::string& kind = ml->at("kind").as_string("kind");
    if (kind != "dense") throw std::runtime_error(where + ": unknown feed-forward kind \"" + kind + "\"");
    sp.mlp = TL_MLP_UNIT;
    sp.act = TL_ACT_XIELU;
    sp.shared_ff = geti(*ml, "ff");
  }
  return sp;
}

// `side` receives the second mixer of a "parallel" layer (the returned entry points at it)
tl_layer_spec potipel_layer(const Json& layers, int index, tl_layer_spec* side) {
  const Json& L = layers.arr[index];
  const std::string where = "layers[" + std::to_string(index) + "]";
  tl_layer_spec sp = {};
  const std::string& type = L.at("type").as_string("type");
  const Json& mx = L.at("mixer");
  if (const Json* wo = present(L, "weights_of")) {
    const int src = (int)wo->as_int("weights_of");
    if (src < 0 || src >= index) throw std::runtime_error(where + ": weights_of must name an earlier layer");
    sp.weights_of = src + 1;
  }
  sp.block = TL_BLOCK_PRE_NORM;
  if (type == "attention") {
    sp.mixer = TL_MIXER_SWA;
    sp.heads = geti(mx, "heads");
    sp.kv_heads = present(mx, "kv_heads") ? geti(mx, "kv_heads") : sp.heads;
    sp.dim = geti(mx, "dim");
    sp.vdim = present(mx, "vdim") ? geti(mx, "vdim") : sp.dim;
    sp.scale = getf(mx, "scale");
    sp.score_maps = 2;
    sp.diff_init = getf(mx, "diff");
    sp.qk_norm = TL_QK_NORM_HEAD_RMS;
    sp.out_gate = 1;
  } else if (type == "hgrn2") {
    sp.mixer = TL_MIXER_LINEAR;
    sp.heads = sp.kv_heads = geti(mx, "heads");
    sp.dim = geti(mx, "dim");
    sp.vdim = present(mx, "vdim") ? geti(mx, "vdim") : sp.dim;
  } else if (type == "parallel") {
    const Json& lt = mx.at("left");
    sp.mixer = TL_MIXER_SWA;
    sp.heads = geti(lt, "heads");
    sp.kv_heads = present(lt, "kv_heads") ? geti(lt, "kv_heads") : sp.heads;
    sp.dim = geti(lt, "dim");
    sp.vdim = present(lt, "vdim") ? geti(lt, "vdim") : sp.dim;
    sp.scale = getf(lt, "scale");
    sp.score_softcap = present(lt, "softcap") ? getf(lt, "softcap") : 0.0f;
    sp.qkv_bias = 1;
    sp.qkv_conv = geti(lt, "conv");
    sp.dist_bias = 1;
    sp.attn_weight = TL_ATTN_SOFTMAX_LEARNED_SINK;
    if (const Json* mask = present(lt, "mask")) sp.window = geti(*mask, "size");
    const Json& rt = mx.at("right");
    tl_layer_spec r = {};
    r.mixer = TL_MIXER_DELTA;
    r.heads = geti(rt, "heads");
    r.kv_heads = present(rt, "kv_heads") ? geti(rt, "kv_heads") : r.heads;
    r.dim = geti(rt, "dim");
    r.vdim = present(rt, "vdim") ? geti(rt, "vdim") : r.dim;
    r.conv_taps = geti(rt, "conv");
    r.decay_per_head = 1;
    r.block = TL_BLOCK_PRE_NORM;
    *side = r;
    sp.side = side;
    sp.mix_scale = getf(mx, "left_scale");
    sp.side_scale = getf(mx, "right_scale");
  } else {
    throw std::runtime_error(where + ": unknown layer type \"" + type + "\"");
  }
  if (const Json* ml = present(L, "mlp")) {
    const std::string& kind = ml->at("kind").as_string("kind");
    if (kind == "dense") {
      sp.mlp = TL_MLP_DENSE;
      sp.glu = TL_GLU_RELU;
      sp.shared_ff = geti(*ml, "ff");
    } else if (kind == "moe") {
      sp.mlp = TL_MLP_MOE;
      sp.glu = TL_GLU_SWISH;
      sp.act_alpha = kGateAlpha;
      sp.glu_up_add = 1.0f;
      sp.route = TL_ROUTE_SIGMOID_GROUPS;
      const Json& r = ml->at("router");
      sp.experts = geti(r, "experts");
      sp.top = geti(r, "top");
      sp.route_groups = sp.route_keep = 1;
      if (const Json* g = present(r, "groups")) {
        sp.route_groups = geti(*g, "count");
        sp.route_keep = geti(*g, "keep");
      }
      sp.expert_ff = geti(ml->at("expert"), "ff");
      sp.expert_limit = getf(ml->at("expert"), "limit");
    } else {
      throw std::runtime_error(where + ": unknown feed-forward kind \"" + kind + "\"");
    }
  }
  return sp;
}

}  // namespace

void load_stack_folder(const std::string& dir, int device, int max_context, LoadedModel* out) {
  const auto t0 = std::chrono::steady_clock::now();
  std::ifstream in(dir + "/config.json");
  if (!in) throw std::runtime_error("cannot open " + dir + "/config.json");
  std::stringstream ss;
  ss << in.rdbuf();
  const Json cfg = Json::parse(ss.str());
  const Json& layers = cfg.at("layers");
  if (layers.kind != Json::ARRAY || layers.arr.empty()) throw std::runtime_error("config.json: \"layers\" is empty");
  const std::string arch = cfg.at("architecture").as_string("architecture");
  const bool madalorn = arch == "Madalorn", sogalix = arch == "Sogalix", potipel = arch == "Potipel";
  SafeTensorsFile file;
  file.open(dir + "/model.safetensors");
  std::vector<tl_layer_spec> specs, sides(layers.arr.size());  // (sides: second mixers, addressed by the entries of specs)
  for (size_t i = 0; i < layers.arr.size(); ++i)
    specs.push_back(madalorn  ? madalorn_layer(layers, (int)i, file)
                    : sogalix ? sogalix_layer(layers, (int)i, file)
                    : potipel ? potipel_layer(layers, (int)i, &sides[i])
                              : ralasun_layer(layers.arr[i], (int)i, file));
  tl_stack_config sc = {};
  sc.width = geti(cfg, "width");
  sc.vocab = geti(cfg, "vocab");
  sc.n_layers = (int)specs.size();
  sc.max_positions = max_context > 0 ? max_context : kDefaultContext;
  sc.norm_eps = (float)cfg.at("norm").at("eps").as_double("norm.eps");
  sc.layers = specs.data();
  sc.norm = madalorn ? TL_NORM_DYT : sogalix ? TL_NORM_LAYER : potipel ? TL_NORM_RMS : TL_NORM_RMS_ONE_PLUS;
  sc.embed_norm = madalorn || potipel ? 0 : 1;
  if (potipel) {
    sc.embed_scale = (float)cfg.at("embedding").at("scale").as_double("embedding.scale");
    sc.canon_taps = (int)cfg.at("canon").at("taps").as_int("canon.taps");
  }
  if (madalorn)
    if (const Json* cap = present(cfg, "logit_softcap")) sc.logit_softcap = (float)cap->as_double("logit_softcap");

  ModelConfig& mc = out->config;
  mc.architecture = cfg.at("architecture").as_string("architecture");
  mc.name = mc.architecture;
  mc.hidden_size = sc.width;
  mc.vocab_size = sc.vocab;
  mc.num_hidden_layers = sc.n_layers;
  mc.max_position_embeddings = sc.max_positions;
  mc.rms_norm_eps = sc.norm_eps;
  mc.num_attention_heads = specs[0].heads;
  mc.num_key_value_heads = specs[0].kv_heads;
  mc.intermediate_size = specs[0].mlp == TL_MLP_DENSE || specs[0].mlp == TL_MLP_UNIT ? specs[0].shared_ff : specs[0].expert_ff;
  mc.bos_token_id = -1;  // token ids in, token ids out: such a checkpoint carries no tokenizer
  mc.eos_token_id = -1;
  if (const Json* e = cfg.find("eos"))
    if (e->kind == Json::NUMBER) mc.eos_token_id = (int)e->as_int("eos");

  hip_check(tl_init(device), "tl_init");
  hip_check(tl_model_create_stack(&sc, &out->model), "tl_model_create_stack");
  try {
    for (const SafeTensor& t : file.tensors()) {
      int type = -1;
      if (t.dtype == "BF16") type = TL_BF16;
      else if (t.dtype == "F32") type = TL_F32;
      else if (t.dtype == "I32" || t.dtype == "I64") continue;  // integer tables belong to other designs
      else throw std::runtime_error("tensor " + t.name + " has dtype " + t.dtype + "; this family holds BF16 (and F32 vectors)");
      hip_check(tl_model_set_tensor_named(out->model, t.name.c_str(), type, t.shape.data(), (int)t.shape.size(), t.data),
                "tl_model_set_tensor_named " + t.name);
      ++out->stats.tensors;
      out->stats.quantized_bytes += t.nbytes;
    }
    hip_check(tl_model_finalize(out->model), "tl_model_finalize");
  } catch (...) {
    tl_model_free(out->model);
    out->model = nullptr;
    throw;
  }
  out->multi_sequence = false;
  out->exact_terms = 3;
  out->serving_terms = 1;
  out->stats.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

}  // namespace tlhost
