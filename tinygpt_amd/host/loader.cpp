#include "loader.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <set>
#include <sstream>

#include "json.h"

namespace tgxh {

namespace {

bool read_file(const std::string& path, std::string& out) {
  std::ifstream ifs(path, std::ios::binary);
  if (!ifs.is_open()) return false;
  std::stringstream ss;
  ss << ifs.rdbuf();
  out = ss.str();
  return true;
}

bool file_exists(const std::string& p) { struct stat st; return stat(p.c_str(), &st) == 0; }

std::string join_path(const std::string& a, const std::string& b) { return (a.empty() || a.back() == '/') ? a + b : a + "/" + b; }
std::string base_dir(const std::string& p) { size_t k = p.find_last_of('/'); return k == std::string::npos ? "." : p.substr(0, k); }

int family_of(const std::string& t) {
  if (t == "gpt2") return TGX_FAMILY_GPT2;
  if (t == "llama") return TGX_FAMILY_LLAMA;
  if (t == "qwen2") return TGX_FAMILY_QWEN2;
  if (t == "qwen3") return TGX_FAMILY_QWEN3;
  if (t == "mistral") return TGX_FAMILY_MISTRAL;
  return 0;
}

}  // namespace

// every dimension the device shim allocates from must be a positive 32-bit integer (a missing key or a value of the wrong JSON type reads as -1)
static bool check_dims(const tgx_model_desc& d, const std::string& path, std::string& err) {
  struct { const char* name; int64_t v; } f[] = {{"hidden size", d.hidden}, {"layer count", d.layers}, {"attention heads", d.heads}, {"key/value heads", d.kv_heads},
                                                 {"head_dim", d.head_dim}, {"intermediate size", d.inter}, {"vocab_size", d.vocab}, {"context size", d.max_ctx}};
  for (auto& e : f)
    if (e.v <= 0 || e.v > (int64_t)1 << 30) { err = "config.json: " + std::string(e.name) + " is missing, not an integer or out of range in " + path; return false; }
  return true;
}

// one entry of a Modepel config's "layers": {"type": "attention" | "mlstm", "mixer": {...}, "mlp": null | {"kind": "dense" | "moe", ...}}
static bool load_modepel_layer(const Json& L, size_t i, tgx_layer_desc& l, std::string& err) {
  auto dim = [](const Json& j, const char* key) -> int32_t { const int64_t v = j.get_int(key, -1); return (v < 0 || v > ((int64_t)1 << 30)) ? -1 : (int32_t)v; };
  const Json* mx = L.get("mixer");
  const Json* ff = L.get("mlp");
  const std::string type = L.get_str("type", "");
  if ((type != "attention" && type != "mlstm") || !mx || mx->kind != Json::Obj) { err = "config.json: layer " + std::to_string(i) + ": mixer '" + type + "' is not implemented"; return false; }
  l.heads = dim(*mx, "heads"); l.dim = dim(*mx, "dim"); l.vdim = dim(*mx, "vdim");
  if (type == "attention") {
    l.mixer = TGX_MIXER_ATTENTION;
    l.kv_heads = dim(*mx, "kv_heads"); l.scale = mx->get_float("scale", 1.f);
    const Json* vm = mx->get("v_mix");
    l.v_mix = vm && vm->kind == Json::Bool && vm->b ? 1 : 0;
    const Json* rot = mx->get("rot");
    if (rot && rot->kind == Json::Obj) { l.rot_dims = dim(*rot, "dims"); l.rot_base = rot->get_float("base", 10000.f); }
  } else {
    l.mixer = TGX_MIXER_MLSTM;
    l.gate_cap = mx->get_float("gate_cap", 0.f);
  }
  if (!ff || ff->kind != Json::Obj) return true;
  const std::string kind = ff->get_str("kind", "");
  if (kind == "dense") { l.mlp = TGX_MLP_DENSE; l.ff = dim(*ff, "ff"); return true; }
  const Json* ex = ff->get("expert");
  const Json* ro = ff->get("router");
  if (kind != "moe" || !ro || ro->kind != Json::Obj) { err = "config.json: layer " + std::to_string(i) + ": feed-forward kind '" + kind + "' is not implemented"; return false; }
  l.mlp = TGX_MLP_MOE;
  l.experts = dim(*ro, "experts"); l.top = dim(*ro, "top"); l.router_scale = ro->get_float("scale", 1.f);
  l.identity = ro->has("identity") ? dim(*ro, "identity") : 0;
  const Json* gr = ro->get("groups");
  l.groups = 1; l.groups_keep = 1;
  if (gr && gr->kind == Json::Obj) { l.groups = dim(*gr, "count"); l.groups_keep = gr->has("keep") ? dim(*gr, "keep") : l.groups; }
  l.ff = l.experts > 0 && ex && ex->kind == Json::Obj ? dim(*ex, "ff") : 0;
  const Json* sh = ff->get("shared");
  l.shared_ff = sh && sh->kind == Json::Obj ? dim(*sh, "ff") : 0;
  return true;
}

// the attention entries of a Vitudra mixer (an "attention" layer's, or the "left" half of a "parallel" one); what is absent is off
static void load_vitudra_attention(const Json& m, int mask_kind, tgx_layer_desc& l) {
  auto dim = [](const Json& j, const char* key) -> int32_t { const int64_t v = j.get_int(key, -1); return (v < 0 || v > ((int64_t)1 << 30)) ? -1 : (int32_t)v; };
  l.heads = dim(m, "heads"); l.kv_heads = m.has("kv_heads") ? dim(m, "kv_heads") : l.heads; l.dim = dim(m, "dim"); l.vdim = m.has("vdim") ? dim(m, "vdim") : l.dim;
  l.scale = m.get_float("scale", 1.f); l.softcap = m.get_float("softcap", 0.f);
  const Json* mask = m.get("mask");
  if (mask && mask->kind == Json::Obj) { l.mask_kind = mask_kind; l.mask_size = dim(*mask, "size"); }
  const Json* rot = m.get("rot");
  if (rot && rot->kind == Json::Obj) {
    l.rot_dims = dim(*rot, "dims"); l.rot_base = rot->get_float("base", 10000.f); l.rot_pairs = 1; l.rot_factor = 1.f;
    const Json* sc = rot->get("scaling");
    if (sc && sc->kind == Json::Obj) l.rot_factor = sc->get_float("factor", 1.f);
  }
  const Json* qt = m.get("q_temp");
  if (qt && qt->kind == Json::Obj) { l.q_temp_coef = qt->get_float("coef", 0.f); l.q_temp_every = dim(*qt, "every"); }
}

// one entry of a Vitudra config's "layers": {"type": "attention" | "wkv" | "parallel", "mixer": {...}, "mlp": null | {"kind": "dense", "ff"}}.  An attention
// layer has a sliding window, a distance bias and a query temperature and may read another layer's keys and values ("kv_from"); a parallel mixer is
// {"left": attention with neighbour-pair rotation, soft cap and chunked mask, "right": gated delta rule, "left_scale", "right_scale"}.  A wkv layer's decay
// rank is left open: the device library takes it from the tensor's shape.
static bool load_vitudra_layer(const Json& L, size_t i, tgx_layer_desc& l, std::string& err) {
  auto dim = [](const Json& j, const char* key) -> int32_t { const int64_t v = j.get_int(key, -1); return (v < 0 || v > ((int64_t)1 << 30)) ? -1 : (int32_t)v; };
  const Json* mx = L.get("mixer");
  const Json* ff = L.get("mlp");
  const std::string type = L.get_str("type", "");
  auto bad = [&](const std::string& what) { err = "config.json: layer " + std::to_string(i) + ": " + what; return false; };
  if (!mx || mx->kind != Json::Obj) return bad("no mixer");
  if (type == "attention") {
    l.mixer = TGX_MIXER_ATTENTION;
    load_vitudra_attention(*mx, TGX_MASK_WINDOW, l);
    l.dist_bias = 1;
    if (mx->has("kv_from")) { const int32_t j = dim(*mx, "kv_from"); if (j < 0) return bad("kv_from"); l.kv_share = j + 1; }
  } else if (type == "wkv") {
    l.mixer = TGX_MIXER_WKV;
    l.heads = dim(*mx, "heads"); l.dim = dim(*mx, "dim"); l.vdim = l.dim; l.kv_heads = l.heads;
  } else if (type == "parallel") {
    const Json* left = mx->get("left");
    const Json* right = mx->get("right");
    if (!left || left->kind != Json::Obj || !right || right->kind != Json::Obj) return bad("a parallel mixer needs left and right");
    l.mixer = TGX_MIXER_PARALLEL;
    load_vitudra_attention(*left, TGX_MASK_CHUNK, l);
    l.d_heads = dim(*right, "heads"); l.d_kv_heads = right->has("kv_heads") ? dim(*right, "kv_heads") : l.d_heads; l.d_dim = dim(*right, "dim");
    l.d_vdim = right->has("vdim") ? dim(*right, "vdim") : l.d_dim; l.conv_taps = right->has("conv") ? dim(*right, "conv") : 1;
    l.left_scale = mx->get_float("left_scale", 1.f); l.right_scale = mx->get_float("right_scale", 1.f);
  } else return bad("mixer '" + type + "' is not implemented");
  if (!ff || ff->kind != Json::Obj) return true;
  if (ff->get_str("kind", "") != "dense") return bad("feed-forward kind '" + ff->get_str("kind", "") + "' is not implemented");
  l.mlp = TGX_MLP_DENSE; l.ff = dim(*ff, "ff");
  return true;
}

// one entry of a Zaluvik config's "layers": {"type": "attention" | "latent_attention", "mixer": {...}, "mlp": null | {"kind": "dense" | "moe", ...}}.
// Attention: unit queries and keys, a sliding window, sigmoid weights with a per-head bias mixed across heads, a gate per output channel.  Latent attention:
// rot_dim rotated dimensions beside dim per head, one rotated key part for all heads, a sliding window, softmax, a gate per head.  Dense feed-forwards use
// the erf gelu; experts are chosen by sigmoid scores inside the best groups (a group counts as the sum of its two largest scores), weights normalised.
static bool load_zaluvik_layer(const Json& L, size_t i, tgx_layer_desc& l, std::string& err) {
  auto dim = [](const Json& j, const char* key) -> int32_t { const int64_t v = j.get_int(key, -1); return (v < 0 || v > ((int64_t)1 << 30)) ? -1 : (int32_t)v; };
  const Json* mx = L.get("mixer");
  const Json* ff = L.get("mlp");
  const std::string type = L.get_str("type", "");
  auto bad = [&](const std::string& what) { err = "config.json: layer " + std::to_string(i) + ": " + what; return false; };
  if (!mx || mx->kind != Json::Obj) return bad("no mixer");
  l.heads = dim(*mx, "heads"); l.dim = dim(*mx, "dim"); l.vdim = mx->has("vdim") ? dim(*mx, "vdim") : l.dim; l.scale = mx->get_float("scale", 1.f);
  const Json* mask = mx->get("mask");
  if (mask && mask->kind == Json::Obj) { l.mask_kind = TGX_MASK_WINDOW; l.mask_size = dim(*mask, "size"); }
  if (type == "attention") {
    l.mixer = TGX_MIXER_ATTENTION;
    l.kv_heads = mx->has("kv_heads") ? dim(*mx, "kv_heads") : l.heads;
    l.qk_norm = 1; l.score_fn = 1; l.head_mix = 1; l.gate_kind = 1;
  } else if (type == "latent_attention") {
    l.mixer = TGX_MIXER_LATENT_ATTENTION;
    l.kv_rank = dim(*mx, "kv_rank"); l.rot_dim = mx->has("rot_dim") ? dim(*mx, "rot_dim") : 0; l.gate_kind = 2;
    const Json* rot = mx->get("rot");
    l.rot_dims = l.rot_dim; l.rot_base = 10000.f;
    if (rot && rot->kind == Json::Obj) { if (rot->has("dims")) l.rot_dims = dim(*rot, "dims"); l.rot_base = rot->get_float("base", 10000.f); }
    if (l.rot_dim <= 0) l.rot_dims = 0;
  } else return bad("mixer '" + type + "' is not implemented");
  if (!ff || ff->kind != Json::Obj) return true;
  const std::string kind = ff->get_str("kind", "");
  if (kind == "dense") { l.mlp = TGX_MLP_DENSE; l.ff = dim(*ff, "ff"); l.ff_act = 1; return true; }
  const Json* ex = ff->get("expert");
  const Json* ro = ff->get("router");
  if (kind != "moe" || !ro || ro->kind != Json::Obj || !ex || ex->kind != Json::Obj) return bad("feed-forward kind '" + kind + "' is not implemented");
  l.mlp = TGX_MLP_MOE;
  l.experts = dim(*ro, "experts"); l.top = dim(*ro, "top"); l.ff = dim(*ex, "ff"); l.router_scale = 1.f;
  l.router_fn = 1; l.group_score = 1; l.router_norm = 1;
  const Json* gr = ro->get("groups");
  l.groups = 1; l.groups_keep = 1;
  if (gr && gr->kind == Json::Obj) { l.groups = dim(*gr, "count"); l.groups_keep = gr->has("keep") ? dim(*gr, "keep") : l.groups; }
  const Json* sh = ff->get("shared");
  l.shared_ff = sh && sh->kind == Json::Obj ? dim(*sh, "ff") : 0;
  return true;
}

// config.json of a layered model: {"architecture": "Zakusun", "width", "vocab", "logit_scale", "norm": {"eps", "groups"}, "canon": {"taps"},
// "layers": [{"type": mixer, "mixer": {heads, dim, vdim, kv_rank, scale}, "mlp": null | {"kind": "moe", "expert": {ff, limit}, "router": {experts, top}}}]}
// or {"architecture": "Modepel", "width", "vocab", "norm": {"eps"}, "layers": [...]} with the layer entries of load_modepel_layer
// or {"architecture": "Vitudra", "width", "vocab", "residual_mult", "norm": {"eps"}, "layers": [...]} with the layer entries of load_vitudra_layer
// or {"architecture": "Zaluvik", "width", "vocab", "residual_mult", "embedding": {"scale"}, "loop": {"start", "stop", "times"}, "norm": {"eps"}, "layers": [...]}
// with the layer entries of load_zaluvik_layer (logits against the embedding table)
static bool load_stack_config(const Json& doc, const std::string& path, int compute_dtype, int max_batch, int max_ctx, int budget_tokens, ModelConfig& out, std::string& err) {
  const std::string arch = doc.get_str("architecture", "");
  const bool vitudra = arch == "Vitudra", zaluvik = arch == "Zaluvik", modepel = arch == "Modepel" || vitudra || zaluvik;      // (all three: a config header without norm groups, taps and logit scale)
  if (arch != "Zakusun" && !modepel) { err = "Unsupported architecture: " + arch; return false; }
  auto dim = [](const Json& j, const char* key) -> int32_t { const int64_t v = j.get_int(key, -1); return (v < 0 || v > ((int64_t)1 << 30)) ? -1 : (int32_t)v; };
  out.layered = true;
  out.model_type = zaluvik ? "zaluvik" : vitudra ? "vitudra" : modepel ? "modepel" : "zakusun";
  tgx_stack_desc& s = out.stack;
  s.family = zaluvik ? TGX_FAMILY_ZALUVIK : vitudra ? TGX_FAMILY_VITUDRA : modepel ? TGX_FAMILY_MODEPEL : TGX_FAMILY_ZAKUSUN;
  s.residual_mult = doc.get_float("residual_mult", 1.f);
  s.embed_scale = 1.f; s.loop_times = 1;
  if (zaluvik) {
    const Json* em = doc.get("embedding");
    if (em && em->kind == Json::Obj) s.embed_scale = em->get_float("scale", 1.f);
    const Json* lp = doc.get("loop");
    if (lp && lp->kind == Json::Obj) { s.loop_start = dim(*lp, "start"); s.loop_stop = dim(*lp, "stop"); s.loop_times = dim(*lp, "times"); }
  }
  s.width = dim(doc, "width"); s.vocab = dim(doc, "vocab"); s.compute_dtype = compute_dtype;
  s.max_seqs = max_batch < 1 ? 1 : max_batch;
  s.max_ctx = max_ctx > 0 ? max_ctx : 4096;
  s.budget_tokens = budget_tokens > 0 ? budget_tokens : 0;
  s.page_tokens = 0;
  s.logit_scale = modepel ? 1.f : doc.get_float("logit_scale", 1.f);
  const Json* norm = doc.get("norm");
  const Json* canon = doc.get("canon");
  const Json* layers = doc.get("layers");
  if (!norm || norm->kind != Json::Obj || (!modepel && (!canon || canon->kind != Json::Obj)) || !layers || layers->kind != Json::Arr || layers->arr.empty()) {
    err = "config.json: norm / canon / layers are missing in " + path; return false;
  }
  s.norm_groups = modepel ? 1 : dim(*norm, "groups"); s.norm_eps = norm->get_float("eps", 1e-6f); s.canon_taps = modepel ? 1 : dim(*canon, "taps");
  for (size_t i = 0; i < layers->arr.size(); i++) {
    const Json& L = layers->arr[i];
    tgx_layer_desc l{};
    if (modepel) {
      if (!(zaluvik ? load_zaluvik_layer(L, i, l, err) : vitudra ? load_vitudra_layer(L, i, l, err) : load_modepel_layer(L, i, l, err))) return false;
      out.layers.push_back(l);
      continue;
    }
    const Json* mx = L.get("mixer");
    const Json* ff = L.get("mlp");
    const std::string type = L.get_str("type", "");
    if (type != "latent_attention" || !mx || mx->kind != Json::Obj) { err = "config.json: layer " + std::to_string(i) + ": mixer '" + type + "' is not implemented"; return false; }
    l.mixer = TGX_MIXER_LATENT_ATTENTION;
    l.heads = dim(*mx, "heads"); l.dim = dim(*mx, "dim"); l.vdim = dim(*mx, "vdim"); l.kv_rank = dim(*mx, "kv_rank"); l.scale = mx->get_float("scale", 1.f);
    if (ff && ff->kind == Json::Obj) {
      const Json* ex = ff->get("expert");
      const Json* ro = ff->get("router");
      if (ff->get_str("kind", "") != "moe" || !ex || !ro) { err = "config.json: layer " + std::to_string(i) + ": feed-forward kind '" + ff->get_str("kind", "") + "' is not implemented"; return false; }
      l.mlp = TGX_MLP_MOE;
      l.ff = dim(*ex, "ff"); l.limit = ex->get_float("limit", 0.f); l.experts = dim(*ro, "experts"); l.top = dim(*ro, "top");
    }
    out.layers.push_back(l);
  }
  s.layers = (int32_t)out.layers.size();
  tgx_model_desc& d = out.desc;
  d.family = s.family; d.hidden = s.width; d.layers = s.layers; d.vocab = s.vocab; d.max_ctx = s.max_ctx; d.max_batch = s.max_seqs; d.compute_dtype = compute_dtype; d.tied = modepel && !zaluvik ? 0 : 1;
  if (s.width <= 0 || s.vocab <= 0 || s.norm_groups <= 0 || s.canon_taps <= 0) { err = "config.json: width / vocab / norm.groups / canon.taps missing or out of range in " + path; return false; }
  return true;
}

bool load_model_config(const std::string& path, int compute_dtype, int max_batch, ModelConfig& out, std::string& err, int max_ctx, int budget_tokens) {
  std::string text;
  if (!read_file(path, text) || text.empty()) { err = "Failed to open file: " + path; return false; }
  Json doc;
  if (!JsonParser::parse(text.data(), text.size(), doc) || doc.kind != Json::Obj) { err = "JSON parse error in: " + path; return false; }
  out = ModelConfig();
  if (!doc.has("model_type") && doc.has("architecture")) return load_stack_config(doc, path, compute_dtype, max_batch, max_ctx, budget_tokens, out, err);
  out.model_type = doc.get_str("model_type", "");
  if (out.model_type.empty()) { err = "Missing or invalid model_type in config.json"; return false; }
  const int fam = family_of(out.model_type);
  if (!fam) { err = "Unsupported model_type: " + out.model_type; return false; }
  tgx_model_desc& d = out.desc;
  d.family = fam;
  d.compute_dtype = compute_dtype;
  d.max_batch = max_batch < 1 ? 1 : max_batch;
  // 64-bit values are range-checked before narrowing (2^32 + 5 must not read as 5)
  auto dim = [](const Json& j, const char* key, int64_t def) -> int32_t { const int64_t v = j.get_int(key, def); return (v < 0 || v > ((int64_t)1 << 30)) ? -1 : (int32_t)v; };
  out.torch_dtype = doc.get_str("torch_dtype", doc.get_str("dtype", ""));
  out.bos_token_id = doc.get_int("bos_token_id", -1);
  out.eos_token_id = doc.get_int("eos_token_id", -1);
  d.vocab = dim(doc, "vocab_size", -1);
  if (fam == TGX_FAMILY_GPT2) {
    d.hidden = dim(doc, "n_embd", -1);
    d.layers = dim(doc, "n_layer", -1);
    d.heads = d.kv_heads = dim(doc, "n_head", -1);
    d.head_dim = d.heads > 0 ? d.hidden / d.heads : 0;
    d.inter = 4 * d.hidden;
    d.n_positions = dim(doc, "n_positions", -1);
    d.max_ctx = dim(doc, "n_ctx", d.n_positions);      // contextSize = n_ctx (ModelGPT2.h:230)
    d.norm_eps = doc.get_float("layer_norm_epsilon", 1e-5f);
    d.qkv_bias = 1; d.tied = 1;
    return check_dims(d, path, err);
  }
  d.hidden = dim(doc, "hidden_size", -1);
  d.layers = dim(doc, "num_hidden_layers", -1);
  d.heads = dim(doc, "num_attention_heads", -1);
  d.kv_heads = dim(doc, "num_key_value_heads", d.heads);
  d.inter = dim(doc, "intermediate_size", -1);
  d.max_ctx = dim(doc, "max_position_embeddings", -1);
  d.norm_eps = doc.get_float("rms_norm_eps", 1e-5f);
  d.tied = doc.get_bool("tie_word_embeddings", false) ? 1 : 0;
  d.head_dim = d.heads > 0 ? d.hidden / d.heads : 0;               // ModelLlama.h:37 ignores "head_dim"
  if (fam == TGX_FAMILY_QWEN3) d.head_dim = dim(doc, "head_dim", d.head_dim);   // ModelQwen3.h:25
  d.qkv_bias = fam == TGX_FAMILY_QWEN2 ? 1 : 0;                    // ModelQwen2.h:26-31
  d.qk_norm = fam == TGX_FAMILY_QWEN3 ? 1 : 0;                     // AttentionWithQKNorm (ModelQwen3.h:29-33)
  // rope: hub-era flat keys (what the reference parses) or the nested rope_parameters newer transformers write
  const Json* rp = doc.get("rope_parameters");
  const Json* rs = doc.get("rope_scaling");
  if ((!rs || rs->kind != Json::Obj) && rp && rp->kind == Json::Obj && rp->get_str("rope_type", "default") != "default") rs = rp;
  const float def_theta = fam == TGX_FAMILY_LLAMA ? 1.f : 10000.f;  // ModelConfig.cpp:88,91,99
  float theta = doc.get_float("rope_theta", -1.f);
  if (theta < 0.f) theta = (rp && rp->kind == Json::Obj) ? rp->get_float("rope_theta", def_theta) : def_theta;
  d.rope_theta = theta;
  if (fam == TGX_FAMILY_LLAMA && rs && rs->kind == Json::Obj) {     // ModelConfig.cpp:79-87
    d.rope_factor = rs->get_float("factor", 1.f);
    d.rope_high_freq = rs->get_float("high_freq_factor", 1.f);
    d.rope_low_freq = rs->get_float("low_freq_factor", 1.f);
    d.rope_orig_ctx = dim(*rs, "original_max_position_embeddings", -1);
    if (d.rope_orig_ctx > 0) d.max_ctx = d.rope_orig_ctx;           // getContextSize (ModelLlama.h:26-31)
  }
  return check_dims(d, path, err);
}

bool load_generation_config(const std::string& path, GenerationConfig& out, std::string& err) {
  std::string text;
  if (!read_file(path, text) || text.empty()) { err = "Failed to open file: " + path; return false; }
  Json doc;
  if (!JsonParser::parse(text.data(), text.size(), doc) || doc.kind != Json::Obj) { err = "JSON parse error in: " + path; return false; }
  out = GenerationConfig();
  out.bos_token_id = doc.get_int("bos_token_id", -1);
  if (const Json* e = doc.get("eos_token_id")) {
    if (e->kind == Json::Arr) { for (const Json& v : e->arr) if (v.kind == Json::Num && v.is_int) out.eos_token_ids.push_back(v.i); }
    else if (e->kind == Json::Num && e->is_int) out.eos_token_ids.push_back(e->i);
  }
  out.do_sample = doc.get_bool("do_sample", false);
  out.temperature = doc.get_float("temperature", 0.f);
  out.top_k = doc.get_int("top_k", 0);
  out.top_p = doc.get_float("top_p", 1.f);
  return true;
}

namespace {

// one .safetensors file: u64 header size | JSON header | data (SafeTensors.cpp:141-229)
bool load_one(const Backend& be, tgx_ctx* ctx, const std::string& path, const std::set<std::string>* only, int& loaded, std::string& err) {
  int fd = ::open(path.c_str(), O_RDONLY);
  if (fd < 0) { err = "Error mapFileForRead: " + path; return false; }
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 8) { ::close(fd); err = "Error mapFileForRead: " + path; return false; }
  void* map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
  ::close(fd);
  if (map == MAP_FAILED) { err = "Error mapFileForRead: " + path; return false; }
  bool ok = true;
  const uint64_t header_size = *static_cast<const uint64_t*>(map);
  // st_size >= 8 was checked above; written so that a header_size near 2^64 cannot wrap past the check
  if (header_size > (uint64_t)st.st_size - 8) { err = "corrupt safetensors header: " + path; munmap(map, (size_t)st.st_size); return false; }
  const char* header = static_cast<const char*>(map) + 8;
  const char* data = header + header_size;
  const uint64_t data_size = (uint64_t)st.st_size - 8 - header_size;
  Json doc;
  if (!JsonParser::parse(header, (size_t)header_size, doc) || doc.kind != Json::Obj) { err = "safetensors header is not JSON: " + path; ok = false; }
  for (size_t t = 0; ok && t < doc.obj.size(); t++) {
    const std::string& name = doc.obj[t].first;
    if (name == "__metadata__") continue;
    if (only && !only->count(name)) continue;
    const Json& info = doc.obj[t].second;
    const Json* shape = info.get("shape");
    const Json* off = info.get("data_offsets");
    const std::string dt = info.get_str("dtype", "");
    if (!shape || shape->kind != Json::Arr || !off || off->kind != Json::Arr || off->arr.size() != 2) { err = "bad tensor entry: " + name; ok = false; break; }
    int src = -1;
    size_t esz = 0;
    if (dt == "BF16") { src = TGX_BF16; esz = 2; } else if (dt == "F16") { src = TGX_F16; esz = 2; } else if (dt == "F32") { src = TGX_F32; esz = 4; }
    std::vector<int64_t> dims;
    uint64_t numel = 1;
    bool shape_ok = true;
    for (const Json& v : shape->arr) {      // non-negative integers whose product (times the element size) stays inside 64 bits
      if (v.kind != Json::Num || !v.is_int || v.i < 0) { shape_ok = false; break; }
      if (v.i != 0 && numel > (UINT64_MAX / 8) / (uint64_t)v.i) { shape_ok = false; break; }
      dims.push_back(v.i); numel *= (uint64_t)v.i;
    }
    if (!shape_ok || off->arr[0].kind != Json::Num || !off->arr[0].is_int || off->arr[0].i < 0 || off->arr[1].kind != Json::Num || !off->arr[1].is_int || off->arr[1].i < 0) {
      err = "bad tensor entry: " + name; ok = false; break;
    }
    if (src < 0) {
      // a dtype this path never consumes (I64 position_ids, BOOL / U8 mask buffers of old hub checkpoints): the reference looks the name
      // up first and only warns about keys it does not know (SafeTensors.cpp:176-183) — ask the shim whether it wants the tensor
      static const float probe = 0.f;
      static const int64_t no_dims = 0;
      const int prc = be.upload(ctx, name.c_str(), &probe, dims.empty() ? &no_dims : dims.data(), -1, TGX_F32);     // nd = -1: name lookup only, nothing is copied
      if (prc == TGX_ERR_NAME) { fprintf(stderr, "[tgx] Unexpected key: %s\n", name.c_str()); continue; }
      if (prc == TGX_OK) continue;                                                         // a known non-parameter buffer (GPT-2's attn.bias masks)
      err = "dtype not supported for tensor: " + name + " (" + dt + ")"; ok = false; break;
    }
    const uint64_t b0 = (uint64_t)off->arr[0].i, b1 = (uint64_t)off->arr[1].i;
    if (b1 < b0 || b1 > data_size || b1 - b0 != numel * esz) { err = "size not equal for tensor: " + name; ok = false; break; }
    const int rc = be.upload(ctx, name.c_str(), data + b0, dims.data(), (int)dims.size(), src);
    if (rc == TGX_ERR_NAME) { fprintf(stderr, "[tgx] Unexpected key: %s\n", name.c_str()); continue; }   // non-strict load
    if (rc != TGX_OK) { err = std::string(be.last_error(ctx)); ok = false; break; }
    loaded++;
  }
  munmap(map, (size_t)st.st_size);
  return ok;
}

}  // namespace

bool load_safetensors(const Backend& be, tgx_ctx* ctx, const std::string& path, int& loaded, std::string& err) {
  loaded = 0;
  auto ends_with = [](const std::string& s, const std::string& suf) { return suf.size() <= s.size() && !s.compare(s.size() - suf.size(), suf.size(), suf); };
  if (ends_with(path, ".safetensors")) return load_one(be, ctx, path, nullptr, loaded, err);
  if (!ends_with(path, ".index.json")) { err = "Unknown file type: " + path; return false; }
  std::string text;
  if (!read_file(path, text)) { err = "Error open index file: " + path; return false; }
  Json doc;
  if (!JsonParser::parse(text.data(), text.size(), doc) || doc.kind != Json::Obj) { err = "Invalid index json: " + path; return false; }
  const Json* wm = doc.get("weight_map");
  if (!wm || wm->kind != Json::Obj) { err = "Index json missing weight_map"; return false; }
  std::map<std::string, std::set<std::string>> shard2keys;          // SafeTensors.cpp:258-263
  for (const auto& kv : wm->obj) if (kv.second.kind == Json::Str) shard2keys[kv.second.str].insert(kv.first);
  const std::string dir = base_dir(path);
  for (const auto& sk : shard2keys)
    if (!load_one(be, ctx, join_path(dir, sk.first), &sk.second, loaded, err)) { err = "Failed to load shard: " + sk.first + ": " + err; return false; }
  return true;
}

bool load_model_dir(const Backend& be, const std::string& dir, int device_ordinal, int compute_dtype, int max_batch,
                    LoadedModel& out, std::string& err, int max_ctx, int budget_tokens) {
  if (!load_model_config(join_path(dir, "config.json"), compute_dtype, max_batch, out.config, err, max_ctx, budget_tokens)) return false;
  if (out.config.layered) {      // generation_config.json is optional for a layered model (no HF export defines one)
    if (file_exists(join_path(dir, "generation_config.json")) && !load_generation_config(join_path(dir, "generation_config.json"), out.generation, err)) return false;
    if (!be.create_stack) { err = "the device shim does not provide layered models (tgx_create_stack)"; return false; }
  } else if (!load_generation_config(join_path(dir, "generation_config.json"), out.generation, err)) return false;   // required (ModelLoader.cpp:34-38)
  int rc = out.config.layered ? be.create_stack(&out.config.stack, out.config.layers.data(), device_ordinal, &out.ctx) : be.create(&out.config.desc, device_ordinal, &out.ctx);
  if (rc != TGX_OK) { err = std::string("create failed: ") + be.last_error(out.ctx); if (out.ctx) be.destroy(out.ctx); out.ctx = nullptr; return false; }
  std::string mp = join_path(dir, "model.safetensors");
  if (!file_exists(mp)) mp = join_path(dir, "model.safetensors.index.json");          // ModelLoader.cpp:72-75
  int loaded = 0;
  if (!load_safetensors(be, out.ctx, mp, loaded, err)) { be.destroy(out.ctx); out.ctx = nullptr; return false; }
  rc = be.finalize(out.ctx);
  if (rc != TGX_OK) { err = std::string("Load model failed: ") + be.last_error(out.ctx); be.destroy(out.ctx); out.ctx = nullptr; return false; }
  return true;
}

}  // namespace tgxh
