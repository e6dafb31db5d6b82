"""Model description for the decode path: the Python mirror of ``tgx_model_desc`` (include/tgx.h).

The field set and the parsing rules restate what the reference reads from an HF ``config.json``
(reference: src/huggingface/ModelConfig.cpp:43-125) and how each family factory turns it into
layer hyper-parameters (src/model/ModelLlama.h:21-53, ModelQwen2.h:23-45, ModelMistral.h:23-40,
ModelGPT2.h:226-230).  Both the hub-era flat keys the reference parses (``rope_theta``,
``rope_scaling``, ``torch_dtype``) and the nested ``rope_parameters`` / ``dtype`` keys newer
``transformers`` writes are accepted.
"""
from __future__ import annotations

import ctypes
import json
import os
from dataclasses import dataclass, field, asdict

# tgx_family (include/tgx.h)
FAMILY_GPT2, FAMILY_LLAMA, FAMILY_QWEN2, FAMILY_QWEN3, FAMILY_MISTRAL = 1, 2, 3, 4, 5
FAMILY_BY_NAME = {"gpt2": FAMILY_GPT2, "llama": FAMILY_LLAMA, "qwen2": FAMILY_QWEN2,
                  "qwen3": FAMILY_QWEN3, "mistral": FAMILY_MISTRAL}
# tgx_dtype (include/tgx.h)
DTYPE_F32, DTYPE_BF16, DTYPE_F16 = 0, 1, 2
DTYPE_BY_NAME = {"float32": DTYPE_F32, "fp32": DTYPE_F32, "bfloat16": DTYPE_BF16, "bf16": DTYPE_BF16,
                 "float16": DTYPE_F16, "fp16": DTYPE_F16}


class CDesc(ctypes.Structure):
    """ctypes image of ``struct tgx_model_desc`` — keep in lock-step with include/tgx.h."""
    _fields_ = [
        ("family", ctypes.c_int32),
        ("hidden", ctypes.c_int32),
        ("layers", ctypes.c_int32),
        ("heads", ctypes.c_int32),
        ("kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("inter", ctypes.c_int32),
        ("vocab", ctypes.c_int32),
        ("max_ctx", ctypes.c_int32),
        ("qkv_bias", ctypes.c_int32),
        ("tied", ctypes.c_int32),
        ("compute_dtype", ctypes.c_int32),
        ("norm_eps", ctypes.c_float),
        ("rope_theta", ctypes.c_float),
        ("rope_factor", ctypes.c_float),
        ("rope_low_freq", ctypes.c_float),
        ("rope_high_freq", ctypes.c_float),
        ("rope_orig_ctx", ctypes.c_int32),
        ("n_positions", ctypes.c_int32),
        ("max_batch", ctypes.c_int32),
        ("qk_norm", ctypes.c_int32),
    ]


@dataclass
class ModelDesc:
    family: str = "llama"
    hidden: int = 0
    layers: int = 0
    heads: int = 0
    kv_heads: int = 0
    head_dim: int = 0
    inter: int = 0
    vocab: int = 0
    max_ctx: int = 0            # == GPTModel::contextSize(): KV-cache capacity and RoPE table length
    qkv_bias: bool = False
    tied: bool = False
    compute_dtype: str = "bf16"  # the CLI's --dtype; weights are cast to it after load
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_factor: float = 0.0     # 0 => no llama3 scaling (std::nullopt in Qwen2/Mistral factories)
    rope_low_freq: float = 1.0
    rope_high_freq: float = 1.0
    rope_orig_ctx: int = 0
    n_positions: int = 0         # GPT-2 learned position table rows
    max_batch: int = 1
    qk_norm: bool = False        # Qwen3: per-head RMSNorm on q, k before RoPE (Attention.h:128-167)
    name: str = ""               # label only (bench/config reporting)

    # ---- derived sizes -------------------------------------------------------------------
    @property
    def q_dim(self): return self.heads * self.head_dim

    @property
    def kv_dim(self): return self.kv_heads * self.head_dim

    def to_c(self) -> CDesc:
        return CDesc(FAMILY_BY_NAME[self.family], self.hidden, self.layers, self.heads, self.kv_heads,
                     self.head_dim, self.inter, self.vocab, self.max_ctx, int(self.qkv_bias), int(self.tied),
                     DTYPE_BY_NAME[self.compute_dtype], self.norm_eps, self.rope_theta, self.rope_factor,
                     self.rope_low_freq, self.rope_high_freq, self.rope_orig_ctx, self.n_positions,
                     self.max_batch, int(self.qk_norm))

    def to_dict(self):
        return asdict(self)

    # ---- tensor inventory (HF checkpoint names the reference loads by, SafeTensors.cpp:157-215) ----
    def tensor_shapes(self) -> "dict[str, tuple]":
        H, I, V = self.hidden, self.inter, self.vocab
        out = {}
        if self.family == "gpt2":
            # hub layout without the "transformer." prefix (ModelGPT2.h:226)
            out["wte.weight"] = (V, H)
            out["wpe.weight"] = (self.n_positions, H)
            for i in range(self.layers):
                p = f"h.{i}."
                out[p + "ln_1.weight"] = (H,); out[p + "ln_1.bias"] = (H,)
                out[p + "attn.c_attn.weight"] = (H, 3 * H); out[p + "attn.c_attn.bias"] = (3 * H,)
                out[p + "attn.c_proj.weight"] = (H, H); out[p + "attn.c_proj.bias"] = (H,)
                out[p + "ln_2.weight"] = (H,); out[p + "ln_2.bias"] = (H,)
                out[p + "mlp.c_fc.weight"] = (H, 4 * H); out[p + "mlp.c_fc.bias"] = (4 * H,)
                out[p + "mlp.c_proj.weight"] = (4 * H, H); out[p + "mlp.c_proj.bias"] = (H,)
            out["ln_f.weight"] = (H,); out["ln_f.bias"] = (H,)
            return out
        out["model.embed_tokens.weight"] = (V, H)
        for i in range(self.layers):
            p = f"model.layers.{i}."
            out[p + "input_layernorm.weight"] = (H,)
            out[p + "self_attn.q_proj.weight"] = (self.q_dim, H)
            out[p + "self_attn.k_proj.weight"] = (self.kv_dim, H)
            out[p + "self_attn.v_proj.weight"] = (self.kv_dim, H)
            if self.qkv_bias:
                out[p + "self_attn.q_proj.bias"] = (self.q_dim,)
                out[p + "self_attn.k_proj.bias"] = (self.kv_dim,)
                out[p + "self_attn.v_proj.bias"] = (self.kv_dim,)
            if self.qk_norm:
                out[p + "self_attn.q_norm.weight"] = (self.head_dim,)
                out[p + "self_attn.k_norm.weight"] = (self.head_dim,)
            out[p + "self_attn.o_proj.weight"] = (H, self.q_dim)
            out[p + "post_attention_layernorm.weight"] = (H,)
            out[p + "mlp.gate_proj.weight"] = (I, H)
            out[p + "mlp.up_proj.weight"] = (I, H)
            out[p + "mlp.down_proj.weight"] = (H, I)
        out["model.norm.weight"] = (H,)
        if not self.tied:
            out["lm_head.weight"] = (V, H)
        return out

    def param_count(self) -> int:
        n = 0
        for s in self.tensor_shapes().values():
            k = 1
            for d in s:
                k *= d
            n += k
        return n

    # ---- algorithmic HBM bytes per decoded token at context T ------------
    def bytes_per_token(self, T: int, elem: int = 2) -> int:
        H, I, V, L = self.hidden, self.inter, self.vocab, self.layers
        q, kv = self.q_dim, self.kv_dim
        if self.family == "gpt2":   # c_attn, c_proj, c_fc, mlp.c_proj with biases, two LayerNorms (w + b); ln_f, one wpe row, the wte head
            per_layer = 3 * H * H + 3 * H + H * H + H + I * H + I + H * I + H + 4 * H
            return elem * (L * per_layer + 2 * H + H + V * H) + elem * 2 * L * kv * T
        per_layer = (q + 2 * kv) * H + ((q + 2 * kv) if self.qkv_bias else 0) + H * q + 2 * I * H + H * I + 2 * H
        return elem * (L * per_layer + H + V * H) + elem * 2 * L * kv * T


def desc_from_hf_config(cfg: dict, compute_dtype: str = "bf16", max_batch: int = 1) -> ModelDesc:
    """config.json dict -> ModelDesc, following ModelConfig.cpp:63-122 and the family factories."""
    mt = cfg.get("model_type", "")
    if mt not in FAMILY_BY_NAME:
        raise ValueError(f"Unsupported model_type: {mt!r}")          # ModelConfig.cpp:108-110
    if mt == "gpt2":
        E = int(cfg.get("n_embd", -1))
        return ModelDesc(family="gpt2", hidden=E, layers=int(cfg.get("n_layer", -1)), heads=int(cfg.get("n_head", -1)),
                         kv_heads=int(cfg.get("n_head", -1)), head_dim=E // int(cfg.get("n_head", 1)), inter=4 * E,
                         vocab=int(cfg.get("vocab_size", -1)),
                         max_ctx=int(cfg.get("n_ctx", cfg.get("n_positions", -1))),   # contextSize = n_ctx (ModelGPT2.h:230)
                         qkv_bias=True, tied=True, compute_dtype=compute_dtype,
                         norm_eps=float(cfg.get("layer_norm_epsilon", 1e-5)), rope_theta=0.0,
                         n_positions=int(cfg.get("n_positions", -1)), max_batch=max_batch, name=cfg.get("_name_or_path", ""))
    rp = cfg.get("rope_parameters") or {}
    rs = cfg.get("rope_scaling") or {}
    if not rs and rp.get("rope_type", "default") not in ("default", None):
        rs = rp
    default_theta = 1.0 if mt == "llama" else 10000.0                  # ModelConfig.cpp:88,91,99
    theta = float(cfg.get("rope_theta", rp.get("rope_theta", default_theta)))
    heads = int(cfg["num_attention_heads"])
    hidden = int(cfg["hidden_size"])
    head_dim = hidden // heads                                         # ModelLlama.h:37 ignores "head_dim"
    if mt == "qwen3":
        head_dim = int(cfg.get("head_dim", head_dim))                  # ModelQwen3.h:25
    d = ModelDesc(family=mt, hidden=hidden, layers=int(cfg["num_hidden_layers"]), heads=heads,
                  kv_heads=int(cfg.get("num_key_value_heads", heads)), head_dim=head_dim,
                  inter=int(cfg["intermediate_size"]), vocab=int(cfg["vocab_size"]),
                  max_ctx=int(cfg.get("max_position_embeddings", -1)),
                  qkv_bias=(mt == "qwen2"),                            # ModelQwen2.h:26-31
                  tied=bool(cfg.get("tie_word_embeddings", False)),
                  compute_dtype=compute_dtype, norm_eps=float(cfg.get("rms_norm_eps", 1e-5)),
                  rope_theta=theta, max_batch=max_batch, qk_norm=(mt == "qwen3"), name=cfg.get("_name_or_path", ""))
    if mt == "llama" and rs:
        d.rope_factor = float(rs.get("factor", 1.0))
        d.rope_high_freq = float(rs.get("high_freq_factor", 1.0))
        d.rope_low_freq = float(rs.get("low_freq_factor", 1.0))
        d.rope_orig_ctx = int(rs.get("original_max_position_embeddings", -1))
        if d.rope_orig_ctx > 0:
            d.max_ctx = d.rope_orig_ctx                                # ModelLlama.h:26-31
    return d


def load_desc(model_dir: str, compute_dtype: str = "bf16", max_batch: int = 1, **stack_kw):
    """the model class by config.json: "model_type" names a flat family (ModelDesc), "architecture" a layered one (StackDesc; stack_kw = max_ctx, budget_tokens)"""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    if is_stack_config(cfg):
        return stack_desc_from_config(cfg, compute_dtype, max_seqs=max_batch, **stack_kw)
    return desc_from_hf_config(cfg, compute_dtype, max_batch)


# ---- the public HF hyper-parameters of BASELINE.json's configs (SURVEY.md §8 header) --------
def _llama(name, H, L, nh, nkv, I, V, tied, theta=500000.0, scaled=True, max_pos=131072):
    cfg = {"model_type": "llama", "hidden_size": H, "num_hidden_layers": L, "num_attention_heads": nh,
           "num_key_value_heads": nkv, "intermediate_size": I, "vocab_size": V, "tie_word_embeddings": tied,
           "rms_norm_eps": 1e-5, "rope_theta": theta, "max_position_embeddings": max_pos, "torch_dtype": "bfloat16",
           "_name_or_path": name}
    if scaled:
        cfg["rope_scaling"] = {"factor": 32.0, "high_freq_factor": 4.0, "low_freq_factor": 1.0,
                               "original_max_position_embeddings": 8192, "rope_type": "llama3"}
    return cfg


KNOWN_CONFIGS = {
    "llama-3.2-1b": _llama("Llama-3.2-1B", 2048, 16, 32, 8, 8192, 128256, True),
    "llama-3.2-3b": _llama("Llama-3.2-3B", 3072, 28, 24, 8, 8192, 128256, True),
    "qwen2.5-0.5b": {"model_type": "qwen2", "hidden_size": 896, "num_hidden_layers": 24, "num_attention_heads": 14,
                     "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936,
                     "tie_word_embeddings": True, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
                     "max_position_embeddings": 32768, "torch_dtype": "bfloat16", "_name_or_path": "Qwen2.5-0.5B"},
    "mistral-7b-v0.3": {"model_type": "mistral", "hidden_size": 4096, "num_hidden_layers": 32,
                        "num_attention_heads": 32, "num_key_value_heads": 8, "intermediate_size": 14336,
                        "vocab_size": 32768, "tie_word_embeddings": False, "rms_norm_eps": 1e-5,
                        "rope_theta": 1000000.0, "max_position_embeddings": 32768, "torch_dtype": "bfloat16",
                        "_name_or_path": "Mistral-7B-v0.3"},
    # the other checkpoints the reference's README names (README.md:50-56), public config.json values
    "qwen2.5-3b": {"model_type": "qwen2", "hidden_size": 2048, "num_hidden_layers": 36, "num_attention_heads": 16,
                   "num_key_value_heads": 2, "intermediate_size": 11008, "vocab_size": 151936,
                   "tie_word_embeddings": True, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
                   "max_position_embeddings": 32768, "torch_dtype": "bfloat16", "_name_or_path": "Qwen2.5-3B"},
    "qwen3-1.7b": {"model_type": "qwen3", "hidden_size": 2048, "num_hidden_layers": 28, "num_attention_heads": 16,
                   "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 6144, "vocab_size": 151936,
                   "tie_word_embeddings": True, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
                   "max_position_embeddings": 40960, "torch_dtype": "bfloat16", "attention_bias": False,
                   "_name_or_path": "Qwen3-1.7B"},
    # 70B-class geometry (Llama-3.1-70B): 141 GB of bf16 parameters — one MI355X holds it in its 288 GB of HBM3E
    "llama-3.1-70b": {"model_type": "llama", "hidden_size": 8192, "num_hidden_layers": 80, "num_attention_heads": 64,
                      "num_key_value_heads": 8, "intermediate_size": 28672, "vocab_size": 128256,
                      "tie_word_embeddings": False, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
                      "max_position_embeddings": 131072, "torch_dtype": "bfloat16", "_name_or_path": "Llama-3.1-70B",
                      "rope_scaling": {"factor": 8.0, "high_freq_factor": 4.0, "low_freq_factor": 1.0,
                                       "original_max_position_embeddings": 8192, "rope_type": "llama3"}},
    # Qwen3-0.6B (public config.json): per-head q/k RMSNorm, explicit head_dim 128 with q_dim 2048 != hidden 1024
    "qwen3-0.6b": {"model_type": "qwen3", "hidden_size": 1024, "num_hidden_layers": 28, "num_attention_heads": 16,
                   "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 3072, "vocab_size": 151936,
                   "tie_word_embeddings": True, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
                   "max_position_embeddings": 40960, "torch_dtype": "bfloat16", "attention_bias": False,
                   "_name_or_path": "Qwen3-0.6B"},
    "gpt2": {"model_type": "gpt2", "n_embd": 768, "n_layer": 12, "n_head": 12, "n_ctx": 1024, "n_positions": 1024,
             "vocab_size": 50257, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
             "torch_dtype": "float32", "_name_or_path": "gpt2"},
}


def known_desc(key: str, compute_dtype: str | None = None, max_batch: int = 1) -> ModelDesc:
    cfg = KNOWN_CONFIGS[key.lower()]
    if compute_dtype is None:
        compute_dtype = "fp32" if cfg["model_type"] == "gpt2" else "bf16"
    return desc_from_hf_config(cfg, compute_dtype, max_batch)


# ---- layered models (include/tgx.h tgx_stack_desc / tgx_layer_desc) -------------------------------------------------------------
FAMILY_ZAKUSUN = 6
FAMILY_MODEPEL = 7
FAMILY_VITUDRA = 8
FAMILY_ZALUVIK = 9
STACK_FAMILY = {"zakusun": FAMILY_ZAKUSUN, "modepel": FAMILY_MODEPEL, "vitudra": FAMILY_VITUDRA, "zaluvik": FAMILY_ZALUVIK}
MIXER_BY_NAME = {"latent_attention": 1, "attention": 2, "mlstm": 3, "wkv": 4, "parallel": 5}
MLP_BY_NAME = {None: 0, "moe": 1, "dense": 2}
MASK_BY_NAME = {None: 0, "window": 1, "chunk": 2}
# which mixers a design is made of (config.json "architecture" -> layer "type")
MIXERS_OF = {"zakusun": ("latent_attention",), "modepel": ("attention", "mlstm"), "vitudra": ("attention", "wkv", "parallel"),
             "zaluvik": ("attention", "latent_attention")}


class CLayerDesc(ctypes.Structure):
    """ctypes image of ``struct tgx_layer_desc``."""
    _fields_ = [("mixer", ctypes.c_int32), ("heads", ctypes.c_int32), ("dim", ctypes.c_int32), ("vdim", ctypes.c_int32),
                ("kv_rank", ctypes.c_int32), ("scale", ctypes.c_float), ("mlp", ctypes.c_int32), ("experts", ctypes.c_int32),
                ("top", ctypes.c_int32), ("ff", ctypes.c_int32), ("limit", ctypes.c_float),
                ("kv_heads", ctypes.c_int32), ("rot_dims", ctypes.c_int32), ("rot_base", ctypes.c_float), ("v_mix", ctypes.c_int32),
                ("gate_cap", ctypes.c_float), ("identity", ctypes.c_int32), ("groups", ctypes.c_int32), ("groups_keep", ctypes.c_int32),
                ("router_scale", ctypes.c_float), ("shared_ff", ctypes.c_int32),
                ("mask_kind", ctypes.c_int32), ("mask_size", ctypes.c_int32), ("softcap", ctypes.c_float), ("dist_bias", ctypes.c_int32),
                ("q_temp_coef", ctypes.c_float), ("q_temp_every", ctypes.c_int32), ("rot_pairs", ctypes.c_int32), ("rot_factor", ctypes.c_float),
                ("kv_share", ctypes.c_int32), ("decay_rank", ctypes.c_int32), ("d_heads", ctypes.c_int32), ("d_kv_heads", ctypes.c_int32),
                ("d_dim", ctypes.c_int32), ("d_vdim", ctypes.c_int32), ("conv_taps", ctypes.c_int32), ("left_scale", ctypes.c_float),
                ("right_scale", ctypes.c_float),
                ("qk_norm", ctypes.c_int32), ("score_fn", ctypes.c_int32), ("head_mix", ctypes.c_int32), ("gate_kind", ctypes.c_int32),
                ("rot_dim", ctypes.c_int32), ("ff_act", ctypes.c_int32), ("router_fn", ctypes.c_int32), ("group_score", ctypes.c_int32),
                ("router_norm", ctypes.c_int32)]


class CStackDesc(ctypes.Structure):
    """ctypes image of ``struct tgx_stack_desc``."""
    _fields_ = [("family", ctypes.c_int32), ("width", ctypes.c_int32), ("layers", ctypes.c_int32), ("vocab", ctypes.c_int32),
                ("compute_dtype", ctypes.c_int32), ("max_seqs", ctypes.c_int32), ("max_ctx", ctypes.c_int32),
                ("budget_tokens", ctypes.c_int32), ("page_tokens", ctypes.c_int32), ("norm_groups", ctypes.c_int32),
                ("norm_eps", ctypes.c_float), ("canon_taps", ctypes.c_int32), ("logit_scale", ctypes.c_float), ("residual_mult", ctypes.c_float),
                ("embed_scale", ctypes.c_float), ("loop_start", ctypes.c_int32), ("loop_stop", ctypes.c_int32), ("loop_times", ctypes.c_int32)]


@dataclass
class LayerDesc:
    mixer: str = "latent_attention"
    heads: int = 0
    dim: int = 0
    vdim: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    mlp: "str | None" = None      # None: the layer has no feed-forward
    experts: int = 0
    top: int = 0
    ff: int = 0
    limit: float = 0.0
    # grouped-query attention (mixer "attention")
    kv_heads: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    v_mix: bool = False
    # matrix memory (mixer "mlstm")
    gate_cap: float = 0.0
    # grouped-choice experts (Modepel's "moe"): router outputs beyond `experts` hand the input through
    identity: int = 0
    groups: int = 1
    groups_keep: int = 1
    router_scale: float = 1.0
    shared_ff: int = 0
    # attention of the parallel-sublayer design (Vitudra): mask, score shaping, rotary variant, shared keys and values
    mask: "str | None" = None     # None: causal; "window": the last mask_size positions; "chunk": the position's own block of mask_size
    mask_size: int = 0
    softcap: float = 0.0
    dist_bias: bool = False
    q_temp_coef: float = 0.0
    q_temp_every: int = 0
    rot_pairs: bool = False       # neighbours (2i, 2i + 1) turn together instead of (i, i + rot_dims / 2)
    rot_factor: float = 1.0       # every angle is divided by this
    kv_from: "int | None" = None  # the layer whose keys and values this one reads
    # token-shift mixer ("wkv")
    decay_rank: int = 0
    # the gated-delta-rule half of a "parallel" mixer (heads .. rot_* above describe its attention half)
    d_heads: int = 0
    d_kv_heads: int = 0
    d_dim: int = 0
    d_vdim: int = 0
    conv_taps: int = 0
    left_scale: float = 1.0
    right_scale: float = 1.0
    # the layer-norm design (Zaluvik): unit queries and keys, sigmoid weights mixed across heads, the kind of output gate, the rotated part of a
    # latent layer's queries and keys, the dense feed-forward's activation, the sigmoid router
    qk_norm: bool = False
    score_fn: "str | None" = None     # None: softmax; "sigmoid": sigmoid(score + per-head bias), not normalised over the keys
    head_mix: bool = False
    gate_kind: "str | None" = None    # None: the family's own; "channel" | "head"
    rot_dim: int = 0
    ff_act: "str | None" = None       # None: the family's own; "gelu"
    router_fn: "str | None" = None    # None: softmax + correction; "sigmoid"
    group_score: "str | None" = None  # None: a group's largest score; "top2": the sum of its two largest
    router_norm: bool = False

    def to_c(self) -> CLayerDesc:
        return CLayerDesc(MIXER_BY_NAME[self.mixer], self.heads, self.dim, self.vdim, self.kv_rank, self.scale,
                          MLP_BY_NAME[self.mlp], self.experts, self.top, self.ff, self.limit,
                          self.kv_heads, self.rot_dims, self.rot_base, int(self.v_mix), self.gate_cap, self.identity, self.groups,
                          self.groups_keep, self.router_scale, self.shared_ff,
                          MASK_BY_NAME[self.mask], self.mask_size, self.softcap, int(self.dist_bias), self.q_temp_coef, self.q_temp_every,
                          int(self.rot_pairs), self.rot_factor, 0 if self.kv_from is None else self.kv_from + 1, self.decay_rank,
                          self.d_heads, self.d_kv_heads, self.d_dim, self.d_vdim, self.conv_taps, self.left_scale, self.right_scale,
                          int(self.qk_norm), {None: 0, "sigmoid": 1}[self.score_fn], int(self.head_mix), {None: 0, "channel": 1, "head": 2}[self.gate_kind],
                          self.rot_dim, {None: 0, "gelu": 1}[self.ff_act], {None: 0, "sigmoid": 1}[self.router_fn], {None: 0, "top2": 1}[self.group_score],
                          int(self.router_norm))


@dataclass
class StackDesc:
    """A model described layer by layer (Zakusun, Modepel): the Python mirror of tgx_stack_desc + its tgx_layer_desc array."""
    family: str = "zakusun"
    width: int = 0
    vocab: int = 0
    layers: "list[LayerDesc]" = field(default_factory=list)
    compute_dtype: str = "bf16"
    max_seqs: int = 4            # sequence slots
    max_ctx: int = 4096          # longest sequence of a slot
    budget_tokens: int = 0       # tokens of the shared latent pool (0: max_seqs * max_ctx)
    page_tokens: int = 64
    norm_groups: int = 1
    norm_eps: float = 1e-6
    canon_taps: int = 1
    logit_scale: float = 1.0
    residual_mult: float = 1.0   # Vitudra, Zaluvik: the factor on what a (sub)layer adds to the stream
    embed_scale: float = 1.0     # Zaluvik: the factor on the embedding rows
    loop_start: int = 0          # Zaluvik: layers loop_start .. loop_stop - 1 run loop_times times with the same weights, a cache per pass
    loop_stop: int = 0
    loop_times: int = 1
    name: str = ""

    # the fields the flat description shares (bench / reporting code reads them)
    @property
    def hidden(self): return self.width

    @property
    def max_batch(self): return self.max_seqs

    def to_c(self):
        arr = (CLayerDesc * len(self.layers))(*[l.to_c() for l in self.layers])
        sd = CStackDesc(STACK_FAMILY[self.family], self.width, len(self.layers), self.vocab, DTYPE_BY_NAME[self.compute_dtype], self.max_seqs,
                        self.max_ctx, self.budget_tokens, self.page_tokens, self.norm_groups, self.norm_eps, self.canon_taps,
                        self.logit_scale, self.residual_mult, self.embed_scale, self.loop_start, self.loop_stop, self.loop_times)
        return sd, arr

    @property
    def looped(self) -> bool:
        return self.loop_times >= 1 and self.loop_stop > self.loop_start      # (a single pass still has the loop's input product in front)

    def layer_runs(self) -> "list[int]":
        """the layers in the order they run (a looped span repeats)"""
        n = len(self.layers)
        if not self.looped:
            return list(range(n))
        span = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + span * self.loop_times + list(range(self.loop_stop, n))

    def tensor_shapes(self) -> "dict[str, tuple]":
        """checkpoint name -> shape, in file order"""
        W, out = self.width, {}
        out["embed"] = (self.vocab, W)
        if self.family == "modepel":
            return self._modepel_shapes(out)
        if self.family == "vitudra":
            return _vitudra_shapes(self, out)
        if self.family == "zaluvik":
            return _zaluvik_shapes(self, out)
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = (W,)
            if l.mlp:
                out[p + "norm2"] = (W,)
            out[p + "mix.q"] = (l.heads * l.dim, W); out[p + "mix.dkv"] = (l.kv_rank, W); out[p + "mix.dkv.norm"] = (l.kv_rank,)
            out[p + "mix.uk"] = (l.heads * l.dim, l.kv_rank); out[p + "mix.uv"] = (l.heads * l.vdim, l.kv_rank)
            out[p + "mix.sink"] = (l.heads,); out[p + "mix.g"] = (l.heads * l.vdim, W); out[p + "mix.o"] = (W, l.heads * l.vdim)
            if l.mlp == "moe":
                for e in range(l.experts):
                    out[p + f"mlp.e{e}.gate"] = (l.ff, W); out[p + f"mlp.e{e}.up"] = (l.ff, W); out[p + f"mlp.e{e}.down"] = (W, l.ff)
                out[p + "mlp.router"] = (l.experts, W); out[p + "mlp.router.b"] = (l.experts,)
            out[p + "canon1"] = (W, self.canon_taps)
            if l.mlp:
                out[p + "canon2"] = (W, self.canon_taps)
            out[p + "dwa"] = (i + 2,)
        out["final.norm"] = (W,)
        return out


    def _modepel_shapes(self, out):
        W = self.width
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            for n in ("norm1", "norm2", "norm1b", "norm2b") if l.mlp else ("norm1", "norm1b"):
                out[p + n] = ()
            qd, vd = l.heads * l.dim, l.heads * l.vdim
            if l.mixer == "attention":
                kd, kv = l.kv_heads * l.dim, l.kv_heads * l.vdim
                out[p + "mix.q"] = (qd, W); out[p + "mix.q.b"] = (qd,); out[p + "mix.k"] = (kd, W); out[p + "mix.k.b"] = (kd,)
                out[p + "mix.v"] = (kv, W); out[p + "mix.v.b"] = (kv,)
                if l.v_mix:
                    out[p + "mix.vmix"] = ()
                out[p + "mix.g"] = (vd, W); out[p + "mix.o"] = (W, vd)
            else:
                out[p + "mix.q"] = (qd, W); out[p + "mix.k"] = (qd, W); out[p + "mix.v"] = (vd, W); out[p + "mix.g"] = (vd, W); out[p + "mix.o"] = (W, vd)
                out[p + "mix.norm"] = (vd,); out[p + "mix.i"] = (l.heads, W); out[p + "mix.i.b"] = (l.heads,)
                out[p + "mix.f"] = (l.heads, W); out[p + "mix.f.b"] = (l.heads,)
            if l.mlp == "dense":
                out[p + "mlp.up"] = (l.ff, W); out[p + "mlp.down"] = (W, l.ff); out[p + "mlp.act"] = (4,)
            elif l.mlp == "moe":
                for e in range(l.experts):
                    out[p + f"mlp.e{e}.gate"] = (l.ff, W); out[p + f"mlp.e{e}.up"] = (l.ff, W); out[p + f"mlp.e{e}.down"] = (W, l.ff)
                out[p + "mlp.router"] = (l.experts + l.identity, W); out[p + "mlp.correction"] = (l.experts + l.identity,)
                if l.shared_ff:
                    out[p + "mlp.shared.gate"] = (l.shared_ff, W); out[p + "mlp.shared.up"] = (l.shared_ff, W)
                    out[p + "mlp.shared.down"] = (W, l.shared_ff); out[p + "mlp.shared.sg"] = (1, W)
        out["final.norm"] = ()
        out["head"] = (self.vocab, W)
        return out


def _vitudra_shapes(self: StackDesc, out: dict) -> dict:
    """checkpoint names and shapes of a Vitudra model, in file order"""
    W = self.width
    for i, l in enumerate(self.layers):
        p = f"l{i}."
        out[p + "norm1"] = (W,)
        if l.mixer == "attention":
            out[p + "mix.q"] = (l.heads * l.dim, W)
            if l.kv_from is None:
                out[p + "mix.k"] = (l.kv_heads * l.dim, W); out[p + "mix.v"] = (l.kv_heads * l.vdim, W)
            out[p + "mix.o"] = (W, l.heads * l.vdim)
        elif l.mixer == "wkv":
            HD = l.heads * l.dim
            for s in "rkvgw":
                out[p + "mix.mu." + s] = (W,)
            for s in "rkvg":
                out[p + "mix." + s] = (HD, W)
            out[p + "mix.w1"] = (l.decay_rank, W); out[p + "mix.w2"] = (HD, l.decay_rank); out[p + "mix.w0"] = (HD,)
            out[p + "mix.u"] = (l.heads, l.dim); out[p + "mix.norm"] = (HD,); out[p + "mix.o"] = (W, HD)
        else:
            q = p + "mix.left."
            out[q + "q"] = (l.heads * l.dim, W); out[q + "k"] = (l.kv_heads * l.dim, W); out[q + "v"] = (l.kv_heads * l.vdim, W); out[q + "o"] = (W, l.heads * l.vdim)
            q = p + "mix.right."
            gd, vd = l.d_kv_heads * l.d_dim, l.d_heads * l.d_vdim
            for s, n in (("q", gd), ("k", gd), ("v", vd)):
                out[q + s] = (n, W); out[q + s + ".conv"] = (n, l.conv_taps)
            out[q + "b"] = (l.d_heads, W); out[q + "a"] = (l.d_heads, W); out[q + "A_log"] = (l.d_heads,); out[q + "dt_bias"] = (l.d_heads,)
            out[q + "norm"] = (l.d_vdim,); out[q + "g"] = (vd, W); out[q + "o"] = (W, vd)
        if l.mlp == "dense":
            out[p + "mlp.gate"] = (l.ff, W); out[p + "mlp.up"] = (l.ff, W); out[p + "mlp.down"] = (W, l.ff)
    out["final.norm"] = (W,)
    out["head"] = (self.vocab, W)
    return out



def _zaluvik_shapes(self: StackDesc, out: dict) -> dict:
    """checkpoint names and shapes of a Zaluvik model, in file order"""
    W = self.width
    if self.looped:
        out["loop.in"] = (W, 2 * W)
    for i, l in enumerate(self.layers):
        p = f"l{i}."
        for n in ("norm1", "norm2", "norm1b", "norm2b") if l.mlp else ("norm1", "norm1b"):
            out[p + n] = (W,); out[p + n + ".b"] = (W,)
        if l.mixer == "attention":
            out[p + "mix.q"] = (l.heads * l.dim, W); out[p + "mix.k"] = (l.kv_heads * l.dim, W); out[p + "mix.v"] = (l.kv_heads * l.vdim, W)
            out[p + "mix.talk"] = (l.heads, l.heads); out[p + "mix.pb"] = (l.heads,)
            out[p + "mix.g"] = (l.heads * l.vdim, W); out[p + "mix.o"] = (W, l.heads * l.vdim)
        else:
            out[p + "mix.q"] = (l.heads * (l.dim + l.rot_dim), W); out[p + "mix.dkv"] = (l.kv_rank + l.rot_dim, W); out[p + "mix.dkv.norm"] = (l.kv_rank,)
            out[p + "mix.uk"] = (l.heads * l.dim, l.kv_rank); out[p + "mix.uv"] = (l.heads * l.vdim, l.kv_rank)
            out[p + "mix.g"] = (l.heads, W); out[p + "mix.o"] = (W, l.heads * l.vdim)
        if l.mlp == "dense":
            out[p + "mlp.up"] = (l.ff, W); out[p + "mlp.down"] = (W, l.ff)
        elif l.mlp == "moe":
            for e in range(l.experts):
                out[p + f"mlp.e{e}.gate"] = (l.ff, W); out[p + f"mlp.e{e}.up"] = (l.ff, W); out[p + f"mlp.e{e}.down"] = (W, l.ff)
            out[p + "mlp.router"] = (l.experts, W)
            if l.shared_ff:
                out[p + "mlp.shared.gate"] = (l.shared_ff, W); out[p + "mlp.shared.up"] = (l.shared_ff, W); out[p + "mlp.shared.down"] = (W, l.shared_ff)
    out["final.norm"] = (W,); out["final.norm.b"] = (W,)
    return out


def _zaluvik_layer(i: int, l: dict) -> LayerDesc:
    """one entry of a Zaluvik config's "layers": {"type": "attention" | "latent_attention", "mixer": {...}, "mlp": null | {"kind": "dense" | "moe", ...}}.
    Attention: unit queries and keys, a sliding window, sigmoid weights with a per-head bias mixed across heads, a gate per output channel.
    Latent attention: `rot_dim` rotated dimensions beside `dim` per head, one rotated key part for all heads, a sliding window, softmax, a gate per head."""
    m, f = l["mixer"], l.get("mlp")
    ld = LayerDesc(mixer=l["type"], heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]))
    if m.get("mask"):
        ld.mask = "window"; ld.mask_size = int(m["mask"]["size"])
    if l["type"] == "attention":
        ld.kv_heads = int(m.get("kv_heads", m["heads"])); ld.qk_norm = True; ld.score_fn = "sigmoid"; ld.head_mix = True; ld.gate_kind = "channel"
    else:
        rot = m.get("rot") or {}
        ld.kv_rank = int(m["kv_rank"]); ld.rot_dim = int(m.get("rot_dim", 0)); ld.gate_kind = "head"
        ld.rot_dims = int(rot.get("dims", ld.rot_dim)) if ld.rot_dim else 0; ld.rot_base = float(rot.get("base", 10000.0))
        if ld.rot_dims > ld.rot_dim:
            raise ValueError(f"layer {i}: {ld.rot_dims} rotated dimensions of a rotated part of {ld.rot_dim}")
    if f is None:
        return ld
    if f.get("kind") == "dense":
        ld.mlp = "dense"; ld.ff = int(f["ff"]); ld.ff_act = "gelu"
    elif f.get("kind") == "moe":
        r, g = f["router"], f["router"].get("groups") or {}
        ld.mlp = "moe"; ld.experts = int(r["experts"]); ld.top = int(r["top"]); ld.ff = int(f["expert"]["ff"])
        ld.groups = int(g.get("count", 1)); ld.groups_keep = int(g.get("keep", ld.groups))
        ld.router_fn = "sigmoid"; ld.group_score = "top2"; ld.router_norm = True
        ld.shared_ff = int(f["shared"]["ff"]) if f.get("shared") else 0
    else:
        raise ValueError(f"layer {i}: feed-forward kind {f.get('kind')!r} is not implemented")
    return ld


def _attention_fields(ld: LayerDesc, m: dict, mask: str):
    """the attention entries of a Vitudra mixer (an "attention" layer's, or the "left" half of a "parallel" one); what is absent is off"""
    ld.heads = int(m["heads"]); ld.kv_heads = int(m.get("kv_heads", m["heads"])); ld.dim = int(m["dim"]); ld.vdim = int(m.get("vdim", m["dim"]))
    ld.scale = float(m["scale"]); ld.softcap = float(m.get("softcap") or 0.0)
    if m.get("mask"):
        ld.mask = mask; ld.mask_size = int(m["mask"]["size"])
    rot = m.get("rot")
    if rot:
        ld.rot_dims = int(rot["dims"]); ld.rot_base = float(rot["base"]); ld.rot_pairs = True
        ld.rot_factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    qt = m.get("q_temp")
    if qt:
        ld.q_temp_coef = float(qt["coef"]); ld.q_temp_every = int(qt["every"])


def _vitudra_layer(i: int, l: dict, decay_rank: int = 0) -> LayerDesc:
    """one entry of a Vitudra config's "layers": {"type": "attention" | "wkv" | "parallel", "mixer": {...}, "mlp": null | {"kind": "dense", "ff"}}.
    An attention layer has a sliding window, a distance bias and a query temperature and may read another layer's keys and values ("kv_from");
    a parallel mixer's attention half ("left") has neighbour-pair rotation with linear scaling, a soft cap and a chunked mask."""
    m, f = l["mixer"], l.get("mlp")
    ld = LayerDesc(mixer=l["type"])
    if l["type"] == "attention":
        _attention_fields(ld, m, "window")
        ld.dist_bias = True
        ld.kv_from = int(m["kv_from"]) if m.get("kv_from") is not None else None
    elif l["type"] == "wkv":
        ld.heads = int(m["heads"]); ld.dim = int(m["dim"]); ld.vdim = ld.dim; ld.kv_heads = ld.heads; ld.decay_rank = int(decay_rank)
    else:
        _attention_fields(ld, m["left"], "chunk")
        r = m["right"]
        ld.d_heads = int(r["heads"]); ld.d_kv_heads = int(r.get("kv_heads", r["heads"])); ld.d_dim = int(r["dim"]); ld.d_vdim = int(r.get("vdim", r["dim"]))
        ld.conv_taps = int(r.get("conv", 1)); ld.left_scale = float(m.get("left_scale", 1.0)); ld.right_scale = float(m.get("right_scale", 1.0))
    if f is not None:
        if f.get("kind") != "dense":
            raise ValueError(f"layer {i}: feed-forward kind {f.get('kind')!r} is not implemented")
        ld.mlp = "dense"; ld.ff = int(f["ff"])
    return ld


def _modepel_layer(i: int, l: dict) -> LayerDesc:
    """one entry of a Modepel config's "layers": {"type": "attention" | "mlstm", "mixer": {...}, "mlp": null | {"kind": "dense" | "moe", ...}}"""
    m, f = l["mixer"], l.get("mlp")
    ld = LayerDesc(mixer=l["type"], heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]))
    if l["type"] == "attention":
        rot = m.get("rot") or {}
        ld.kv_heads = int(m["kv_heads"]); ld.scale = float(m["scale"]); ld.v_mix = bool(m.get("v_mix", False))
        ld.rot_dims = int(rot.get("dims", 0)); ld.rot_base = float(rot.get("base", 10000.0))
    else:
        ld.gate_cap = float(m["gate_cap"])
    if f is None:
        return ld
    if f.get("kind") == "dense":
        ld.mlp = "dense"; ld.ff = int(f["ff"])
    elif f.get("kind") == "moe":
        r, g = f["router"], f["router"].get("groups") or {}
        ld.mlp = "moe"; ld.experts = int(r["experts"]); ld.identity = int(r.get("identity", 0)); ld.top = int(r["top"])
        ld.router_scale = float(r.get("scale", 1.0)); ld.groups = int(g.get("count", 1)); ld.groups_keep = int(g.get("keep", ld.groups))
        ld.ff = int(f["expert"]["ff"]) if ld.experts else 0
        ld.shared_ff = int(f["shared"]["ff"]) if f.get("shared") else 0
    else:
        raise ValueError(f"layer {i}: feed-forward kind {f.get('kind')!r} is not implemented")
    return ld


def stack_desc_from_config(cfg: dict, compute_dtype: str = "bf16", max_seqs: int = 4, max_ctx: int = 4096, budget_tokens: int = 0, tensor_shapes=None) -> StackDesc:
    """config.json of a layered model ("architecture": "Zakusun" | "Modepel" | "Vitudra" | "Zaluvik") -> StackDesc.  Every size and constant comes from the file;
    tensor_shapes (checkpoint name -> shape, optional) gives the sizes that only a tensor's shape tells (a wkv layer's decay rank; left open without it:
    the device library then takes it from the tensor at upload)."""
    arch = str(cfg.get("architecture")).lower()
    if arch not in MIXERS_OF:
        raise ValueError(f"Unsupported architecture: {cfg.get('architecture')!r}")
    for i, l in enumerate(cfg["layers"]):
        if l["type"] not in MIXERS_OF[arch]:
            raise ValueError(f"layer {i}: mixer {l['type']!r} is not implemented")
    if arch == "vitudra":
        ts = tensor_shapes or {}
        layers = [_vitudra_layer(i, l, (ts.get(f"l{i}.mix.w1") or (0,))[0]) for i, l in enumerate(cfg["layers"])]
        return StackDesc(family="vitudra", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=layers, compute_dtype=compute_dtype, max_seqs=max_seqs,
                         max_ctx=max_ctx, budget_tokens=budget_tokens, norm_groups=1, norm_eps=float(cfg["norm"]["eps"]), canon_taps=1, logit_scale=1.0,
                         residual_mult=float(cfg.get("residual_mult", 1.0)), name="vitudra")
    if arch == "zaluvik":
        lp = cfg.get("loop") or {}
        return StackDesc(family="zaluvik", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=[_zaluvik_layer(i, l) for i, l in enumerate(cfg["layers"])],
                         compute_dtype=compute_dtype, max_seqs=max_seqs, max_ctx=max_ctx, budget_tokens=budget_tokens, norm_groups=1,
                         norm_eps=float(cfg["norm"]["eps"]), canon_taps=1, logit_scale=1.0, residual_mult=float(cfg.get("residual_mult", 1.0)),
                         embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)), loop_start=int(lp.get("start", 0)), loop_stop=int(lp.get("stop", 0)),
                         loop_times=int(lp.get("times", 1)), name="zaluvik")
    if arch == "modepel":
        return StackDesc(family="modepel", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=[_modepel_layer(i, l) for i, l in enumerate(cfg["layers"])],
                         compute_dtype=compute_dtype, max_seqs=max_seqs, max_ctx=max_ctx, budget_tokens=budget_tokens, norm_groups=1,
                         norm_eps=float(cfg["norm"]["eps"]), canon_taps=1, logit_scale=1.0, name="modepel")
    layers = []
    for i, l in enumerate(cfg["layers"]):
        if l["type"] not in MIXER_BY_NAME:
            raise ValueError(f"layer {i}: mixer {l['type']!r} is not implemented")
        m, f = l["mixer"], l.get("mlp")
        ld = LayerDesc(mixer=l["type"], heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                       scale=float(m["scale"]))
        if f is not None:
            if f.get("kind") not in MLP_BY_NAME:
                raise ValueError(f"layer {i}: feed-forward kind {f.get('kind')!r} is not implemented")
            ld.mlp = f["kind"]; ld.experts = int(f["router"]["experts"]); ld.top = int(f["router"]["top"])
            ld.ff = int(f["expert"]["ff"]); ld.limit = float(f["expert"]["limit"])
        layers.append(ld)
    return StackDesc(width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=layers, compute_dtype=compute_dtype, max_seqs=max_seqs,
                     max_ctx=max_ctx, budget_tokens=budget_tokens, norm_groups=int(cfg["norm"]["groups"]), norm_eps=float(cfg["norm"]["eps"]),
                     canon_taps=int(cfg["canon"]["taps"]), logit_scale=float(cfg["logit_scale"]), name="zakusun")


def is_stack_config(cfg: dict) -> bool:
    return "architecture" in cfg and "model_type" not in cfg
