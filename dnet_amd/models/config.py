"""Model configuration parsed from HF-style config.json dicts.

Covers the reference's model families (llama, qwen2/2.5, qwen3, mixtral,
gpt-oss, deepseek-v2 — reference: src/dnet/core/models/*) with one dataclass.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass
class QuantConfig:
    """Weight quantization: grouped symmetric int8/int4 (W8A16/W4A16), or
    OCP MXFP4 (fmt="mxfp4": e2m1 nibbles + e8m0 32-block scales — applied
    to MoE expert banks only, like gpt-oss checkpoints)."""
    bits: int = 8
    group: int = 128
    fmt: str = ""          # "" = grouped-int, "mxfp4"

    @property
    def name(self) -> str:
        if self.fmt == "mxfp4":
            return "mxfp4"
        return f"int{self.bits}-g{self.group}"


@dataclass
class ModelConfig:
    model_type: str = "llama"
    hidden_size: int = 4096
    num_layers: int = 32
    num_q_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 14336
    vocab_size: int = 128256
    rms_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    tie_word_embeddings: bool = False
    attention_bias: bool = False        # qwen2-style qkv bias
    qk_norm: bool = False               # qwen3-style per-head q/k rmsnorm
    max_position_embeddings: int = 32768
    # MoE (mixtral / qwen-moe / gpt-oss)
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    # sliding-window attention (gpt-oss / mistral): 0 = disabled
    sliding_window: int = 0
    sliding_window_pattern: Optional[list] = None  # per-layer types
    # deepseek-v2 MLA
    q_lora_rank: int = 0
    kv_lora_rank: int = 0
    qk_nope_head_dim: int = 0
    qk_rope_head_dim: int = 0
    v_head_dim: int = 0
    first_k_dense_replace: int = 0
    n_shared_experts: int = 0
    shared_expert_intermediate_size: int = 0   # qwen2-moe gated shared expert
    scoring_func: str = "softmax"              # deepseek-v3: "sigmoid"
    n_group: int = 1                           # deepseek-v3 group-limited
    topk_group: int = 1                        #   routing (noaux_tc)
    routed_scaling_factor: float = 1.0
    norm_topk_prob: bool = False
    quant: Optional[QuantConfig] = None
    # heterogeneous layer stacks (posudra): one dict per layer with its
    # mixer type + sizes and its feed-forward (None = no feed-forward);
    # num_q_heads / head_dim / ... above then hold layer 0's sizes
    layer_specs: Optional[list] = None
    embedding_scale: float = 1.0
    # per-layer token input (gegorax): width of each layer's slice of the
    # second embedding table; 0 = none
    token_side_dim: int = 0
    # layer loops (komizen): layer run i uses the stored weights of layer
    # layer_weight_ids[i] (a looped span repeats its ids; every run has its
    # own cache / state); None = run i uses layer i
    layer_weight_ids: Optional[list] = None
    # hyper-connections (komizen): number of residual streams a layer mixes
    # (0 = one plain residual)
    hc_streams: int = 0
    # hashed pair embedding (lurisun): {"buckets", "mul_prev", "mul_cur"} of
    # the table added to the token embedding; None = no such table
    pair_embedding: Optional[dict] = None
    # taps of the causal convolution over a mixer's input (lurisun); 0 = none
    input_conv_taps: int = 0
    # factor on the output logits
    logit_scale: float = 1.0
    # "bfloat16": bf16 weights/activations with 32-bit accumulation;
    # "float32": weights, activations and matrix products in true fp32
    # (honoured by the model families that implement it)
    compute_dtype: str = "bfloat16"

    @property
    def qkv_out(self) -> int:
        return (self.num_q_heads + 2 * self.num_kv_heads) * self.head_dim

    def stored_layers(self, layer_ids) -> list:
        """Ids of the checkpoint layers whose tensors the given layer runs
        read (sorted, each once)."""
        if self.layer_weight_ids is None:
            return list(layer_ids)
        return sorted({self.layer_weight_ids[l] for l in layer_ids})

    @classmethod
    def from_posudra(cls, cfg: dict,
                     quant: Optional[QuantConfig] = None) -> "ModelConfig":
        """Posudra checkpoints describe themselves layer by layer:
        {"architecture": "Posudra", "vocab", "width", "norm": {"eps"},
        "embedding": {"scale"}, "layers": [{"type", "mixer": {...},
        "mlp": {...} | null}, ...]}. Every size is per layer."""
        specs = [dict(s) for s in cfg["layers"]]
        for i, s in enumerate(specs):
            if s.get("type") != "attention":
                raise ValueError(f"posudra layer {i}: unknown mixer type "
                                 f"{s.get('type')!r}")
            ff = s.get("mlp")
            if ff is not None and ff.get("kind", "dense") != "dense":
                raise ValueError(f"posudra layer {i}: unknown feed-forward "
                                 f"kind {ff.get('kind')!r}")
        m0 = specs[0]["mixer"]
        ffs = [s["mlp"]["ff"] for s in specs if s.get("mlp") is not None]
        return cls(
            model_type="posudra",
            hidden_size=cfg["width"],
            num_layers=len(specs),
            num_q_heads=m0["heads"],
            num_kv_heads=m0["kv_heads"],
            head_dim=m0["dim"],
            v_head_dim=m0["vdim"],
            intermediate_size=max(ffs) if ffs else 0,
            vocab_size=cfg["vocab"],
            rms_eps=cfg["norm"]["eps"],
            embedding_scale=float((cfg.get("embedding") or {}).get("scale",
                                                                   1.0)),
            layer_specs=specs,
            quant=quant,
        )

    @classmethod
    def from_gegorax(cls, cfg: dict,
                     quant: Optional[QuantConfig] = None) -> "ModelConfig":
        """Gegorax checkpoints list their layers: {"architecture":
        "Gegorax", "vocab", "width", "norm": {"eps"}, "token_side":
        {"dim"} (optional), "layers": [{"type": "parallel" |
        "general_delta", "mixer": {...}, "mlp": {"kind": "dense" | "moe",
        ...} | null}, ...]}. Every size and constant is per layer."""
        specs = [dict(s) for s in cfg["layers"]]
        att = None
        for i, s in enumerate(specs):
            kind, m = s.get("type"), s.get("mixer") or {}
            if kind == "parallel":
                need = {"left": ("heads", "kv_heads", "dim", "vdim", "scale"),
                        "right": ("conv", "groups", "heads", "norm_groups",
                                  "state", "vdim")}
                for side, keys in need.items():
                    missing = [k for k in keys if k not in (m.get(side) or {})]
                    if missing:
                        raise ValueError(f"gegorax layer {i}: mixer.{side} "
                                         f"lacks {missing}")
                lf, rt = m["left"], m["right"]
                if lf["heads"] % lf["kv_heads"] or rt["heads"] % rt["groups"] \
                        or (rt["heads"] * rt["vdim"]) % rt["norm_groups"]:
                    raise ValueError(f"gegorax layer {i}: head counts do "
                                     "not divide")
                mask = lf.get("mask") or {}
                if mask.get("pool") and not mask.get("size"):
                    raise ValueError(f"gegorax layer {i}: pooled blocks "
                                     "need a window size")
                att = att or lf
            elif kind == "general_delta":
                if "heads" not in m or "dim" not in m:
                    raise ValueError(f"gegorax layer {i}: mixer lacks "
                                     "heads/dim")
            else:
                raise ValueError(f"gegorax layer {i}: unknown mixer type "
                                 f"{kind!r}")
            ff = s.get("mlp")
            if ff is not None and ff.get("kind") not in ("dense", "moe"):
                raise ValueError(f"gegorax layer {i}: unknown feed-forward "
                                 f"kind {ff.get('kind')!r}")
        att = att or {}
        ffs = [s["mlp"]["ff"] for s in specs
               if s.get("mlp") and s["mlp"].get("kind") == "dense"]
        moe = [s["mlp"] for s in specs
               if s.get("mlp") and s["mlp"].get("kind") == "moe"]
        return cls(
            model_type="gegorax",
            hidden_size=cfg["width"],
            num_layers=len(specs),
            num_q_heads=att.get("heads", 1),
            num_kv_heads=att.get("kv_heads", 1),
            head_dim=att.get("dim", 1),
            v_head_dim=att.get("vdim", 1),
            intermediate_size=max(ffs) if ffs else 0,
            num_experts=max((m["router"]["experts"] for m in moe), default=0),
            num_experts_per_tok=max((m["router"]["top"] for m in moe),
                                    default=0),
            vocab_size=cfg["vocab"],
            rms_eps=cfg["norm"]["eps"],
            token_side_dim=int((cfg.get("token_side") or {}).get("dim", 0)),
            layer_specs=specs,
            quant=quant,
        )

    @classmethod
    def from_komizen(cls, cfg: dict,
                     quant: Optional[QuantConfig] = None) -> "ModelConfig":
        """Komizen checkpoints list their layers: {"architecture":
        "Komizen", "vocab", "width", "norm": {"eps"}, "embedding":
        {"scale"}, "streams" (optional), "loop": {"start", "stop", "times"}
        (optional), "layers": [{"type": "delta" | "mamba2" |
        "latent_attention", "mixer": {...}, "mlp": {"kind": "moe", ...} |
        null}, ...]}. A looped span of layers is unrolled here: the model
        then holds one layer run per pass (``num_layers`` counts runs) and
        ``layer_weight_ids`` names the stored layer each run reads."""
        need = {"delta": ("conv", "dim", "heads", "kv_heads", "vdim"),
                "mamba2": ("conv", "groups", "heads", "norm_groups", "state",
                           "vdim"),
                "latent_attention": ("dim", "heads", "kv_rank", "q_rank",
                                     "rot", "rot_dim", "scale", "vdim")}
        stored = [dict(s) for s in cfg["layers"]]
        for i, s in enumerate(stored):
            kind, m = s.get("type"), s.get("mixer") or {}
            if kind not in need:
                raise ValueError(f"komizen layer {i}: unknown mixer type "
                                 f"{kind!r}")
            missing = [k for k in need[kind] if k not in m]
            if missing:
                raise ValueError(f"komizen layer {i}: mixer lacks {missing}")
            if kind == "delta" and m["heads"] % m["kv_heads"]:
                raise ValueError(f"komizen layer {i}: heads % kv_heads")
            if kind == "mamba2" and (
                    m["heads"] % m["groups"]
                    or (m["heads"] * m["vdim"]) % m["norm_groups"]):
                raise ValueError(f"komizen layer {i}: head counts do not "
                                 "divide")
            if kind == "latent_attention":
                rot = m["rot"]
                if int(rot["dims"]) != int(m["rot_dim"]) \
                        or int(rot["dims"]) % 2:
                    raise ValueError(f"komizen layer {i}: rot.dims must be "
                                     "the (even) rotated size")
            ff = s.get("mlp")
            if ff is not None:
                if ff.get("kind") != "moe":
                    raise ValueError(f"komizen layer {i}: unknown "
                                     f"feed-forward kind {ff.get('kind')!r}")
                if not 0 < ff["router"]["top"] <= ff["router"]["experts"]:
                    raise ValueError(f"komizen layer {i}: router.top")
        ids = list(range(len(stored)))
        loop = cfg.get("loop")
        if loop:
            a, b, k = int(loop["start"]), int(loop["stop"]), \
                int(loop["times"])
            if not (0 <= a <= b <= len(stored)) or k < 1:
                raise ValueError("komizen: loop span out of range")
            ids = ids[:a] + ids[a:b] * k + ids[b:]
        specs = [stored[i] for i in ids]
        att = next((s["mixer"] for s in specs
                    if s["type"] == "latent_attention"), {})
        moe = [s["mlp"] for s in specs if s.get("mlp")]
        return cls(
            model_type="komizen",
            hidden_size=cfg["width"],
            num_layers=len(specs),
            num_q_heads=att.get("heads", 1),
            num_kv_heads=1,
            head_dim=att.get("dim", 1),
            v_head_dim=att.get("vdim", 1),
            intermediate_size=0,
            num_experts=max((m["router"]["experts"] for m in moe), default=0),
            num_experts_per_tok=max((m["router"]["top"] for m in moe),
                                    default=0),
            moe_intermediate_size=max((m["expert"]["ff"] for m in moe),
                                      default=0),
            vocab_size=cfg["vocab"],
            rms_eps=cfg["norm"]["eps"],
            embedding_scale=float((cfg.get("embedding") or {}).get("scale",
                                                                   1.0)),
            tie_word_embeddings=True,
            layer_specs=specs,
            layer_weight_ids=ids,
            hc_streams=int(cfg.get("streams") or 0),
            quant=quant,
        )

    @classmethod
    def from_lurisun(cls, cfg: dict,
                     quant: Optional[QuantConfig] = None) -> "ModelConfig":
        """Lurisun checkpoints list their layers: {"architecture":
        "Lurisun", "vocab", "width", "norm": {"eps"}, "canon": {"taps"}
        (optional), "embedding": {"bigram": {"buckets", "mul_prev",
        "mul_cur"}} (optional), "logit_scale" (optional), "layers":
        [{"type": "lightning" | "attention" | "latent_attention", "mixer":
        {...}, "mlp": {"kind": "dense", "ff"} | null}, ...]}. Every size is
        per layer."""
        need = {"lightning": ("decay", "dim", "heads", "vdim"),
                "attention": ("dim", "heads", "kv_heads", "mask", "scale",
                              "vdim"),
                "latent_attention": ("dim", "heads", "kv_rank", "mask",
                                     "q_rank", "scale", "vdim")}
        specs = [dict(s) for s in cfg["layers"]]
        for i, s in enumerate(specs):
            kind, m = s.get("type"), s.get("mixer") or {}
            if kind not in need:
                raise ValueError(f"lurisun layer {i}: unknown mixer type "
                                 f"{kind!r}")
            missing = [k for k in need[kind] if k not in m]
            if missing:
                raise ValueError(f"lurisun layer {i}: mixer lacks {missing}")
            if kind == "lightning" and len(m["decay"]) != m["heads"]:
                raise ValueError(f"lurisun layer {i}: one decay per head")
            if kind == "attention":
                if m["heads"] % m["kv_heads"]:
                    raise ValueError(f"lurisun layer {i}: heads % kv_heads")
                if m["vdim"] != m["dim"]:
                    raise ValueError(f"lurisun layer {i}: the values are "
                                     "the key projections (vdim == dim)")
                rot = m.get("rot")
                if rot and (int(rot["dims"]) % 2
                            or int(rot["dims"]) > m["dim"]):
                    raise ValueError(f"lurisun layer {i}: rot.dims must be "
                                     "even and at most dim")
            if kind != "lightning" and int(m["mask"]["size"]) < 1:
                raise ValueError(f"lurisun layer {i}: mask.size")
            ff = s.get("mlp")
            if ff is not None and ff.get("kind", "dense") != "dense":
                raise ValueError(f"lurisun layer {i}: unknown feed-forward "
                                 f"kind {ff.get('kind')!r}")
        att = next((s["mixer"] for s in specs if s["type"] == "attention"),
                   specs[0]["mixer"])
        ffs = [s["mlp"]["ff"] for s in specs if s.get("mlp") is not None]
        pair = (cfg.get("embedding") or {}).get("bigram")
        return cls(
            model_type="lurisun",
            hidden_size=cfg["width"],
            num_layers=len(specs),
            num_q_heads=att["heads"],
            num_kv_heads=att.get("kv_heads", 1),
            head_dim=att["dim"],
            v_head_dim=att["vdim"],
            intermediate_size=max(ffs) if ffs else 0,
            vocab_size=cfg["vocab"],
            rms_eps=cfg["norm"]["eps"],
            layer_specs=specs,
            pair_embedding=dict(pair) if pair else None,
            input_conv_taps=int((cfg.get("canon") or {}).get("taps") or 0),
            logit_scale=float(cfg.get("logit_scale", 1.0)),
            quant=quant,
        )

    @classmethod
    def from_hf(cls, cfg: dict, quant: Optional[QuantConfig] = None) -> "ModelConfig":
        arch = str(cfg.get("architecture", "")).lower()
        if arch == "lurisun" or cfg.get("model_type") == "lurisun":
            return cls.from_lurisun(cfg, quant)
        if arch == "posudra" or cfg.get("model_type") == "posudra":
            return cls.from_posudra(cfg, quant)
        if arch == "gegorax" or cfg.get("model_type") == "gegorax":
            return cls.from_gegorax(cfg, quant)
        if arch == "komizen" or cfg.get("model_type") == "komizen":
            return cls.from_komizen(cfg, quant)
        mt = cfg.get("model_type", "llama")
        hidden = cfg["hidden_size"]
        nq = cfg.get("num_attention_heads", 32)
        hd = cfg.get("head_dim") or hidden // nq
        mc = cls(
            model_type=mt,
            hidden_size=hidden,
            num_layers=cfg.get("num_hidden_layers", 32),
            num_q_heads=nq,
            num_kv_heads=cfg.get("num_key_value_heads", nq),
            head_dim=hd,
            intermediate_size=cfg.get("intermediate_size", 4 * hidden),
            vocab_size=cfg.get("vocab_size", 32000),
            rms_eps=cfg.get("rms_norm_eps", 1e-5),
            rope_theta=(cfg.get("rope_theta")
                        or (cfg.get("rope_parameters") or {}).get("rope_theta")
                        or 10000.0),
            rope_scaling=cfg.get("rope_scaling") or cfg.get("rope_parameters"),
            tie_word_embeddings=cfg.get("tie_word_embeddings", False),
            attention_bias=cfg.get("attention_bias", mt == "qwen2"),
            qk_norm=mt in ("qwen3", "qwen3_moe"),
            max_position_embeddings=cfg.get("max_position_embeddings", 32768),
            sliding_window=(cfg.get("sliding_window") or 0
                            if cfg.get("use_sliding_window", True) else 0),
            quant=quant,
        )
        mc.sliding_window_pattern = cfg.get("layer_types")
        if mt in ("deepseek_v2", "deepseek_v3"):
            mc.q_lora_rank = cfg.get("q_lora_rank") or 0
            mc.kv_lora_rank = cfg.get("kv_lora_rank", 512)
            mc.qk_nope_head_dim = cfg.get("qk_nope_head_dim", 128)
            mc.qk_rope_head_dim = cfg.get("qk_rope_head_dim", 64)
            mc.v_head_dim = cfg.get("v_head_dim", 128)
            mc.first_k_dense_replace = cfg.get("first_k_dense_replace", 0)
            mc.n_shared_experts = cfg.get("n_shared_experts") or 0
            mc.routed_scaling_factor = cfg.get("routed_scaling_factor", 1.0)
            mc.norm_topk_prob = cfg.get("norm_topk_prob", False)
            mc.num_experts = cfg.get("n_routed_experts") or 0
            mc.num_experts_per_tok = cfg.get("num_experts_per_tok", 0)
            mc.moe_intermediate_size = cfg.get("moe_intermediate_size", 0)
            mc.scoring_func = cfg.get("scoring_func", "softmax")
            mc.n_group = cfg.get("n_group") or 1
            mc.topk_group = cfg.get("topk_group") or 1
        if mt in ("mixtral", "qwen2_moe", "qwen3_moe", "gpt_oss"):
            mc.num_experts = cfg.get("num_local_experts",
                                     cfg.get("num_experts", 8))
            mc.num_experts_per_tok = cfg.get("num_experts_per_tok", 2)
            mc.moe_intermediate_size = cfg.get("moe_intermediate_size",
                                               cfg.get("intermediate_size"))
            mc.norm_topk_prob = cfg.get("norm_topk_prob", False)
            mc.shared_expert_intermediate_size = cfg.get(
                "shared_expert_intermediate_size", 0)
        return mc


def posudra_config(width: int, layers: int, heads: int, kv_heads: int,
                   dim: int, vdim: int, ff: int, vocab: int,
                   softcap: float = 50.0, eps: float = 1e-5,
                   embedding_scale: float = 1.0) -> dict:
    """A uniform posudra stack in the checkpoint's config.json layout."""
    layer = {"type": "attention",
             "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                       "vdim": vdim, "scale": dim ** -0.5,
                       "softcap": softcap},
             "mlp": {"kind": "dense", "ff": ff} if ff else None}
    return {"architecture": "Posudra", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "embedding": {"scale": embedding_scale},
            "layers": [dict(layer) for _ in range(layers)]}


def gegorax_config(width: int, layers: int, vocab: int, heads: int,
                   kv_heads: int, dim: int, vdim: int, window: int, pool: int,
                   ssm_heads: int, ssm_vdim: int, ssm_state: int,
                   delta_heads: int, delta_dim: int, ff: int,
                   experts: int = 0, top: int = 0, expert_ff: int = 0,
                   shared_ff: int = 0, side_dim: int = 0,
                   pattern: str = "pd", rot_base: float = 10000.0,
                   eps: float = 1e-6) -> dict:
    """A gegorax stack in the checkpoint's config.json layout. ``pattern``
    repeats over the layers: 'p' = attention + state-space side by side,
    'd' = generalized delta rule; every second layer's feed-forward is a
    mixture of experts when ``experts`` > 0, dense otherwise."""
    par = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                    "vdim": vdim, "scale": dim ** -0.5,
                    "mask": {"size": window, "pool": pool},
                    "rot": {"dims": dim, "base": rot_base}},
           "right": {"conv": 4, "groups": max(1, ssm_heads // 8),
                     "heads": ssm_heads, "norm_groups": 1,
                     "state": ssm_state, "vdim": ssm_vdim}}
    dl = {"heads": delta_heads, "dim": delta_dim}
    dense = {"kind": "dense", "ff": ff} if ff else None
    moe = {"kind": "moe", "router": {"experts": experts, "top": top},
           "expert": {"ff": expert_ff, "limit": 7.0}}
    if shared_ff:
        moe["shared"] = {"ff": shared_ff, "limit": 7.0}
    out = []
    for i in range(layers):
        t = pattern[i % len(pattern)]
        out.append({"type": "parallel" if t == "p" else "general_delta",
                    "mixer": par if t == "p" else dl,
                    "mlp": moe if (experts and i % 2 == 1) else dense})
    cfg = {"architecture": "Gegorax", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "layers": out}
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
    return cfg


def komizen_config(width: int, vocab: int, pattern: str = "ldm",
                   layers: int = 0, heads: int = 4, dim: int = 32,
                   rot_dim: int = 16, vdim: int = 32, kv_rank: int = 64,
                   q_rank: int = 48, delta_heads: int = 4,
                   delta_kv_heads: int = 2, delta_dim: int = 16,
                   delta_vdim: int = 32, ssm_heads: int = 4,
                   ssm_vdim: int = 16, ssm_state: int = 16,
                   ssm_groups: int = 1, norm_groups: int = 1, conv: int = 4,
                   experts: int = 4, top: int = 2, expert_ff: int = 64,
                   router_scale: float = 1.0, streams: int = 2,
                   loop: Optional[tuple] = None, rot_base: float = 10000.0,
                   eps: float = 1e-6, embedding_scale: float = 1.0) -> dict:
    """A komizen stack in the checkpoint's config.json layout. ``pattern``
    repeats over the ``layers`` stored layers (default: once): 'l' = latent
    attention, 'd' = gated delta rule, 'm' = mamba2; every layer has a
    mixture-of-experts feed-forward when ``experts`` > 0. ``loop`` =
    (start, stop, times)."""
    mix = {
        "l": ("latent_attention",
              {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
               "kv_rank": kv_rank, "q_rank": q_rank,
               "scale": (dim + rot_dim) ** -0.5,
               "rot": {"base": rot_base, "dims": rot_dim}}),
        "d": ("delta", {"heads": delta_heads, "kv_heads": delta_kv_heads,
                        "dim": delta_dim, "vdim": delta_vdim, "conv": conv}),
        "m": ("mamba2", {"heads": ssm_heads, "vdim": ssm_vdim,
                         "state": ssm_state, "groups": ssm_groups,
                         "norm_groups": norm_groups, "conv": conv}),
    }
    ff = ({"kind": "moe", "expert": {"ff": expert_ff},
           "router": {"experts": experts, "top": top, "scale": router_scale}}
          if experts else None)
    out = []
    for i in range(layers or len(pattern)):
        kind, m = mix[pattern[i % len(pattern)]]
        out.append({"type": kind, "mixer": dict(m), "mlp": ff})
    cfg = {"architecture": "Komizen", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "embedding": {"scale": embedding_scale},
           "layers": out}
    if streams:
        cfg["streams"] = streams
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def lurisun_config(width: int, vocab: int, pattern: str = "nla",
                   layers: int = 0, heads: int = 4, kv_heads: int = 2,
                   dim: int = 32, rot_dims: int = 16, chunk: int = 24,
                   latent_heads: int = 4, latent_dim: int = 16,
                   latent_vdim: int = 24, kv_rank: int = 32, q_rank: int = 48,
                   window: int = 20, lin_heads: int = 4, lin_dim: int = 16,
                   lin_vdim: int = 32, decay: Optional[list] = None,
                   ff: int = 192, taps: int = 4, buckets: int = 509,
                   mul_prev: int = 53, mul_cur: int = 29,
                   logit_scale: float = 1.0, rot_base: float = 10000.0,
                   eps: float = 1e-6) -> dict:
    """A lurisun stack in the checkpoint's config.json layout. ``pattern``
    repeats over ``layers`` layers (default: once): 'n' = constant-decay
    linear attention, 'a' = chunked sigmoid attention, 'l' = windowed latent
    attention; every layer has a dense gated feed-forward when ``ff`` > 0.
    ``taps`` 0: no input convolution; ``buckets`` 0: no pair table."""
    if decay is None:
        decay = [1.0 - 2.0 ** -(2 + 2 * h) for h in range(lin_heads)]
    att = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
           "scale": dim ** -0.5, "mask": {"size": chunk}}
    if rot_dims:
        att["rot"] = {"base": rot_base, "dims": rot_dims}
    mix = {
        "n": ("lightning", {"heads": lin_heads, "dim": lin_dim,
                            "vdim": lin_vdim, "decay": list(decay)}),
        "a": ("attention", att),
        "l": ("latent_attention",
              {"heads": latent_heads, "dim": latent_dim, "vdim": latent_vdim,
               "kv_rank": kv_rank, "q_rank": q_rank,
               "scale": latent_dim ** -0.5, "mask": {"size": window}}),
    }
    out = []
    for i in range(layers or len(pattern)):
        kind, m = mix[pattern[i % len(pattern)]]
        out.append({"type": kind, "mixer": dict(m),
                    "mlp": {"kind": "dense", "ff": ff} if ff else None})
    cfg = {"architecture": "Lurisun", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "logit_scale": logit_scale, "layers": out}
    if taps:
        cfg["canon"] = {"taps": taps}
    if buckets:
        cfg["embedding"] = {"bigram": {"buckets": buckets,
                                       "mul_prev": mul_prev,
                                       "mul_cur": mul_cur}}
    return cfg


# Known configs for synthetic benchmarking (random-init weights; no network).
PRESETS: dict[str, dict] = {
    "llama-3-8b": dict(model_type="llama", hidden_size=4096, num_hidden_layers=32,
                       num_attention_heads=32, num_key_value_heads=8,
                       intermediate_size=14336, vocab_size=128256,
                       rope_theta=500000.0, rms_norm_eps=1e-5),
    "llama-3-70b": dict(model_type="llama", hidden_size=8192, num_hidden_layers=80,
                        num_attention_heads=64, num_key_value_heads=8,
                        intermediate_size=28672, vocab_size=128256,
                        rope_theta=500000.0, rms_norm_eps=1e-5),
    "qwen-2.5-32b": dict(model_type="qwen2", hidden_size=5120, num_hidden_layers=64,
                         num_attention_heads=40, num_key_value_heads=8,
                         intermediate_size=27648, vocab_size=152064,
                         rope_theta=1000000.0, rms_norm_eps=1e-5,
                         attention_bias=True),
    "qwen3-8b": dict(model_type="qwen3", hidden_size=4096, num_hidden_layers=36,
                     num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     intermediate_size=12288, vocab_size=151936,
                     rope_theta=1000000.0, rms_norm_eps=1e-6),
    "mixtral-8x7b": dict(model_type="mixtral", hidden_size=4096,
                         num_hidden_layers=32, num_attention_heads=32,
                         num_key_value_heads=8, intermediate_size=14336,
                         vocab_size=32000, rope_theta=1000000.0,
                         num_local_experts=8, num_experts_per_tok=2),
    "opt-125m-like": dict(model_type="llama", hidden_size=768, num_hidden_layers=12,
                          num_attention_heads=12, num_key_value_heads=12,
                          head_dim=64, intermediate_size=3072, vocab_size=50272,
                          rope_theta=10000.0),
    "gpt-oss-20b": dict(model_type="gpt_oss", hidden_size=2880,
                        num_hidden_layers=24, num_attention_heads=64,
                        num_key_value_heads=8, head_dim=64,
                        intermediate_size=2880, vocab_size=201088,
                        num_local_experts=32, num_experts_per_tok=4,
                        sliding_window=128, rope_theta=150000.0,
                        attention_bias=True, rms_norm_eps=1e-5),
    "deepseek-v2-lite": dict(model_type="deepseek_v2", hidden_size=2048,
                             num_hidden_layers=27, num_attention_heads=16,
                             num_key_value_heads=16, vocab_size=102400,
                             intermediate_size=10944, kv_lora_rank=512,
                             qk_nope_head_dim=128, qk_rope_head_dim=64,
                             v_head_dim=128, n_routed_experts=64,
                             num_experts_per_tok=6, n_shared_experts=2,
                             moe_intermediate_size=1408,
                             first_k_dense_replace=1,
                             routed_scaling_factor=1.0, rope_theta=10000.0),
    "deepseek-v3-lite": dict(model_type="deepseek_v3", hidden_size=2048,
                             num_hidden_layers=27, num_attention_heads=16,
                             num_key_value_heads=16, vocab_size=102400,
                             intermediate_size=10944, q_lora_rank=0,
                             kv_lora_rank=512, qk_nope_head_dim=128,
                             qk_rope_head_dim=64, v_head_dim=128,
                             n_routed_experts=64, num_experts_per_tok=6,
                             n_shared_experts=2, moe_intermediate_size=1408,
                             first_k_dense_replace=1, n_group=8,
                             topk_group=4, scoring_func="sigmoid",
                             norm_topk_prob=True,
                             routed_scaling_factor=2.5, rope_theta=10000.0),
    # posudra at qwen3-8b's layer sizes (equal-size family comparison)
    "posudra-8b-like": posudra_config(4096, 36, 32, 8, 128, 128, 12288,
                                      151936),
    "posudra-tiny": posudra_config(128, 4, 4, 2, 32, 16, 192, 256,
                                   softcap=8.0, embedding_scale=4.0),
    "gegorax-tiny": gegorax_config(128, 4, 256, 4, 2, 32, 16, 24, 4, 4, 16,
                                   16, 2, 32, 192, experts=6, top=2,
                                   expert_ff=64, shared_ff=64, side_dim=16),
    "komizen-tiny": komizen_config(128, 256, "ldm", layers=4, loop=(1, 3, 2),
                                   embedding_scale=4.0),
    "lurisun-tiny": lurisun_config(128, 256, "nla", layers=4,
                                   logit_scale=0.5),
    "tiny": dict(model_type="llama", hidden_size=128, num_hidden_layers=4,
                 num_attention_heads=2, num_key_value_heads=2, head_dim=64,
                 intermediate_size=256, vocab_size=256, rope_theta=10000.0),
}
