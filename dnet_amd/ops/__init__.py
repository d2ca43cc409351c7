"""dnet_amd.ops — gfx950 HIP kernels with CPU reference fallback.

GPU tensors dispatch to the in-tree ``_C.so`` extension (hand-written
CDNA4/HIP kernels); if the extension is missing on a GPU machine the ops
FAIL LOUDLY — there is no silent eager fallback on the GPU path. CPU
tensors use the fp32 reference implementations (tests / no-GPU machines).
"""
from __future__ import annotations

import importlib.util
from pathlib import Path

import torch

from . import reference as ref

_SO = Path(__file__).resolve().parent / "_C.so"
_C = None
_load_error: Exception | None = None


def _try_load():
    global _C, _load_error
    if _C is not None or _load_error is not None:
        return _C
    try:
        spec = importlib.util.spec_from_file_location("dnet_amd.ops._C", _SO)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _C = mod
    except Exception as e:  # pragma: no cover
        _load_error = e
    return _C


def has_native() -> bool:
    return _try_load() is not None


def _native():
    c = _try_load()
    if c is None:
        raise RuntimeError(
            f"dnet_amd native extension not available ({_SO}): {_load_error}. "
            "Run `python -m dnet_amd.ops.build` — GPU tensors never fall back "
            "to eager.")
    return c


def rmsnorm(x: torch.Tensor, residual: torch.Tensor | None, w: torch.Tensor,
            eps: float = 1e-6) -> torch.Tensor:
    if x.is_cuda:
        y = torch.empty_like(x)
        _native().rmsnorm(x, residual, w, y, eps)
        return y
    return ref.rmsnorm(x, residual, w, eps)


# split-K f32 scratch, cached per device (max 64 rows x N<8192 cols)
_scratch: dict = {}


def _get_scratch(device) -> torch.Tensor:
    key = str(device)
    if key not in _scratch:
        # zero-initialized: the split-k path relies on it (the combine
        # kernel re-zeroes after each use instead of a per-launch memset)
        # sized for the largest M=64 pass (lm_head-class N): too small a
        # scratch silently disables split-k (launch_m16 falls back to
        # sk=1) — measured on gateup N=55296: 864 blocks quantize badly
        # onto 256 CUs at 3 blocks/CU
        _scratch[key] = torch.zeros(64 * 152064, dtype=torch.float32,
                                    device=device)
    return _scratch[key]


def scratch_clean(device) -> None:
    """Zero what plain split-k combines left in the scratch (a fill kernel,
    launched only when something is dirty). The decode-graph executor calls
    it before a replay and as the last node of every captured step, so
    eager small-M GEMMs (prefill logits) and graph replays can alternate."""
    if torch.device(device).type == "cuda" and str(device) in _scratch:
        _native().scratch_clean(_scratch[str(device)])


def gemv_bf16(x: torch.Tensor, w: torch.Tensor,
              bias: torch.Tensor | None = None) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty(x.shape[0], w.shape[0], dtype=x.dtype, device=x.device)
        if x.shape[1] % 64 == 0:
            _native().gemm_m16(x, w, None, bias, out, _get_scratch(x.device),
                               0, False, 16)
        else:
            _native().gemv_bf16(x, w, out, bias)
        return out
    return ref.gemv_bf16(x, w, bias)


def gemv_int8(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
              group: int, bias: torch.Tensor | None = None,
              packed: bool = False) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty(x.shape[0], w.shape[0], dtype=x.dtype, device=x.device)
        if packed and x.shape[0] > 2:
            _native().gemm_m16(x, w, scales, bias, out, _get_scratch(x.device),
                               group, True, 8)
        else:
            # M<=2: the scalar GEMV reads 16B/lane and hits 4-5.6 TB/s
            _native().gemv_int8(x, w, scales, out, group, bias, packed)
        return out
    if packed:
        w = ref.unpack_int8_mfma(w)
    return ref.gemv_int8(x, w, scales, group, bias)


def gemv_int4(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
              group: int, bias: torch.Tensor | None = None,
              packed: bool = False) -> torch.Tensor:
    if x.is_cuda:
        assert packed, "GPU int4 path needs the packed layout"
        out = torch.empty(x.shape[0], w.shape[0], dtype=x.dtype, device=x.device)
        _native().gemm_m16(x, w, scales, bias, out, _get_scratch(x.device),
                           group, True, 4)
        return out
    return ref.gemv_int4(x, w, scales, group, bias)


def dequant_int4(w: torch.Tensor, scales: torch.Tensor, group: int,
                 packed: bool = True) -> torch.Tensor:
    if w.is_cuda:
        assert packed
        out = torch.empty(w.shape[0], w.shape[1] * 2, dtype=torch.bfloat16,
                          device=w.device)
        _native().dequant_int4(w, scales, out, group)
        return out
    return ref.dequant_int4(w, scales, group)


def dequant_int8(w: torch.Tensor, scales: torch.Tensor, group: int,
                 packed: bool = False) -> torch.Tensor:
    if w.is_cuda:
        out = torch.empty(w.shape, dtype=torch.bfloat16, device=w.device)
        _native().dequant_int8(w, scales, out, group, packed)
        return out
    if packed:
        w = ref.unpack_int8_mfma(w)
    return ref.dequant_int8(w, scales, group)


def _attn_splits(b: int, hkv: int, smax: int) -> int:
    # fill ~1024 blocks (4/CU); cap so each split owns >= ~512 positions of
    # capacity (short actual sequences leave idle splits + combine overhead)
    import os
    force = os.environ.get("DNET_ATTN_SPLITS")
    if force:
        return max(1, int(force))
    splits = 1
    cap = max(1, smax // 512)
    # target ~2048 blocks (8/CU): measured at 2k ctx batch 32 (qwen-32b,
    # 512 base blocks) splits=4 runs 21.5 ms/step vs 27.2 at splits=2 —
    # serial chunks per block hurt more than combine overhead until the
    # per-split span drops under ~512 positions (the cap)
    while (b * hkv * splits * 2 <= 2048 and splits * 2 <= cap):
        splits *= 2
    return splits


def attn_decode(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                pos: torch.Tensor, scale: float, window: int = 0,
                sinks: torch.Tensor | None = None,
                kscale: torch.Tensor | None = None,
                vscale: torch.Tensor | None = None) -> torch.Tensor:
    if q.is_cuda:
        # q may be a strided slice of the fused QKV buffer; out is contiguous.
        B, Hq, D = q.shape
        dv = vcache.shape[-1]           # MLA: v head dim < qk head dim
        out = torch.empty(B, Hq, dv, dtype=q.dtype, device=q.device)
        splits = _attn_splits(B, kcache.shape[1], kcache.shape[2])
        partials = None
        if splits > 1:
            partials = torch.empty(B * Hq * splits * (dv + 2),
                                   dtype=torch.float32, device=q.device)
        _native().attn_decode(q, kcache, vcache, pos, out, scale, window,
                              sinks, kscale, vscale, partials, splits)
        return out
    return ref.attn_decode(q, kcache, vcache, pos, scale, window, sinks,
                           kscale, vscale)


_PREFILL_DIMS = {(128, 128), (64, 64), (192, 128), (96, 96)}


def attn_prefill_supported(d: int, dv: int) -> bool:
    return (d, dv) in _PREFILL_DIMS


def attn_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                 scale: float, q_off: int, window: int = 0,
                 sinks: torch.Tensor | None = None) -> torch.Tensor:
    """Fused MFMA flash prefill attention (causal + window + sinks).

    q [B,Hq,T,D], k/v [B,Hkv,S,D(v)] -> [B,Hq,T,Dv]. GPU-only; callers
    gate on attn_prefill_supported and fall back to the chunked-einsum
    path otherwise (models/base.py)."""
    B, Hq, T, D = q.shape
    Dv = v.shape[-1]
    out = torch.empty(B, Hq, T, Dv, dtype=q.dtype, device=q.device)
    _native().attn_prefill(q.contiguous(), k.contiguous(), v.contiguous(),
                           sinks, out, q_off, window, scale)
    return out


def rope_append(q, k, v, kcache, vcache, pos, cos, sin,
                kscale=None, vscale=None, wpos=None) -> None:
    if q.is_cuda:
        _native().rope_append(q, k, v, kcache, vcache, pos, cos, sin,
                              kscale, vscale, wpos)
        return
    ref.rope_append(q, k, v, kcache, vcache, pos, cos, sin, kscale, vscale,
                    wpos)


_defer_cache: dict = {}


def _will_defer(M: int, N: int, K: int, group: int, bits: int,
                scratch_elems: int) -> bool:
    key = (M, N, K, group, bits)
    v = _defer_cache.get(key)
    if v is None:
        v = _native().gemm_m16_will_defer(M, N, K, group, bits, scratch_elems)
        _defer_cache[key] = v
    return v


def gemv_qkv_rope(y: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
                  group: int, bits: int, bias, nq: int, nkv: int, d: int,
                  kcache, vcache, pos, cos, sin, kscale=None, vscale=None,
                  wpos=None):
    """Fused qkv GEMM + RoPE + KV append for the decode path: when the
    GEMM runs split-k, RoPE reads (and re-zeroes) the f32 scratch
    directly, applies the qkv bias itself, writes the rotated q to a
    dedicated buffer and k/v straight to the cache — the combine kernel
    and the bf16 k/v round trip disappear from the dependency chain.
    Returns the rotated q [B, nq, d]."""
    B = y.shape[0]
    scratch = _get_scratch(y.device)
    if _will_defer(B, w.shape[0], y.shape[1], group, bits, scratch.numel()):
        out = torch.empty(B, w.shape[0], dtype=y.dtype, device=y.device)
        deferred = _native().gemm_m16(y, w, scales, None, out, scratch,
                                      group, True, bits, True)
        assert deferred, "will_defer disagreed with gemm_m16"
        q = torch.empty(B, nq, d, dtype=y.dtype, device=y.device)
        _native().rope_append_f32(scratch, bias, q, nkv, kcache, vcache,
                                  pos, cos, sin, kscale, vscale, wpos)
        return q
    gemv = gemv_int8 if bits == 8 else gemv_int4
    qkv = gemv(y, w, scales, group, bias, True)
    q = qkv[:, :nq * d].view(B, nq, d)
    k = qkv[:, nq * d:(nq + nkv) * d].view(B, nkv, d)
    v = qkv[:, (nq + nkv) * d:].view(B, nkv, d)
    rope_append(q, k, v, kcache, vcache, pos, cos, sin, kscale, vscale,
                wpos=wpos)
    return q


class _Deferred:
    """Sentinel: the projection's result lives (un-combined, f32) in the
    split-k scratch; the consumer must read+re-zero it."""


DEFERRED = _Deferred()


def gemv_defer(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
               group: int, bits: int) -> bool:
    """Launch the GEMM leaving the f32 split-k result in the scratch
    (caller checked _will_defer). Returns True."""
    out = torch.empty(x.shape[0], w.shape[0], dtype=x.dtype, device=x.device)
    d = _native().gemm_m16(x, w, scales, None, out, _get_scratch(x.device),
                           group, True, bits, True)
    assert d, "will_defer disagreed with gemm_m16"
    return True


def rmsnorm_f32_scratch(residual: torch.Tensor, wn: torch.Tensor,
                        eps: float) -> torch.Tensor:
    """RMSNorm(+residual) whose x input is the deferred f32 scratch."""
    y = torch.empty_like(residual)
    _native().rmsnorm_f32(_get_scratch(residual.device), residual, wn, y,
                          eps)
    return y


def resid_add_scratch(h: torch.Tensor) -> None:
    _native().resid_add_f32(h, _get_scratch(h.device))


def linear_will_defer(x: torch.Tensor, w: torch.Tensor, group: int,
                      bits: int) -> bool:
    return _will_defer(x.shape[0], w.shape[0], x.shape[1], group, bits,
                       _get_scratch(x.device).numel())


def gemv_rmsnorm(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
                 group: int, bits: int, residual: torch.Tensor,
                 wn: torch.Tensor, eps: float) -> torch.Tensor:
    """Fused projection GEMM + RMSNorm(+residual) for the decode path:
    when the GEMM runs split-k, the norm reads (and re-zeroes) the f32
    scratch directly — the combine kernel disappears from the chain.
    Updates `residual` in place (residual += proj) like ops.rmsnorm."""
    scratch = _get_scratch(x.device)
    if _will_defer(x.shape[0], w.shape[0], x.shape[1], group, bits,
                   scratch.numel()):
        out = torch.empty(x.shape[0], w.shape[0], dtype=x.dtype,
                          device=x.device)
        _native().gemm_m16(x, w, scales, None, out, scratch, group, True,
                           bits, True)
        y = torch.empty_like(residual)
        _native().rmsnorm_f32(scratch, residual, wn, y, eps)
        return y
    gemv = gemv_int8 if bits == 8 else gemv_int4
    o = gemv(x, w, scales, group, None, True)
    return rmsnorm(o, residual, wn, eps)


def gemv_swiglu(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
                group: int, bits: int = 8,
                packed: bool = True) -> torch.Tensor:
    """Fused gate/up GEMM + SwiGLU for the decode path: when the GEMM
    runs split-k, SwiGLU reads (and re-zeroes) the f32 scratch directly
    instead of going through the f32->bf16 combine kernel — one fewer
    dependent ~5 us kernel per layer per step."""
    if not (x.is_cuda and packed and 2 < x.shape[0] <= 64):
        gemv = gemv_int8 if bits == 8 else gemv_int4
        return swiglu(gemv(x, w, scales, group, None, packed))
    M, N = x.shape[0], w.shape[0]
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    scratch = _get_scratch(x.device)
    deferred = _native().gemm_m16(x, w, scales, None, out, scratch, group,
                                  True, bits, True)
    y = torch.empty(M, N // 2, dtype=x.dtype, device=x.device)
    if deferred:
        _native().swiglu_f32(scratch, y, N)
    else:
        _native().swiglu(out, y)
    return y


def swiglu(gu: torch.Tensor) -> torch.Tensor:
    if gu.is_cuda:
        i = gu.shape[-1] // 2
        y = torch.empty(*gu.shape[:-1], i, dtype=gu.dtype, device=gu.device)
        if gu.dtype == torch.bfloat16 and i % 8 == 0:
            _native().swiglu(gu, y)
        else:           # fp32 models, widths that are no multiple of 8
            _native().silu_mul_halves(gu.contiguous(), y)
        return y
    return ref.swiglu(gu)


def moe_gateup(x: torch.Tensor, w: torch.Tensor, scales, bias,
               we: torch.Tensor, group: int = 0, packed: bool = False,
               glu: int = 0, alpha: float = 1.702,
               limit: float = 7.0) -> torch.Tensor:
    """Grouped expert gate+up with fused GLU: x [M,K], stacked w [E,2I,K]
    (bf16 or grouped-int8), we [M,E] f32 routing weights -> act [E,M,I].
    Experts with all-zero we are skipped on GPU (their act rows hold
    garbage; moe_down never reads them)."""
    if x.is_cuda:
        e, i2, _ = w.shape
        act = torch.empty(e, x.shape[0], i2 // 2, dtype=torch.bfloat16,
                          device=x.device)
        _native().moe_gateup(x, w, scales, bias, we, act, group, packed,
                             glu, alpha, limit)
        return act
    return ref.moe_gateup(x, w, scales, bias, we, group, packed, glu,
                          alpha, limit)


def moe_down(act: torch.Tensor, w: torch.Tensor, scales, bias,
             we: torch.Tensor, group: int = 0,
             packed: bool = False) -> torch.Tensor:
    """Grouped expert down projection, weighted f32 accumulation:
    act [E,M,I], stacked w [E,H,I], we [M,E] -> out [M,H] f32."""
    if act.is_cuda:
        out = torch.zeros(act.shape[1], w.shape[1], dtype=torch.float32,
                          device=act.device)
        _native().moe_down(act, w, scales, bias, we, out, group, packed)
        return out
    return ref.moe_down(act, w, scales, bias, we, group, packed)


quantize_int8 = ref.quantize_int8
quantize_int4 = ref.quantize_int4
pack_int8_mfma = ref.pack_int8_mfma
pack_int4_mfma = ref.pack_int4_mfma
unpack_int8_mfma = ref.unpack_int8_mfma
rope_tables = ref.rope_tables
rope_apply = ref.rope_apply
mxfp4_dequant = ref.mxfp4_dequant
quantize_mxfp4 = ref.quantize_mxfp4


def dequant_mxfp4(w: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """MXFP4 row-major (nibbles [N, K/2] + e8m0 [N, K/32]) -> bf16."""
    if w.is_cuda and has_native():
        out = torch.empty(w.shape[0], w.shape[1] * 2, dtype=torch.bfloat16,
                          device=w.device)
        _native().dequant_mxfp4(w, scales, out)
        return out
    return ref.dequant_mxfp4(w, scales)


def attn_decode_partials(q, kcache, vcache, pos, scale,
                         kscale=None, vscale=None) -> torch.Tensor:
    """Local flash-decode partials [B, Hq, splits, Dv+2] f32 over THIS
    cache shard — the combinable form for context-parallel attention
    (combine with ``attn_combine`` after gathering shards)."""
    if q.is_cuda:
        B, Hq, _ = q.shape
        dv = vcache.shape[-1]
        splits = _attn_splits(B, kcache.shape[1], kcache.shape[2])
        partials = torch.zeros(B, Hq, splits, dv + 2, dtype=torch.float32,
                               device=q.device)
        partials[..., dv] = -1e30   # empty shards stay neutral in combine
        out = torch.empty(B, Hq, dv, dtype=q.dtype, device=q.device)
        _native().attn_decode(q, kcache, vcache, pos, out, scale, 0, None,
                              kscale, vscale, partials.view(-1), splits,
                              False)
        return partials
    return ref.attn_decode_partials(q, kcache, vcache, pos, scale,
                                    kscale, vscale)


def attn_combine(partials: torch.Tensor,
                 sinks: torch.Tensor | None = None) -> torch.Tensor:
    """partials [B, Hq, S, Dv+2] -> out [B, Hq, Dv]."""
    if partials.is_cuda:
        B, Hq, S, W = partials.shape
        out = torch.empty(B, Hq, W - 2, dtype=torch.bfloat16,
                          device=partials.device)
        _native().attn_combine(partials.contiguous().view(-1), sinks, out, S)
        return out
    return ref.attn_combine(partials, sinks)


# ---- fp32-residual / score-modified attention family (posudra) ----
# Residual stream and every statistic in fp32; activations in the model's
# compute dtype (bf16 or fp32). Kernels: csrc/resid_f32.hip.cpp,
# csrc/attn_mod.hip.cpp.

def rmsnorm_rows(x: torch.Tensor, w: torch.Tensor, eps: float,
                 out_dtype: torch.dtype) -> torch.Tensor:
    if x.is_cuda:
        y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _native().rmsnorm_rows(x.contiguous(), w, y, eps)
        return y
    return ref.rmsnorm_rows(x, w, eps, out_dtype)


def ls_resid_rmsnorm(h: torch.Tensor, a: torch.Tensor, s1: torch.Tensor,
                     b: torch.Tensor | None, s2: torch.Tensor | None,
                     wn: torch.Tensor | None, eps: float,
                     out_dtype: torch.dtype) -> torch.Tensor | None:
    """h (fp32, in place) += s1*a (+ s2*b); returns rms(h)*wn (or None
    when wn is None) — one kernel per layer boundary."""
    if h.is_cuda:
        assert h.dtype == torch.float32 and h.is_contiguous()
        y = (torch.empty(h.shape, dtype=out_dtype, device=h.device)
             if wn is not None else None)
        _native().ls_resid_rmsnorm(h, a, s1, b, s2, wn, y, eps)
        return y
    return ref.ls_resid_rmsnorm(h, a, s1, b, s2, wn, eps, out_dtype)


def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    if z.is_cuda:
        y = torch.empty_like(z)
        _native().xielu(z, pq, y)
        return y
    return ref.xielu(z, pq)


def qknorm_append(qkv: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor,
                  eps: float, nq: int, nkv: int, d: int, dv: int,
                  kcache: torch.Tensor, vcache: torch.Tensor,
                  pos: torch.Tensor, T: int, lens=None, slots=None,
                  per_head: bool = False,
                  rot_freq: torch.Tensor | None = None) -> torch.Tensor:
    """``rot_freq`` fp32 [n] (per-head norm only): interleaved channel pairs
    (2i, 2i+1), i < n, turn by position * rot_freq[i] after the norm."""
    if qkv.is_cuda:
        q = torch.empty(qkv.shape[0], nq * d, dtype=qkv.dtype,
                        device=qkv.device)
        _native().qknorm_append(qkv, qw, kw, q, kcache, vcache, pos, lens,
                                slots, eps, nq, nkv, d, dv, T, per_head,
                                rot_freq)
        return q
    return ref.qknorm_append(qkv, qw, kw, eps, nq, nkv, d, dv, kcache,
                             vcache, pos, T, lens, slots, per_head, rot_freq)


def _attn_mod_splits(blocks: int, smax: int) -> int:
    """Split-KV factor for the decode kernel: aim at >= ~1024 workgroups
    (4 per CU) while every split keeps >= 256 positions of cache capacity.
    A function of static shapes only, so captured graphs stay valid."""
    splits = 1
    while blocks * splits < 1024 and splits * 2 * 256 <= smax:
        splits *= 2
    return splits


def attn_mod(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
             pos: torch.Tensor, T: int, scale: float, lens=None, slots=None,
             temp=None, softcap: float = 0.0, dist_r1=None, dist_r2=None,
             sinks=None, window: int = 0, pool_k=None, pool_v=None,
             pool: int = 0, v_dim: int = 0, chunk: int = 0,
             sig_bias=None) -> torch.Tensor:
    """Causal attention against the cache with per-head temperature, tanh
    soft cap, logarithmic distance penalty and a sink in the softmax
    denominator (each optional). One entry point for decode (T=1) and
    ragged batched prefill (T = padded length, lens = real lengths).
    ``window`` > 0 limits the tokens seen to the last ``window``; with
    ``pool`` > 0 every whole block of ``pool`` positions before the window
    is seen as one entry of the pooled caches (see ``kv_pool_update``).
    ``vcache`` None (latent attention): the values are the first ``v_dim``
    entries of the key rows, which the kernels then stage once for both.
    ``chunk`` > 0: a query sees only the keys of its own block of ``chunk``
    positions (blocks count from position 0). ``sig_bias`` fp32 [Hq]: no
    softmax, the weight of a visible key is sigmoid(score + sig_bias[h])."""
    if sig_bias is not None:
        assert sinks is None and not pool
    if pool:
        assert window and pool_k is not None and pool_v is not None
    if vcache is None:
        assert 0 < v_dim <= kcache.shape[3] and not pool
    if q.is_cuda:
        Hkv, D = kcache.shape[1], kcache.shape[3]
        Dv = vcache.shape[3] if vcache is not None else v_dim
        Hq = q.shape[1] // D
        # padded rows of a ragged batch are never written by the kernel
        out = (torch.zeros if lens is not None else torch.empty)(
            q.shape[0], Hq * Dv, dtype=q.dtype, device=q.device)
        splits, partials = 1, None
        if T == 1:
            # a windowed row scans at most window + pooled entries
            span = kcache.shape[2]
            if window:
                span = min(span, window + 64
                           + (pool_k.shape[2] if pool else 0))
            if chunk:
                span = min(span, chunk + 64)
            G = Hq // Hkv
            if (q.dtype == torch.bfloat16 and G >= 16 and not pool
                    and not chunk and sig_bias is None
                    and D % 8 == 0 and Dv % 8 == 0):
                # grouped heads on the matrix cores (the extension picks the
                # kernel by the same rule): 64 heads per workgroup, splits of
                # at least 128 keys of capacity (measured: more splits cost
                # more in the merge than they gain), partials at every split
                # count
                splits = 1
                blocks = q.shape[0] * Hkv * -(-G // 64)
                while blocks * splits < 1024 and splits * 256 <= span:
                    splits *= 2
                partials = torch.empty(q.shape[0] * Hq * splits * (Dv + 2),
                                       dtype=torch.float32, device=q.device)
            else:
                splits = _attn_mod_splits(q.shape[0] * Hkv * -(-G // 16),
                                          span)
            if splits > 1 and partials is None:
                partials = torch.empty(q.shape[0] * Hq * splits * (Dv + 2),
                                       dtype=torch.float32, device=q.device)
        _native().attn_mod(q, kcache, vcache, pos, lens, slots, out, T,
                           scale, temp, softcap or 0.0, dist_r1, dist_r2,
                           sinks, window or 0, partials, splits,
                           pool_k if pool else None,
                           pool_v if pool else None, pool or 0, Dv,
                           chunk or 0, sig_bias)
        return out
    return ref.attn_mod(q, kcache, vcache, pos, T, scale, lens, slots, temp,
                        softcap, dist_r1, dist_r2, sinks, window, pool_k,
                        pool_v, pool, v_dim, chunk, sig_bias)


# ---- pooled-block caches, short convolutions, linear recurrences ----
# Sequence-state mixers (gegorax): csrc/seq_state.hip.cpp and
# csrc/row_fused.hip.cpp. Recurrent state, decays, step sizes and gates of
# the recurrences are fp32 whatever the activation dtype.

def kv_pool_update(kcache, vcache, pool_k, pool_v, pos, T: int, pool: int,
                   lens=None, slots=None) -> None:
    if kcache.is_cuda:
        _native().kv_pool_update(kcache, vcache, pool_k, pool_v, pos, lens,
                                 slots, T, pool)
        return
    ref.kv_pool_update(kcache, vcache, pool_k, pool_v, pos, T, pool, lens,
                       slots)


def causal_conv_silu(x, col0: int, w, bias, state, pos, T: int, lens=None,
                     slots=None) -> torch.Tensor:
    if x.is_cuda:
        y = torch.empty(x.shape[0], w.shape[0], dtype=torch.float32,
                        device=x.device)
        _native().causal_conv_silu(x, col0, w, bias, state, y, pos, lens,
                                   slots, T)
        return y
    return ref.causal_conv_silu(x, col0, w, bias, state, pos, T, lens, slots)


def ssd_scan(xbc, dt_src, dt_col0: int, dt_bias, a_log, dskip, state, pos,
             T: int, heads: int, P: int, N: int, G: int, lens=None,
             slots=None) -> torch.Tensor:
    if xbc.is_cuda:
        # padded rows of a ragged batch are never written by the kernel
        y = (torch.zeros if lens is not None else torch.empty)(
            xbc.shape[0], heads * P, dtype=torch.float32, device=xbc.device)
        _native().ssd_scan(xbc, dt_src, dt_col0, dt_bias, a_log, dskip,
                           state, y, pos, lens, slots, T, heads, P, N, G)
        return y
    return ref.ssd_scan(xbc, dt_src, dt_col0, dt_bias, a_log, dskip, state,
                        pos, T, heads, P, N, G, lens, slots)


def delta_scan(src, r0: int, k0: int, v0: int, a0: int, wl, w0, ab, state,
               pos, T: int, H: int, d: int, decay_scale: float,
               unit_eps: float, lens=None, slots=None) -> torch.Tensor:
    if src.is_cuda:
        o = (torch.zeros if lens is not None else torch.empty)(
            src.shape[0], H * d, dtype=torch.float32, device=src.device)
        _native().delta_scan(src, r0, k0, v0, a0, wl, w0, ab, state, o, pos,
                             lens, slots, T, H, d, decay_scale, unit_eps)
        return o
    return ref.delta_scan(src, r0, k0, v0, a0, wl, w0, ab, state, pos, T, H,
                          d, decay_scale, unit_eps, lens, slots)


def gated_group_rmsnorm(y, gate_src, gate_col0: int, w, groups: int,
                        eps: float, gate_act: str, gate_first: bool,
                        out_dtype: torch.dtype) -> torch.Tensor:
    if y.is_cuda:
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        _native().gated_group_rmsnorm(y, gate_src, gate_col0, w, out, groups,
                                      eps, gate_act == "silu", gate_first)
        return out
    return ref.gated_group_rmsnorm(y, gate_src, gate_col0, w, groups, eps,
                                   gate_act, gate_first, out_dtype)


_ACT_KINDS = {"relu_sq": 0, "tanh": 1}


def act_slice(x, col0: int, n: int, kind: str) -> torch.Tensor:
    if x.is_cuda:
        y = torch.empty(x.shape[0], n, dtype=x.dtype, device=x.device)
        _native().act_slice(x, col0, y, _ACT_KINDS[kind])
        return y
    return ref.act_slice(x, col0, n, kind)


def gelu_gather_mul(z, table, tokens, col0: int) -> torch.Tensor:
    if z.is_cuda:
        y = torch.empty_like(z)
        _native().gelu_gather_mul(z, table, tokens.reshape(-1), col0, y)
        return y
    return ref.gelu_gather_mul(z, table, tokens, col0)


def resid_branches_rmsnorm(h, a, wa, b, wb, coef: float, f, wn, eps: float,
                           out_dtype: torch.dtype, want_cast: bool = False):
    """h (fp32, in place) += coef * (nrm(a, wa) + nrm(b, wb)) + f with
    nrm(x, w) = x / rms(x) * w (or x when w is None); returns
    (rms(h) * wn | None, h in out_dtype | None) — one kernel per boundary."""
    if h.is_cuda:
        assert h.dtype == torch.float32 and h.is_contiguous()
        y = (torch.empty(h.shape, dtype=out_dtype, device=h.device)
             if wn is not None else None)
        xc = (torch.empty(h.shape, dtype=out_dtype, device=h.device)
              if want_cast else None)
        _native().resid_branches_rmsnorm(h, a, wa, b, wb, coef, f, wn, y, xc,
                                         eps)
        return y, xc
    return ref.resid_branches_rmsnorm(h, a, wa, b, wb, coef, f, wn, eps,
                                      out_dtype, want_cast)


def clamped_glu(gu: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
    if gu.is_cuda:
        y = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype,
                        device=gu.device)
        _native().clamped_glu(gu, y, alpha, limit)
        return y
    return ref.clamped_glu(gu, alpha, limit)


# ---- residual streams, gated delta rule, latent attention (komizen) ----
# csrc/streams.hip.cpp, csrc/seq_state.hip.cpp (gated_delta_scan),
# csrc/latent.hip.cpp, csrc/attn_mod.hip.cpp, csrc/moe.hip.cpp. The
# streams, the recurrent state, unit norms, decays and angles are fp32
# whatever the activation dtype.

def hc_read_norm(xs, w_in, wn, eps: float,
                 out_dtype: torch.dtype) -> torch.Tensor:
    if xs.is_cuda:
        S = w_in.numel()
        y = torch.empty(xs.shape[0], xs.shape[1] // S, dtype=out_dtype,
                        device=xs.device)
        _native().hc_write_read(xs, None, None, None, w_in, wn, y, eps)
        return y
    return ref.hc_read_norm(xs, w_in, wn, eps, out_dtype)


def hc_write(xs, y, mix, w_out, next_in, next_wn, eps: float,
             out_dtype: torch.dtype):
    """Streams xs fp32 [M, S*W] (in place): x_t <- sum_s mix[s,t] x_s +
    w_out[t] y; returns the next sublayer's normalized read when
    ``next_in`` / ``next_wn`` are given — one kernel per sublayer boundary."""
    if xs.is_cuda:
        assert xs.dtype == torch.float32 and xs.is_contiguous()
        S = w_out.numel()
        nxt = (torch.empty(xs.shape[0], xs.shape[1] // S, dtype=out_dtype,
                           device=xs.device) if next_in is not None else None)
        _native().hc_write_read(xs, y, mix, w_out, next_in, next_wn, nxt, eps)
        return nxt
    return ref.hc_write(xs, y, mix, w_out, next_in, next_wn, eps, out_dtype)


def gated_delta_scan(qkv, gates, b_col0: int, a_col0: int, a_log, dt_bias,
                     state, pos, T: int, H: int, KH: int, d: int, dv: int,
                     unit_eps: float, lens=None, slots=None) -> torch.Tensor:
    if qkv.is_cuda:
        o = (torch.zeros if lens is not None else torch.empty)(
            qkv.shape[0], H * dv, dtype=torch.float32, device=qkv.device)
        _native().gated_delta_scan(qkv, gates, b_col0, a_col0, a_log, dt_bias,
                                   state, o, pos, lens, slots, T, H, KH, d,
                                   dv, unit_eps)
        return o
    return ref.gated_delta_scan(qkv, gates, b_col0, a_col0, a_log, dt_bias,
                                state, pos, T, H, KH, d, dv, unit_eps, lens,
                                slots)


def latent_append(src, col0: int, wn, eps: float, R: int, rot_freq, kcache,
                  pos, T: int, lens=None, slots=None) -> None:
    if src.is_cuda:
        _native().latent_append(src, col0, wn, eps, R, rot_freq, kcache, pos,
                                lens, slots, T)
        return
    ref.latent_append(src, col0, wn, eps, R, rot_freq, kcache, pos, T, lens,
                      slots)


def latent_q_pack(q, qabs, rot_freq, pos, T: int, H: int,
                  d: int) -> torch.Tensor:
    if q.is_cuda:
        rd = 2 * rot_freq.numel()
        out = torch.empty(q.shape[0], H * (qabs.shape[2] + rd),
                          dtype=q.dtype, device=q.device)
        _native().latent_q_pack(q, qabs, rot_freq, pos, out, T, H, d)
        return out
    return ref.latent_q_pack(q, qabs, rot_freq, pos, T, H, d)


def moe_up_act(x, w, we) -> torch.Tensor:
    """Ungated experts, first half: act [E, M, I] = relu(x w_e^T)^2 (bf16;
    experts with all-zero ``we`` are skipped on the GPU)."""
    if x.is_cuda:
        act = torch.empty(w.shape[0], x.shape[0], w.shape[1],
                          dtype=torch.bfloat16, device=x.device)
        _native().moe_up_act(x, w, we, act)
        return act
    return ref.moe_up_act(x, w, we)


def moe_route(logits, top: int, scale: float) -> torch.Tensor:
    """Routing weights [T, E]: softmax over all experts, the ``top`` largest
    kept times ``scale``, not renormalized (one kernel; no host sync)."""
    if logits.is_cuda:
        we = torch.empty_like(logits)
        _native().moe_route(logits.contiguous(), we, top, scale)
        return we
    return ref.moe_route(logits, top, scale)


def moe_weighted_sum(d, we) -> torch.Tensor:
    if d.is_cuda and d.shape[2] % 4 == 0:
        out = torch.empty(d.shape[1], d.shape[2], dtype=torch.float32,
                          device=d.device)
        _native().moe_weighted_sum(d.contiguous(), we, out)
        return out
    return ref.moe_weighted_sum(d, we)


# ---- hashed pair embedding, residual convolution, constant-decay linear
# attention, sigmoid-weighted chunked attention (lurisun) ----
# csrc/token_mix.hip.cpp, csrc/attn_mod.hip.cpp. Embedding sums, the
# convolution over the fp32 residual, the recurrent state, norms and angles
# are fp32 whatever the activation dtype.

def pair_hash_embed(tokens, embed, table, prev, pos, buckets: int,
                    mul_prev: int, mul_cur: int, lens=None,
                    slots=None) -> torch.Tensor:
    """embed[token] + table[hash(previous, token)] as fp32 [B, T, W]; the
    slot's last token (``prev`` int32 [Bc]) is read for the first token of a
    portion and advanced. See ``reference.pair_hash_embed``."""
    if tokens.is_cuda:
        B, T = tokens.shape
        out = torch.empty(B, T, embed.shape[1], dtype=torch.float32,
                          device=tokens.device)
        _native().pair_hash_embed(tokens.contiguous(), embed, table, prev,
                                  out, pos, lens, slots, buckets, mul_prev,
                                  mul_cur)
        return out
    return ref.pair_hash_embed(tokens, embed, table, prev, pos, buckets,
                               mul_prev, mul_cur, lens, slots)


def causal_conv_residual(x, w, state, pos, T: int, out_dtype: torch.dtype,
                         lens=None, slots=None) -> torch.Tensor:
    """x + conv(x) over the fp32 rows x [B*T, C] (no bias, no activation);
    ``state`` fp32 [Bc, taps-1, C] is each slot's input tail."""
    if x.is_cuda:
        y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _native().causal_conv_residual(x, w, state, y, pos, lens, slots, T)
        return y
    return ref.causal_conv_residual(x, w, state, pos, T, out_dtype, lens,
                                    slots)


def decay_scan(src, q0: int, k0: int, v0: int, decay, state, pos, T: int,
               H: int, d: int, dv: int, lens=None, slots=None) -> torch.Tensor:
    """Constant-decay linear attention over SiLU(q), SiLU(k), SiLU(v) taken
    from columns of ``src``: S <- decay[h] S + k v^T, o = S^T q (fp32)."""
    if src.is_cuda:
        # padded rows of a ragged batch are never written by the kernel
        o = (torch.zeros if lens is not None else torch.empty)(
            src.shape[0], H * dv, dtype=torch.float32, device=src.device)
        _native().decay_scan(src, q0, k0, v0, decay, state, o, pos, lens,
                             slots, T, H, d, dv)
        return o
    return ref.decay_scan(src, q0, k0, v0, decay, state, pos, T, H, d, dv,
                          lens, slots)


def qknorm_half_append(qk, qw, kw, eps: float, nq: int, nkv: int, d: int,
                       rot_freq, kcache, vcache, pos, T: int, lens=None,
                       slots=None) -> torch.Tensor:
    """Whole-projection RMS norm of q and k, half-split rotation (channel i
    with i + n), keys appended to ``kcache`` and the raw key projections as
    values to ``vcache``; returns the queries."""
    if qk.is_cuda:
        q = torch.empty(qk.shape[0], nq * d, dtype=qk.dtype, device=qk.device)
        _native().qknorm_half_append(qk, qw, kw, q, kcache, vcache, pos, lens,
                                     slots, eps, nq, nkv, d, T, rot_freq)
        return q
    return ref.qknorm_half_append(qk, qw, kw, eps, nq, nkv, d, rot_freq,
                                  kcache, vcache, pos, T, lens, slots)


def mul_sigmoid(a, gate_src, col0: int) -> torch.Tensor:
    """a [M, N] * sigmoid(gate_src[:, col0:col0+N])."""
    if a.is_cuda:
        y = torch.empty_like(a)
        _native().mul_sigmoid(a.contiguous(), gate_src, col0, y)
        return y
    return ref.mul_sigmoid(a, gate_src, col0)
