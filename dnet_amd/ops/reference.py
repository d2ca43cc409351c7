"""Plain-PyTorch fp32 reference implementations of every dnet_amd HIP kernel.

These serve two purposes:
  * golden references for the GPU numerics tests (kernel vs fp32 eager), and
  * the CPU execution path, so the whole engine (ring executor, policies,
    API server) runs and is testable on machines with no GPU.

They intentionally mirror the kernel contracts exactly (shapes, in-place
semantics, bf16 rounding points).
"""
from __future__ import annotations

import torch


def rmsnorm(x: torch.Tensor, residual: torch.Tensor | None, w: torch.Tensor,
            eps: float) -> torch.Tensor:
    """y = rms_norm(x or x+residual) * w; residual (if given) updated in place."""
    if residual is not None:
        h = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(h)
        src = h.float()
    else:
        src = x.float()
    scale = torch.rsqrt(src.pow(2).mean(-1, keepdim=True) + eps)
    return (src * scale * w.float()).to(x.dtype)


def gemv_bf16(x: torch.Tensor, w: torch.Tensor,
              bias: torch.Tensor | None = None) -> torch.Tensor:
    y = x.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


def dequant_int8(w: torch.Tensor, scales: torch.Tensor, group: int) -> torch.Tensor:
    n, k = w.shape
    wf = w.float().view(n, k // group, group)
    return (wf * scales.float().unsqueeze(-1)).view(n, k).to(torch.bfloat16)


def gemv_int8(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor,
              group: int, bias: torch.Tensor | None = None) -> torch.Tensor:
    wd = dequant_int8(w, scales, group)
    y = x.float() @ wd.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


def pack_int8_mfma(q: torch.Tensor) -> torch.Tensor:
    """Permute each row's K dim into MFMA chunk-pair order so a lane's
    16 B load covers its 8-elem B-fragment slices of two adjacent K=32
    chunks (full 64 B HBM bursts per 16-row group instead of 32 B halves).

    orig [N, cp, half, slice, j] -> packed [N, cp, slice, half, j]
    (cp = 64-k pair, half = which chunk, slice = lane>>4, j = 0..7).
    """
    n, k = q.shape
    assert k % 64 == 0
    v = q.view(n, k // 64, 2, 4, 8)
    return v.permute(0, 1, 3, 2, 4).reshape(n, k).contiguous()


def unpack_int8_mfma(qp: torch.Tensor) -> torch.Tensor:
    n, k = qp.shape
    v = qp.view(n, k // 64, 4, 2, 8)
    return v.permute(0, 1, 3, 2, 4).reshape(n, k).contiguous()


def quantize_int8(w: torch.Tensor, group: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-group int8 quantization along the K (last) dim."""
    n, k = w.shape
    assert k % group == 0
    wf = w.float().view(n, k // group, group)
    amax = wf.abs().amax(dim=-1).clamp_min(1e-8)
    scales = (amax / 127.0).to(torch.bfloat16)
    q = torch.round(wf / scales.float().unsqueeze(-1)).clamp(-127, 127).to(torch.int8)
    return q.view(n, k), scales


def quantize_kv_rows(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """int8 group-64 KV quantization over the last dim (matches the
    rope_append kernel: bf16-rounded scale = amax/127)."""
    *lead, d = x.shape
    ng = d // 64
    xf = x.float().view(*lead, ng, 64)
    amax = xf.abs().amax(dim=-1).clamp_min(1e-8)
    scales = (amax / 127.0).to(torch.bfloat16)
    codes = torch.round(xf / scales.float().unsqueeze(-1)).clamp(-127, 127)
    return codes.to(torch.int8).view(*lead, d), scales.view(*lead, ng)


def dequant_kv(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    *lead, d = codes.shape
    ng = d // 64
    xf = codes.float().view(*lead, ng, 64) * scales.float().unsqueeze(-1)
    return xf.view(*lead, d).to(torch.bfloat16)


def quantize_int4(w: torch.Tensor, group: int = 128
                  ) -> tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-group int4 quantization along K: values in [-7, 7]
    stored offset-by-8 as nibbles, two per byte (even k = low nibble)."""
    n, k = w.shape
    assert k % group == 0 and k % 2 == 0
    wf = w.float().view(n, k // group, group)
    amax = wf.abs().amax(dim=-1).clamp_min(1e-8)
    scales = (amax / 7.0).to(torch.bfloat16)
    q = torch.round(wf / scales.float().unsqueeze(-1)).clamp(-7, 7)
    q = (q + 8).to(torch.uint8).view(n, k)
    packed = (q[:, 0::2] | (q[:, 1::2] << 4)).contiguous()
    return packed, scales


def unpack_int4(q4: torch.Tensor) -> torch.Tensor:
    """[N, K/2] packed nibbles -> [N, K] int8 in [-7, 7] (device-preserving)."""
    n, kb = q4.shape
    lo = (q4 & 0xF).to(torch.int8) - 8
    hi = (q4 >> 4).to(torch.int8) - 8
    out = torch.empty(n, kb * 2, dtype=torch.int8, device=q4.device)
    out[:, 0::2] = lo
    out[:, 1::2] = hi
    return out


def dequant_int4(q4: torch.Tensor, scales: torch.Tensor, group: int
                 ) -> torch.Tensor:
    return dequant_int8(unpack_int4(q4), scales.to(q4.device), group)


def gemv_int4(x: torch.Tensor, q4: torch.Tensor, scales: torch.Tensor,
              group: int, bias: torch.Tensor | None = None) -> torch.Tensor:
    wd = dequant_int4(q4, scales, group)
    y = x.float() @ wd.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


# ---- MXFP4 (OCP microscaling fp4): e2m1 nibbles + one e8m0 (power-of-2
# uint8, bias 127) scale per 32-element block. The gpt-oss checkpoint
# format (reference executes it via MLX nn.quantize,
# src/dnet/core/models/gpt_oss.py:216-287); here it executes natively in
# the grouped MoE kernels at ~4.25 bits/weight resident.

_E2M1 = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def quantize_mxfp4(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """[N, K] -> (packed nibbles [N, K/2] uint8 (even k = low nibble),
    e8m0 scales [N, K/32] uint8). Round-to-nearest onto the e2m1 grid."""
    n, k = w.shape
    assert k % 32 == 0
    wf = w.float().view(n, k // 32, 32)
    amax = wf.abs().amax(dim=-1).clamp_min(1e-30)
    # scale = 2^e with amax/2^e <= 6 (largest e2m1 magnitude)
    e = torch.ceil(torch.log2(amax / 6.0)).clamp(-127, 127)
    scales = (e + 127).to(torch.uint8)
    v = wf / torch.pow(2.0, e).unsqueeze(-1)
    mag = v.abs().unsqueeze(-1)                     # [n, nb, 32, 1]
    idx = (mag - _E2M1.to(w.device).view(1, 1, 1, 8)).abs().argmin(-1)
    code = (idx + torch.where(v < 0, 8, 0)).to(torch.uint8).view(n, k)
    packed = (code[:, 0::2] | (code[:, 1::2] << 4)).contiguous()
    return packed, scales.view(n, k // 32).contiguous()


def dequant_mxfp4(packed: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """(nibbles [N, K/2], e8m0 [N, K/32]) -> bf16 [N, K]."""
    n, kb = packed.shape
    k = kb * 2
    code = torch.empty(n, k, dtype=torch.uint8, device=packed.device)
    code[:, 0::2] = packed & 0xF
    code[:, 1::2] = packed >> 4
    lut = _E2M1.to(packed.device)
    val = lut[(code & 7).long()] * torch.where(code >= 8, -1.0, 1.0)
    sc = torch.pow(2.0, scales.float() - 127.0)
    out = val.view(n, k // 32, 32) * sc.unsqueeze(-1)
    return out.view(n, k).to(torch.bfloat16)


def gemv_mxfp4(x: torch.Tensor, packed: torch.Tensor, scales: torch.Tensor,
               bias: torch.Tensor | None = None) -> torch.Tensor:
    wd = dequant_mxfp4(packed, scales)
    y = x.float() @ wd.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


def pack_int4_mfma(q4: torch.Tensor) -> torch.Tensor:
    """Permute packed-nibble rows into MFMA chunk-quad order: a lane's
    16 B load covers its 8-elem B slices of FOUR adjacent K=32 chunks.

    unpacked orig [N, quad, chunk(4), slice(4), j(8)] ->
    packed nibble bytes [N, quad, slice, chunk, j/2]."""
    n, kb = q4.shape
    k = kb * 2
    assert k % 128 == 0
    vals = unpack_int4(q4) + 8               # [N, K] in [1,15]
    v = vals.view(n, k // 128, 4, 4, 8)      # [N, quad, chunk, slice, j]
    v = v.permute(0, 1, 3, 2, 4).reshape(n, k)  # slice-major
    packed = (v[:, 0::2] | (v[:, 1::2] << 4)).to(torch.uint8)
    return packed.contiguous()


def attn_decode(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                pos: torch.Tensor, scale: float, window: int = 0,
                sinks: torch.Tensor | None = None,
                kscale: torch.Tensor | None = None,
                vscale: torch.Tensor | None = None) -> torch.Tensor:
    """out[b,h] = softmax(q . K^T * scale) @ V over positions
    [max(0, len-window), len) (window=0 -> full)."""
    B, Hq, D = q.shape
    Hkv = kcache.shape[1]
    Dv = vcache.shape[-1]
    G = Hq // Hkv
    out = torch.zeros(B, Hq, Dv, dtype=q.dtype, device=q.device)
    for b in range(B):
        ln = int(pos[b])
        if ln == 0:
            continue
        s0 = max(0, ln - window) if window > 0 else 0
        if kcache.dtype == torch.int8:
            k = dequant_kv(kcache[b, :, s0:ln], kscale[b, :, s0:ln]).float()
            v = dequant_kv(vcache[b, :, s0:ln], vscale[b, :, s0:ln]).float()
        else:
            k = kcache[b, :, s0:ln].float()          # [Hkv, ln-s0, D]
            v = vcache[b, :, s0:ln].float()
        qq = q[b].float().view(Hkv, G, D)      # [Hkv, G, D]
        s = torch.einsum("hgd,hld->hgl", qq, k) * scale
        if sinks is not None:
            sk = sinks.float().view(Hkv, G, 1)
            p = torch.softmax(torch.cat([s, sk], dim=-1), dim=-1)[..., :-1]
        else:
            p = torch.softmax(s, dim=-1)
        o = torch.einsum("hgl,hld->hgd", p, v)
        out[b] = o.reshape(Hq, Dv).to(q.dtype)
    return out


def rope_tables(smax: int, d: int, theta: float,
                device=None, scaling: dict | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Precompute [Smax, D/2] f32 cos/sin tables (neox convention).

    ``scaling`` supports the llama3 rope-scaling dict
    (factor / low_freq_factor / high_freq_factor / original_max_position_embeddings).
    """
    half = d // 2
    inv = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float32) / half))
    attn_factor = 1.0
    if scaling and scaling.get("rope_type", scaling.get("type")) == "yarn":
        # YaRN (gpt-oss / deepseek style): NTK-by-parts interpolation +
        # attention temperature on cos/sin.
        import math
        factor = scaling.get("factor", 1.0)
        orig = scaling.get("original_max_position_embeddings", 4096)
        beta_fast = scaling.get("beta_fast", 32.0)
        beta_slow = scaling.get("beta_slow", 1.0)

        def corr_dim(n_rot):
            return (d * math.log(orig / (n_rot * 2 * math.pi))
                    / (2 * math.log(theta)))

        low = max(math.floor(corr_dim(beta_fast)), 0)
        high = min(math.ceil(corr_dim(beta_slow)), half - 1)
        rng = torch.arange(half, dtype=torch.float32)
        ramp = ((rng - low) / max(high - low, 1e-3)).clamp(0, 1)
        mask = 1 - ramp  # 1 = no interpolation (high freq), 0 = full
        inv = inv / factor * (1 - mask) + inv * mask
        attn_factor = scaling.get("attention_factor") or \
            (0.1 * math.log(factor) + 1.0 if factor > 1 else 1.0)
        mscale = scaling.get("mscale")
        if mscale is not None:
            # deepseek variant: factor from mscale/mscale_all_dim
            def ds_mscale(scale, m):
                return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0
            attn_factor = (ds_mscale(factor, mscale)
                           / ds_mscale(factor, scaling.get("mscale_all_dim", 0)))
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = scaling["factor"]
        lo = scaling.get("low_freq_factor", 1.0)
        hi = scaling.get("high_freq_factor", 4.0)
        orig = scaling.get("original_max_position_embeddings", 8192)
        wavelen = 2 * torch.pi / inv
        low_wl = orig / lo
        high_wl = orig / hi
        smooth = (orig / wavelen - lo) / (hi - lo)
        scaled = torch.where(wavelen > low_wl, inv / factor, inv)
        mid = (1 - smooth) * inv / factor + smooth * inv
        use_mid = (wavelen <= low_wl) & (wavelen >= high_wl)
        inv = torch.where(use_mid, mid, scaled)
    t = torch.arange(smax, dtype=torch.float32)
    freqs = torch.outer(t, inv)
    return (freqs.cos().mul_(attn_factor).to(device),
            freqs.sin().mul_(attn_factor).to(device))


def rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
               positions: torch.Tensor) -> torch.Tensor:
    """Neox rotate-half rope. x: [..., T, H, D] or [B, H, D] with positions [T]/[B]."""
    half = x.shape[-1] // 2
    c = cos[positions].float()  # [P, half]
    s = sin[positions].float()
    # positions index the dim at x.dim()-3 (T for [B,T,H,D], B for [B,H,D])
    shape = [1] * (x.dim() - 3) + [c.shape[0], 1, half]
    c = c.view(shape)
    s = s.view(shape)
    x1 = x[..., :half].float()
    x2 = x[..., half:].float()
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1).to(x.dtype)


def rope_append(q, k, v, kcache, vcache, pos, cos, sin,
                kscale=None, vscale=None, wpos=None):
    """Decode-step fused rope+append reference (in-place on q, k and caches).
    ``wpos`` (context parallelism): local cache write positions; rows with
    wpos outside [0, Smax) are rotated but not stored."""
    B = q.shape[0]
    positions = pos.long()
    q.copy_(rope_apply(q, cos, sin, positions))
    k.copy_(rope_apply(k, cos, sin, positions))
    q8 = kcache.dtype == torch.int8
    smax = kcache.shape[2]
    for b in range(B):
        p = int(pos[b]) if wpos is None else int(wpos[b])
        if p < 0 or p >= smax:
            continue
        if q8:
            kc, ks = quantize_kv_rows(k[b])
            vc, vs = quantize_kv_rows(v[b])
            kcache[b, :, p] = kc
            kscale[b, :, p] = ks
            vcache[b, :, p] = vc
            vscale[b, :, p] = vs
        else:
            kcache[b, :, p] = k[b]
            vcache[b, :, p] = v[b]


def swiglu(gu: torch.Tensor) -> torch.Tensor:
    i = gu.shape[-1] // 2
    g = gu[..., :i].float()
    u = gu[..., i:].float()
    return (torch.nn.functional.silu(g) * u).to(gu.dtype)


def _moe_dense_w(w: torch.Tensor, scales, group: int, packed: bool
                 ) -> torch.Tensor:
    """Stacked expert weights [E, N, K(/2)] (bf16, grouped-int8, or
    mxfp4 nibble rows) -> f32."""
    if w.dtype == torch.uint8:     # mxfp4: [E, N, K/2] + e8m0 [E, N, K/32]
        e, n, kb = w.shape
        return dequant_mxfp4(w.reshape(e * n, kb),
                             scales.reshape(e * n, -1)).float().view(
                                 e, n, kb * 2)
    if w.dtype != torch.int8:
        return w.float()
    e, n, k = w.shape
    q = w.reshape(e * n, k)
    if packed:
        q = unpack_int8_mfma(q)
    return dequant_int8(q, scales.reshape(e * n, -1), group).float().view(
        e, n, k)


def moe_gateup(x: torch.Tensor, w: torch.Tensor, scales, bias,
               we: torch.Tensor, group: int = 0, packed: bool = False,
               glu: int = 0, alpha: float = 1.702, limit: float = 7.0
               ) -> torch.Tensor:
    """x [M,K], w [E,2I,K], we [M,E] -> act [E,M,I] (glu 0=SwiGLU,
    1=gpt-oss clamped GLU). Experts with all-zero we still computed here
    (the kernel skips them; their act rows are never read by moe_down)."""
    wf = _moe_dense_w(w, scales, group, packed)
    gu = torch.einsum("mk,enk->emn", x.float(), wf)
    if bias is not None:
        gu = gu + bias.float().unsqueeze(1)
    i = gu.shape[-1] // 2
    g, u = gu[..., :i], gu[..., i:]
    if glu == 1:
        g = g.clamp(max=limit)
        u = u.clamp(min=-limit, max=limit)
        act = (u + 1.0) * g * torch.sigmoid(g * alpha)
    else:
        act = torch.nn.functional.silu(g) * u
    return act.to(torch.bfloat16)


def moe_down(act: torch.Tensor, w: torch.Tensor, scales, bias,
             we: torch.Tensor, group: int = 0, packed: bool = False
             ) -> torch.Tensor:
    """act [E,M,I], w [E,H,I], we [M,E] -> out [M,H] f32 (weighted sum of
    per-expert down projections; bias applied inside the weighting)."""
    wf = _moe_dense_w(w, scales, group, packed)
    d = torch.einsum("emi,ehi->emh", act.float(), wf)
    if bias is not None:
        d = d + bias.float().unsqueeze(1)
    return (we.t().unsqueeze(-1) * d).sum(dim=0)


_MXFP4_LUT = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
              -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def mxfp4_dequant(blocks: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """OCP MXFP4 -> bf16 (gpt-oss checkpoint format; reference counterpart:
    src/dnet/core/models/gpt_oss.py MXFP4 weight sanitization).

    blocks: uint8 [..., B, 16] — two E2M1 nibbles per byte, low nibble
    first, 32 values per block. scales: uint8 [..., B] — E8M0 power-of-two
    exponents, bias 127. Returns bf16 [..., B*32].
    """
    lut = torch.tensor(_MXFP4_LUT, dtype=torch.float32, device=blocks.device)
    lo = lut[(blocks & 0xF).long()]
    hi = lut[(blocks >> 4).long()]
    vals = torch.stack([lo, hi], dim=-1).reshape(*blocks.shape[:-1],
                                                 blocks.shape[-1] * 2)
    ex = torch.pow(2.0, scales.float() - 127.0)
    out = vals * ex.unsqueeze(-1)
    return out.reshape(*blocks.shape[:-2],
                       blocks.shape[-2] * blocks.shape[-1] * 2).to(
                           torch.bfloat16)


def attn_decode_partials(q, kcache, vcache, pos, scale,
                         kscale=None, vscale=None) -> torch.Tensor:
    """Unnormalized flash-decode partials over this cache shard:
    [B, Hq, 1, Dv+2] f32 with acc (exp(s-m) @ V), m, l — the cross-rank /
    cross-split combinable form (matches the kernel's split-S partials)."""
    B, Hq, D = q.shape
    Hkv = kcache.shape[1]
    Dv = vcache.shape[-1]
    G = Hq // Hkv
    out = torch.zeros(B, Hq, 1, Dv + 2, dtype=torch.float32)
    out[..., Dv] = -1e30
    for b in range(B):
        ln = int(pos[b])
        if ln == 0:
            continue
        if kcache.dtype == torch.int8:
            k = dequant_kv(kcache[b, :, :ln], kscale[b, :, :ln]).float()
            v = dequant_kv(vcache[b, :, :ln], vscale[b, :, :ln]).float()
        else:
            k = kcache[b, :, :ln].float()
            v = vcache[b, :, :ln].float()
        qq = q[b].float().view(Hkv, G, D)
        s = torch.einsum("hgd,hld->hgl", qq, k) * scale
        m = s.amax(dim=-1, keepdim=True)
        p = torch.exp(s - m)
        acc = torch.einsum("hgl,hld->hgd", p, v)
        out[b, :, 0, :Dv] = acc.reshape(Hq, Dv)
        out[b, :, 0, Dv] = m.reshape(Hq)
        out[b, :, 0, Dv + 1] = p.sum(-1).reshape(Hq)
    return out


def attn_combine(partials: torch.Tensor,
                 sinks: torch.Tensor | None = None) -> torch.Tensor:
    """partials [B, Hq, S, Dv+2] -> out [B, Hq, Dv] bf16 (merge shards)."""
    B, Hq, S, W = partials.shape
    Dv = W - 2
    acc, m, l = partials[..., :Dv], partials[..., Dv], partials[..., Dv + 1]
    M = m.amax(dim=-1)
    if sinks is not None:
        M = torch.maximum(M, sinks.float().view(1, Hq))
    w = torch.exp(m - M.unsqueeze(-1))
    denom = (l * w).sum(-1)
    if sinks is not None:
        denom = denom + torch.exp(sinks.float().view(1, Hq) - M)
    num = (acc * w.unsqueeze(-1)).sum(2)
    denom = denom.clamp_min(1e-30)
    return (num / denom.unsqueeze(-1)).to(torch.bfloat16)


# ---- fp32-residual / score-modified attention family (posudra) ----

def rmsnorm_rows(x: torch.Tensor, w: torch.Tensor, eps: float,
                 out_dtype: torch.dtype) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w, statistics in fp32, any in/out
    dtype (fp32 residual in, bf16 or fp32 activations out)."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * r * w.float()).to(out_dtype)


def ls_resid_rmsnorm(h: torch.Tensor, a: torch.Tensor, s1: torch.Tensor,
                     b: torch.Tensor | None, s2: torch.Tensor | None,
                     wn: torch.Tensor | None, eps: float,
                     out_dtype: torch.dtype) -> torch.Tensor | None:
    """Layer-scaled residual update fused with the next norm:
    h (fp32, in place) += s1*a (+ s2*b); returns rms(h)*wn or None."""
    d = s1.float() * a.float()
    if b is not None:
        d = d + s2.float() * b.float()
    h.add_(d)
    if wn is None:
        return None
    return rmsnorm_rows(h, wn, eps, out_dtype)


def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """Two-parameter squared/exponential unit:
    z>0: softplus(p) z^2 + z/2;  z<=0: (1/2+softplus(q)) (e^z-1-z) + z/2."""
    zf = z.float()
    ap = torch.nn.functional.softplus(pq[0].float())
    an = 0.5 + torch.nn.functional.softplus(pq[1].float())
    pos = ap * zf * zf + 0.5 * zf
    neg = an * (torch.expm1(zf.clamp(max=0.0)) - zf) + 0.5 * zf
    return torch.where(zf > 0, pos, neg).to(z.dtype)


def _row_index(B: int, T: int, pos, lens, slots, device):
    p = pos.to(torch.int64)
    ln = (lens.to(torch.int64) if lens is not None
          else torch.full((B,), T, dtype=torch.int64, device=device))
    sl = (slots.to(torch.int64) if slots is not None
          else torch.arange(B, device=device))
    return p, ln, sl


def rotate_pairs(x: torch.Tensor, ang: torch.Tensor) -> torch.Tensor:
    """x [M, H, d] fp32, ang [M, n] fp32: pair (x[2i], x[2i+1]) -> (x[2i] cos
    - x[2i+1] sin, x[2i+1] cos + x[2i] sin) for i < n (interleaved layout)."""
    n = ang.shape[1]
    c, s = torch.cos(ang).unsqueeze(1), torch.sin(ang).unsqueeze(1)
    out = x.clone()
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out[..., 0:2 * n:2] = u * c - v * s
    out[..., 1:2 * n:2] = v * c + u * s
    return out


def qknorm_append(qkv: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor,
                  eps: float, nq: int, nkv: int, d: int, dv: int,
                  kcache: torch.Tensor, vcache: torch.Tensor,
                  pos: torch.Tensor, T: int, lens=None, slots=None,
                  per_head: bool = False,
                  rot_freq: torch.Tensor | None = None) -> torch.Tensor:
    """RMS-normalize q and k (over the whole projection, or per head),
    optionally rotate them by position, and append k, v to the cache.
    qkv [B*T, nq*d + nkv*d + nkv*dv]; token (b,t) sits at position pos[b]+t
    of cache row slots[b]; tokens t >= lens[b] are padding (not appended).
    ``rot_freq`` fp32 [n]: after the norm, channel pairs (2i, 2i+1), i < n,
    of every head turn by the angle position * rot_freq[i] (fp32); channels
    from 2n on pass unchanged. Returns the q rows [B*T, nq*d]."""
    M = qkv.shape[0]
    B = M // T
    q = qkv[:, :nq * d]
    k = qkv[:, nq * d:(nq + nkv) * d]
    v = qkv[:, (nq + nkv) * d:]
    if per_head:
        qn = rmsnorm_rows(q.reshape(M, nq, d), qw, eps, qkv.dtype).reshape(M, -1)
        kn = rmsnorm_rows(k.reshape(M, nkv, d), kw, eps, qkv.dtype).reshape(M, -1)
    else:
        qn = rmsnorm_rows(q, qw, eps, qkv.dtype)
        kn = rmsnorm_rows(k, kw, eps, qkv.dtype)
    p, ln, sl = _row_index(B, T, pos, lens, slots, qkv.device)
    if rot_freq is not None:
        # the rotation reads the fp32 normalized values (one rounding, at
        # the end), like the fused kernel
        if per_head:
            qf = rmsnorm_rows(q.reshape(M, nq, d), qw, eps, torch.float32)
            kf = rmsnorm_rows(k.reshape(M, nkv, d), kw, eps, torch.float32)
        else:
            qf = rmsnorm_rows(q, qw, eps, torch.float32).view(M, nq, d)
            kf = rmsnorm_rows(k, kw, eps, torch.float32).view(M, nkv, d)
        tpos = (p.view(B, 1) + torch.arange(T, device=qkv.device)
                ).reshape(M).to(torch.float32)
        ang = tpos.view(M, 1) * rot_freq.float().view(1, -1)
        qn = rotate_pairs(qf, ang).reshape(M, -1).to(qkv.dtype)
        kn = rotate_pairs(kf, ang).reshape(M, -1).to(qkv.dtype)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        kcache[s, :, p0:p0 + n] = kn[b * T:b * T + n].view(n, nkv, d) \
            .transpose(0, 1).to(kcache.dtype)
        vcache[s, :, p0:p0 + n] = v[b * T:b * T + n].reshape(n, nkv, dv) \
            .transpose(0, 1).to(vcache.dtype)
    return qn


def attn_mod(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
             pos: torch.Tensor, T: int, scale: float, lens=None, slots=None,
             temp=None, softcap: float = 0.0, dist_r1=None, dist_r2=None,
             sinks=None, window: int = 0, pool_k=None, pool_v=None,
             pool: int = 0, v_dim: int = 0, chunk: int = 0,
             sig_bias=None) -> torch.Tensor:
    """Causal attention against the cache with score modifiers, all in
    fp32: s = q.k * scale * temp[h]; s = cap*tanh(s/cap);
    s -= r1[h] * ln(1 + r2[h] * (i-j)); softmax whose denominator also
    holds exp(sink[h]). q [B*T, Hq*D] -> out [B*T, Hq*Dv]; query (b,t) is
    at position pos[b]+t and sees keys j <= that (and > that - window).

    With ``pool`` > 0 (needs a window): beside the window's tokens, query
    i also sees entry c of the pooled caches ``pool_k`` / ``pool_v``
    [Bc, Hkv, Sp, D|Dv] for every block c that ends at or before i - window
    (c < (i - window + 1) // pool), in the same softmax; pooled entries take
    no distance penalty.

    ``vcache`` None: the values are the first ``v_dim`` entries of the key
    rows (latent attention: one cached latent is key and value).

    ``chunk`` > 0: query i sees key j only inside its own block of ``chunk``
    positions (j >= (i // chunk) * chunk; blocks count from position 0).
    ``sig_bias`` fp32 [Hq]: no softmax; the weight of a visible key is
    sigmoid(s + sig_bias[h]), not normalized over the keys."""
    Hkv, D = kcache.shape[1], kcache.shape[3]
    if vcache is None:
        vcache = kcache[..., :v_dim]
    Dv = vcache.shape[3]
    M = q.shape[0]
    B = M // T
    Hq = q.shape[1] // D
    G = Hq // Hkv
    out = torch.zeros(M, Hq * Dv, dtype=q.dtype, device=q.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, q.device)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        S = p0 + n
        kk = kcache[s, :, :S].float()                 # [Hkv, S, D]
        vv = vcache[s, :, :S].float()
        qq = q[b * T:b * T + n].float().view(n, Hkv, G, D)
        sc = torch.einsum("thgd,hsd->hgts", qq, kk) * scale
        if temp is not None:
            sc = sc * temp.float().view(Hkv, G, 1, 1)
        if softcap and softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        i = torch.arange(p0, S, device=q.device).view(n, 1)
        j = torch.arange(S, device=q.device).view(1, S)
        dist = (i - j)
        if dist_r1 is not None:
            sc = sc - dist_r1.float().view(Hkv, G, 1, 1) * torch.log1p(
                dist_r2.float().view(Hkv, G, 1, 1)
                * dist.clamp(min=0).float())
        dead = dist < 0
        if window and window > 0:
            dead = dead | (dist >= window)
        if chunk and chunk > 0:
            dead = dead | (j < torch.div(i, chunk, rounding_mode="floor")
                           * chunk)
        if sig_bias is not None:
            assert not pool and sinks is None
            pr = torch.sigmoid(sc + sig_bias.float().view(Hkv, G, 1, 1))
            pr = pr.masked_fill(dead, 0.0)
            o = torch.einsum("hgts,hsd->thgd", pr, vv)
            out[b * T:b * T + n] = o.reshape(n, Hq * Dv).to(q.dtype)
            continue
        sc = sc.masked_fill(dead, float("-inf"))
        nb = 0
        if pool and window and window > 0:
            nb = max(0, (S - 1 - window + 1) // pool)
        if nb:
            pk = pool_k[s, :, :nb].float()
            pv = pool_v[s, :, :nb].float()
            ps = torch.einsum("thgd,hsd->hgts", qq, pk) * scale
            if temp is not None:
                ps = ps * temp.float().view(Hkv, G, 1, 1)
            if softcap and softcap > 0:
                ps = softcap * torch.tanh(ps / softcap)
            cnt = torch.div(i - window + 1, pool, rounding_mode="floor")
            c = torch.arange(nb, device=q.device).view(1, nb)
            ps = ps.masked_fill(c >= cnt, float("-inf"))
            sc = torch.cat([sc, ps], dim=-1)
            vv = torch.cat([vv, pv], dim=1)
        if sinks is not None:
            sk = sinks.float().view(Hkv, G, 1, 1).expand(Hkv, G, n, 1)
            pr = torch.softmax(torch.cat([sc, sk], dim=-1), dim=-1)[..., :-1]
        else:
            pr = torch.softmax(sc, dim=-1)
        o = torch.einsum("hgts,hsd->thgd", pr, vv)
        out[b * T:b * T + n] = o.reshape(n, Hq * Dv).to(q.dtype)
    return out


# ---- pooled-block caches, short convolutions and linear recurrences ----
# (sequence-state mixers: every state lives per cache row / slot, is taken as
# zero at position 0 and is left untouched by padding tokens, so slots can be
# reused without a reset and ragged batches equal each row alone)

def kv_pool_update(kcache: torch.Tensor, vcache: torch.Tensor,
                   pool_k: torch.Tensor, pool_v: torch.Tensor,
                   pos: torch.Tensor, T: int, pool: int, lens=None,
                   slots=None) -> None:
    """Block means of the cache: for every block c of ``pool`` positions that
    this step completes (its last position c*pool+pool-1 lies in
    [pos[b], pos[b]+len)), pool_k[slot, :, c] = mean of the cached keys of the
    block (fp32 sum of the values as stored, one rounding), same for v."""
    B = pos.shape[0]
    p, ln, sl = _row_index(B, T, pos, lens, slots, kcache.device)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        c0 = -(-(p0 - pool + 1) // pool)          # first block ending >= p0
        c0 = max(c0, 0)
        c = c0
        while c * pool + pool - 1 < p0 + n and c < pool_k.shape[2]:
            blk = slice(c * pool, (c + 1) * pool)
            pool_k[s, :, c] = kcache[s, :, blk].float().mean(1).to(pool_k.dtype)
            pool_v[s, :, c] = vcache[s, :, blk].float().mean(1).to(pool_v.dtype)
            c += 1


def causal_conv_silu(x: torch.Tensor, col0: int, w: torch.Tensor,
                     bias: torch.Tensor, state: torch.Tensor,
                     pos: torch.Tensor, T: int, lens=None,
                     slots=None) -> torch.Tensor:
    """Per-channel causal convolution + SiLU over columns [col0, col0+C) of
    x [B*T, ld]. w fp32 [C, taps] (last tap = current token), bias fp32 [C];
    ``state`` [Bc, taps-1, C] holds each slot's last taps-1 inputs (entry j =
    position pos-(taps-1)+j; positions < 0 count as zero) and is advanced.
    Returns fp32 [B*T, C] (padding rows zero)."""
    C, taps = w.shape
    M = x.shape[0]
    B = M // T
    xin = x[:, col0:col0 + C]
    out = torch.zeros(M, C, dtype=torch.float32, device=x.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, x.device)
    wf, bf = w.float(), bias.float()
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        hist = state[s].float().clone()                    # [taps-1, C]
        for j in range(taps - 1):
            if p0 - (taps - 1) + j < 0:
                hist[j] = 0.0
        seq = torch.cat([hist, xin[b * T:b * T + n].float()])
        acc = bf.expand(n, C).clone()
        for j in range(taps):
            acc = acc + seq[j:j + n] * wf[:, j]
        out[b * T:b * T + n] = acc * torch.sigmoid(acc)
        if taps > 1:
            state[s] = seq[n:].to(state.dtype)
    return out


def ssd_scan(xbc: torch.Tensor, dt_src: torch.Tensor, dt_col0: int,
             dt_bias: torch.Tensor, a_log: torch.Tensor, dskip: torch.Tensor,
             state: torch.Tensor, pos: torch.Tensor, T: int, heads: int,
             P: int, N: int, G: int, lens=None, slots=None) -> torch.Tensor:
    """Selective state-space recurrence with one scalar decay per head, all
    fp32. xbc fp32 [B*T, heads*P + 2*G*N] = [x | B | C]; raw step sizes are
    columns [dt_col0, dt_col0+heads) of dt_src. Per head h (group
    g = h // (heads/G)), with dt = softplus(raw + dt_bias[h]):
        S <- exp(-exp(a_log[h]) dt) S + dt B_g x_h^T      (S [N, P])
        y_h = S^T C_g + dskip[h] x_h
    ``state`` fp32 [Bc, heads, N, P] per slot: zero at position 0, advanced
    by the real tokens. Returns y fp32 [B*T, heads*P]."""
    M = xbc.shape[0]
    B = M // T
    inner = heads * P
    y = torch.zeros(M, inner, dtype=torch.float32, device=xbc.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, xbc.device)
    hg = torch.arange(heads, device=xbc.device) // (heads // G)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        S = state[s].float().clone() if p0 > 0 else \
            torch.zeros(heads, N, P, dtype=torch.float32, device=xbc.device)
        rows = slice(b * T, b * T + n)
        xs = xbc[rows, :inner].float().view(n, heads, P)
        Bm = xbc[rows, inner:inner + G * N].float().view(n, G, N)[:, hg]
        Cm = xbc[rows, inner + G * N:].float().view(n, G, N)[:, hg]
        dt = torch.nn.functional.softplus(
            dt_src[rows, dt_col0:dt_col0 + heads].float() + dt_bias.float(),
            threshold=30.0)
        dec = torch.exp(-torch.exp(a_log.float()) * dt)        # [n, heads]
        for t in range(n):
            S = dec[t].view(heads, 1, 1) * S + dt[t].view(heads, 1, 1) * (
                Bm[t].unsqueeze(-1) * xs[t].unsqueeze(1))
            y[b * T + t] = ((S * Cm[t].unsqueeze(-1)).sum(1)
                            + dskip.float().view(heads, 1) * xs[t]).reshape(-1)
        state[s] = S
    return y


def delta_scan(src: torch.Tensor, r0: int, k0: int, v0: int, a0: int,
               wl: torch.Tensor, w0: torch.Tensor, ab: torch.Tensor,
               state: torch.Tensor, pos: torch.Tensor, T: int, H: int,
               d: int, decay_scale: float, unit_eps: float, lens=None,
               slots=None) -> torch.Tensor:
    """Generalized delta rule, all fp32. r, k, v and the removal logits are
    H*d-wide column ranges of src starting at r0, k0, v0, a0; wl [B*T, H*d]
    holds the decay logits. Per head, with w = exp(-decay_scale *
    sigmoid(wl + w0)), a = sigmoid(al + ab), u = k / sqrt(sum(k^2) +
    unit_eps):
        S <- diag(w) S - (a u)(u^T S) + k v^T     (both terms read the old S)
        o = S^T r
    ``state`` fp32 [Bc, H, d, d] per slot (key channel first): zero at
    position 0. Returns o fp32 [B*T, H*d]."""
    M = src.shape[0]
    B = M // T
    n_ = H * d
    out = torch.zeros(M, n_, dtype=torch.float32, device=src.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, src.device)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        S = state[s].float().clone() if p0 > 0 else \
            torch.zeros(H, d, d, dtype=torch.float32, device=src.device)
        rows = slice(b * T, b * T + n)
        col = lambda c0: src[rows, c0:c0 + n_].float().view(n, H, d)
        r, k, v = col(r0), col(k0), col(v0)
        a = torch.sigmoid(col(a0) + ab.float().view(H, d))
        w = torch.exp(-decay_scale * torch.sigmoid(
            wl[rows].float().view(n, H, d) + w0.float().view(H, d)))
        u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)
        for t in range(n):
            uS = torch.einsum("hi,hij->hj", u[t], S)
            S = w[t].unsqueeze(-1) * S \
                - (a[t] * u[t]).unsqueeze(-1) * uS.unsqueeze(1) \
                + k[t].unsqueeze(-1) * v[t].unsqueeze(1)
            out[b * T + t] = torch.einsum("hij,hi->hj", S, r[t]).reshape(-1)
        state[s] = S
    return out


def gated_group_rmsnorm(y: torch.Tensor, gate_src: torch.Tensor,
                        gate_col0: int, w: torch.Tensor, groups: int,
                        eps: float, gate_act: str, gate_first: bool,
                        out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of y [M, N] in ``groups`` equal parts (each by its own root
    mean square), times w [N], with a gate g = act(gate_src[:, gate_col0:
    gate_col0+N]) (act = "silu" | "sigmoid") multiplied in before the norm
    (gate_first) or after the weight. Statistics in fp32."""
    M, N = y.shape
    g = gate_src[:, gate_col0:gate_col0 + N].float()
    g = g * torch.sigmoid(g) if gate_act == "silu" else torch.sigmoid(g)
    v = y.float()
    if gate_first:
        v = v * g
    v = v.view(M, groups, N // groups)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    v = v.reshape(M, N) * w.float()
    if not gate_first:
        v = v * g
    return v.to(out_dtype)


def act_slice(x: torch.Tensor, col0: int, n: int, kind: str) -> torch.Tensor:
    """Unary activation of columns [col0, col0+n) of x [M, ld], fp32 math:
    "relu_sq" = max(z, 0)^2, "tanh"."""
    z = x[:, col0:col0 + n].float()
    if kind == "relu_sq":
        z = torch.relu(z) ** 2
    elif kind == "tanh":
        z = torch.tanh(z)
    else:
        raise ValueError(kind)
    return z.to(x.dtype)


def gelu_gather_mul(z: torch.Tensor, table: torch.Tensor,
                    tokens: torch.Tensor, col0: int) -> torch.Tensor:
    """gelu_tanh(z[m, :]) * table[tokens[m], col0:col0+n] for z [M, n]."""
    import math
    zf = z.float()
    g = 0.5 * zf * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                     * (zf + 0.044715 * zf ** 3)))
    e = table[tokens.reshape(-1).long(), col0:col0 + z.shape[1]].float()
    return (g * e).to(z.dtype)


def resid_branches_rmsnorm(h: torch.Tensor, a: torch.Tensor, wa, b, wb,
                           coef: float, f, wn, eps: float,
                           out_dtype: torch.dtype, want_cast: bool):
    """h (fp32, in place) += coef * (nrm(a, wa) + nrm(b, wb)) + f, where
    nrm(x, w) = x / rms(x) * w when w is given and x itself otherwise (b and
    f optional). Returns (rms(h) * wn or None, h cast to out_dtype or
    None)."""
    def nrm(x, w):
        xf = x.float()
        if w is None:
            return xf
        return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) \
            * w.float()
    d = nrm(a, wa)
    if b is not None:
        d = d + nrm(b, wb)
    d = d * coef
    if f is not None:
        d = d + f.float()
    h.add_(d)
    y = rmsnorm_rows(h, wn, eps, out_dtype) if wn is not None else None
    return y, (h.to(out_dtype) if want_cast else None)


def clamped_glu(gu: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
    """gu [M, 2I] = [gate | up]: g = min(gate, limit), u = clamp(up,
    -limit, limit); y = g * sigmoid(alpha * g) * (u + 1), fp32 math."""
    i = gu.shape[-1] // 2
    g = gu[..., :i].float().clamp(max=limit)
    u = gu[..., i:].float().clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


# ---- residual streams, gated delta rule, latent attention (komizen) ----

def hc_read_norm(xs: torch.Tensor, w_in: torch.Tensor, wn: torch.Tensor,
                 eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """Read of a set of residual streams: xs fp32 [M, S*W] holds S streams
    of width W side by side; u = sum_s w_in[s] * x_s, returned RMS-normalized
    times wn [W] (statistics in fp32)."""
    S = w_in.numel()
    M = xs.shape[0]
    x = xs.view(M, S, -1)
    u = x[:, 0] * w_in[0]
    for s in range(1, S):
        u = u + x[:, s] * w_in[s]
    return rmsnorm_rows(u, wn, eps, out_dtype)


def hc_write(xs: torch.Tensor, y: torch.Tensor, mix: torch.Tensor,
             w_out: torch.Tensor, next_in, next_wn, eps: float,
             out_dtype: torch.dtype):
    """Write of a sublayer's result y [M, W] into the streams, all streams at
    once from the old ones: x_t <- sum_s mix[s, t] x_s + w_out[t] y (xs fp32
    [M, S*W], in place). With ``next_in`` / ``next_wn`` the read of the next
    sublayer (``hc_read_norm``) is returned as well."""
    S = w_out.numel()
    M = xs.shape[0]
    old = xs.view(M, S, -1).clone()
    new = xs.view(M, S, -1)
    yf = y.float()
    for t in range(S):
        acc = old[:, 0] * mix[0, t]
        for s in range(1, S):
            acc = acc + old[:, s] * mix[s, t]
        new[:, t] = acc + w_out[t] * yf
    if next_in is None:
        return None
    return hc_read_norm(xs, next_in, next_wn, eps, out_dtype)


def gated_delta_scan(qkv: torch.Tensor, gates: torch.Tensor, b_col0: int,
                     a_col0: int, a_log: torch.Tensor, dt_bias: torch.Tensor,
                     state: torch.Tensor, pos: torch.Tensor, T: int, H: int,
                     KH: int, d: int, dv: int, unit_eps: float, lens=None,
                     slots=None) -> torch.Tensor:
    """Gated delta rule, all fp32. qkv fp32 [B*T, 2*KH*d + H*dv] = [q | k |
    v] (KH query/key heads shared by H/KH value heads each); columns
    [b_col0, +H) and [a_col0, +H) of ``gates`` hold the raw write-strength
    and decay projections. Per head h (key head h // (H/KH)), with q, k made
    unit vectors (x / sqrt(sum x^2 + unit_eps)), q scaled by d^-1/2,
    beta = sigmoid(b), g = exp(-exp(a_log[h]) softplus(a + dt_bias[h])):
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    ``state`` fp32 [Bc, H, d, dv] per slot: zero at position 0. Returns o
    fp32 [B*T, H*dv]."""
    M = qkv.shape[0]
    B = M // T
    out = torch.zeros(M, H * dv, dtype=torch.float32, device=qkv.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, qkv.device)
    hk = torch.arange(H, device=qkv.device) // (H // KH)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        S = state[s].float().clone() if p0 > 0 else \
            torch.zeros(H, d, dv, dtype=torch.float32, device=qkv.device)
        rows = slice(b * T, b * T + n)
        q = qkv[rows, :KH * d].float().view(n, KH, d)
        k = qkv[rows, KH * d:2 * KH * d].float().view(n, KH, d)
        v = qkv[rows, 2 * KH * d:].float().view(n, H, dv)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)
        q, k = q[:, hk], k[:, hk]                              # [n, H, d]
        beta = torch.sigmoid(gates[rows, b_col0:b_col0 + H].float())
        g = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(
            gates[rows, a_col0:a_col0 + H].float() + dt_bias.float(),
            threshold=30.0))
        for t in range(n):
            S = g[t].view(H, 1, 1) * S
            u = beta[t].view(H, 1) * (
                v[t] - torch.einsum("hij,hi->hj", S, k[t]))
            S = S + k[t].unsqueeze(-1) * u.unsqueeze(1)
            out[b * T + t] = torch.einsum("hij,hi->hj", S, q[t]).reshape(-1)
        state[s] = S
    return out


def latent_append(src: torch.Tensor, col0: int, wn: torch.Tensor, eps: float,
                  R: int, rot_freq: torch.Tensor, kcache: torch.Tensor,
                  pos: torch.Tensor, T: int, lens=None, slots=None) -> None:
    """Append the shared key/value latent of latent attention to the cache.
    Columns [col0, col0+R) of src [B*T, ld] are RMS-normalized times wn [R];
    the rd = 2*len(rot_freq) columns after them turn by position (interleaved
    pairs, angle = position * rot_freq[i], fp32). The cache row [normed
    latent | turned key part] goes to kcache [Bc, 1, Smax, R+rd] at position
    pos[b]+t of row slots[b]; padding tokens are not appended."""
    M = src.shape[0]
    B = M // T
    rd = 2 * rot_freq.numel()
    c = rmsnorm_rows(src[:, col0:col0 + R], wn, eps, torch.float32)
    p, ln, sl = _row_index(B, T, pos, lens, slots, src.device)
    tpos = (p.view(B, 1) + torch.arange(T, device=src.device)
            ).reshape(M).to(torch.float32)
    ang = tpos.view(M, 1) * rot_freq.float().view(1, -1)
    kr = rotate_pairs(src[:, col0 + R:col0 + R + rd].float().view(M, 1, rd),
                      ang).view(M, rd)
    row = torch.cat([c, kr], dim=1).to(kcache.dtype)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        kcache[s, 0, p0:p0 + n] = row[b * T:b * T + n]


def latent_q_pack(q: torch.Tensor, qabs: torch.Tensor,
                  rot_freq: torch.Tensor, pos: torch.Tensor, T: int, H: int,
                  d: int) -> torch.Tensor:
    """Queries of latent attention in the cache's layout. q [B*T, H*(d+rd)]
    holds per head d plain and rd turning dimensions; qabs [H, B*T, R] the
    plain part already carried into the latent space. Returns [B*T,
    H*(R+rd)] = per head [qabs | turned part] (angles as in
    ``latent_append``)."""
    M = q.shape[0]
    B = M // T
    rd = 2 * rot_freq.numel()
    R = qabs.shape[2]
    tpos = (pos.to(torch.int64).view(B, 1)
            + torch.arange(T, device=q.device)).reshape(M).to(torch.float32)
    ang = tpos.view(M, 1) * rot_freq.float().view(1, -1)
    qr = rotate_pairs(q.view(M, H, d + rd)[..., d:].float(), ang)
    out = torch.cat([qabs.transpose(0, 1).float(), qr], dim=-1)
    return out.reshape(M, H * (R + rd)).to(q.dtype)


def moe_up_act(x: torch.Tensor, w: torch.Tensor, we: torch.Tensor
               ) -> torch.Tensor:
    """Ungated experts' first half: x [M, K], stacked w [E, I, K], we [M, E]
    -> act [E, M, I] = relu(x w_e^T)^2 in bf16 (experts nobody chose may
    hold anything; ``moe_down`` never reads them)."""
    z = torch.einsum("mk,eik->emi", x.float(), w.float())
    return (torch.relu(z) ** 2).to(torch.bfloat16)


def moe_route(logits: torch.Tensor, top: int, scale: float) -> torch.Tensor:
    """Routing weights [T, E] fp32: softmax over all experts, the ``top``
    largest probabilities kept and multiplied by ``scale`` (not
    renormalized), 0 for the rest."""
    probs = torch.softmax(logits.float(), dim=-1)
    val, idx = torch.topk(probs, top, dim=-1)
    we = torch.zeros_like(probs)
    we.scatter_(1, idx, val * scale)
    return we


def moe_weighted_sum(d: torch.Tensor, we: torch.Tensor) -> torch.Tensor:
    """d [E, T, W], we [T, E] -> fp32 [T, W] = sum_e we[t, e] d[e, t]."""
    return torch.einsum("te,etw->tw", we.float(), d.float())


# ---- hashed pair embedding, residual convolution, constant-decay linear
# attention, gated outputs (lurisun) ----

def pair_hash_embed(tokens: torch.Tensor, embed: torch.Tensor,
                    table: torch.Tensor, prev: torch.Tensor,
                    pos: torch.Tensor, buckets: int, mul_prev: int,
                    mul_cur: int, lens=None, slots=None) -> torch.Tensor:
    """Token embedding plus a hashed embedding of the (previous, current)
    token pair, fp32 [B, T, W]. tokens [B, T]; token (b,t) sits at position
    pos[b]+t of slot slots[b]. Row of ``table`` [buckets+1, W]:
    (previous * mul_prev + current * mul_cur) mod buckets, and row ``buckets``
    at position 0. ``prev`` int32 [Bc] holds every slot's last token and is
    advanced by the rows' real tokens (t < lens[b])."""
    B, T = tokens.shape
    out = embed[tokens.long()].float()
    p, ln, sl = _row_index(B, T, pos, lens, slots, tokens.device)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        last = int(prev[s])
        for t in range(n):
            cur = int(tokens[b, t])
            row = buckets if p0 + t == 0 else \
                (last * mul_prev + cur * mul_cur) % buckets
            out[b, t] += table[row].float()
            last = cur
        prev[s] = last
    return out


def causal_conv_residual(x: torch.Tensor, w: torch.Tensor,
                         state: torch.Tensor, pos: torch.Tensor, T: int,
                         out_dtype: torch.dtype, lens=None,
                         slots=None) -> torch.Tensor:
    """y = x + conv(x): per-channel causal convolution of the fp32 rows
    x [B*T, C] without bias or activation, added to its input. w fp32
    [C, taps] (last tap = current token); ``state`` fp32 [Bc, taps-1, C]
    holds each slot's last taps-1 inputs (positions < 0 count as zero) and is
    advanced. Returns [B*T, C] in ``out_dtype`` (padding rows zero)."""
    C, taps = w.shape
    M = x.shape[0]
    B = M // T
    out = torch.zeros(M, C, dtype=torch.float32, device=x.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, x.device)
    wf = w.float()
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        hist = state[s].float().clone()
        for j in range(taps - 1):
            if p0 - (taps - 1) + j < 0:
                hist[j] = 0.0
        seq = torch.cat([hist, x[b * T:b * T + n].float()])
        acc = x[b * T:b * T + n].float().clone()
        for j in range(taps):
            acc = acc + seq[j:j + n] * wf[:, j]
        out[b * T:b * T + n] = acc
        if taps > 1:
            state[s] = seq[n:].to(state.dtype)
    return out.to(out_dtype)


def decay_scan(src: torch.Tensor, q0: int, k0: int, v0: int,
               decay: torch.Tensor, state: torch.Tensor, pos: torch.Tensor,
               T: int, H: int, d: int, dv: int, lens=None,
               slots=None) -> torch.Tensor:
    """Linear attention with one constant decay per head, fp32. q, k [H*d]
    and v [H*dv] are columns q0 / k0 / v0 of src [B*T, ld] with SiLU applied
    here; per head S <- decay[h] S + k v^T (S [d, dv]), o = S^T q. ``state``
    fp32 [Bc, H, d, dv] per slot: zero at position 0, advanced by the rows'
    real tokens. Returns fp32 [B*T, H*dv] (padding rows zero)."""
    M = src.shape[0]
    B = M // T
    out = torch.zeros(M, H * dv, dtype=torch.float32, device=src.device)
    p, ln, sl = _row_index(B, T, pos, lens, slots, src.device)
    f = src.float()
    act = torch.nn.functional.silu
    g = decay.float().view(H, 1, 1)
    for b in range(B):
        n = int(min(ln[b], T))
        if n <= 0:
            continue
        p0, s = int(p[b]), int(sl[b])
        rows = f[b * T:b * T + n]
        q = act(rows[:, q0:q0 + H * d]).view(n, H, d)
        k = act(rows[:, k0:k0 + H * d]).view(n, H, d)
        v = act(rows[:, v0:v0 + H * dv]).view(n, H, dv)
        S = state[s].float().clone() if p0 > 0 else \
            torch.zeros(H, d, dv, dtype=torch.float32, device=src.device)
        for t in range(n):
            S = g * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
            out[b * T + t] = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1)
        state[s] = S
    return out


def qknorm_half_append(qk: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor,
                       eps: float, nq: int, nkv: int, d: int,
                       rot_freq: torch.Tensor | None, kcache: torch.Tensor,
                       vcache: torch.Tensor, pos: torch.Tensor, T: int,
                       lens=None, slots=None) -> torch.Tensor:
    """qk [B*T, nq*d + nkv*d] = [q | k]. The cached VALUES are the key
    projections as they come; the cached keys and the returned queries are
    RMS-normalized over the whole projection (weights qw [nq*d], kw [nkv*d])
    and then, per head, channel i < n pairs with channel i + n
    (n = len(rot_freq)) and the pair turns by position * rot_freq[i]; the
    channels from 2n on pass through. Statistics and angles fp32."""
    M = qk.shape[0]
    B = M // T
    q, k = qk[:, :nq * d], qk[:, nq * d:]
    qf = rmsnorm_rows(q, qw, eps, torch.float32).view(M, nq, d)
    kf = rmsnorm_rows(k, kw, eps, torch.float32).view(M, nkv, d)
    p, ln, sl = _row_index(B, T, pos, lens, slots, qk.device)
    n = 0 if rot_freq is None else rot_freq.numel()
    if n:
        tpos = (p.view(B, 1) + torch.arange(T, device=qk.device)
                ).reshape(M).to(torch.float32)
        ang = tpos.view(M, 1) * rot_freq.float().view(1, -1)
        c, s = torch.cos(ang).unsqueeze(1), torch.sin(ang).unsqueeze(1)

        def turn(x):
            out = x.clone()
            u, v = x[..., :n], x[..., n:2 * n]
            out[..., :n] = u * c - v * s
            out[..., n:2 * n] = v * c + u * s
            return out
        qf, kf = turn(qf), turn(kf)
    for b in range(B):
        cnt = int(min(ln[b], T))
        if cnt <= 0:
            continue
        p0, s_ = int(p[b]), int(sl[b])
        kcache[s_, :, p0:p0 + cnt] = kf[b * T:b * T + cnt].transpose(0, 1) \
            .to(kcache.dtype)
        vcache[s_, :, p0:p0 + cnt] = k[b * T:b * T + cnt].reshape(
            cnt, nkv, d).transpose(0, 1).to(vcache.dtype)
    return qf.reshape(M, nq * d).to(qk.dtype)


def mul_sigmoid(a: torch.Tensor, gate_src: torch.Tensor,
                col0: int) -> torch.Tensor:
    """a [M, N] * sigmoid(gate_src[:, col0:col0+N]), fp32 math."""
    N = a.shape[1]
    return (a.float() * torch.sigmoid(gate_src[:, col0:col0 + N].float())
            ).to(a.dtype)
