"""Plain, slow Komizen forward pass: one function per mechanism, written from
the design's equations with nothing shared with the framework's model code.

Everything runs token by token (or as one dense matrix per sequence) in one
floating dtype, on whole sequences, without any cache: a test feeds a prompt
and compares the framework's cached / batched / chunked results against it.

``cfg`` is the checkpoint's config.json as a dict; ``sd`` maps tensor names
to tensors.
"""
from __future__ import annotations

import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_centered(x, w, eps):
    """Layer / final norm: the stored weight sits around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def silu(x):
    return x / (1.0 + torch.exp(-x))


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def short_conv(x, w, b=None):
    """x [T, C]; w [C, taps], last column multiplies the current token."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += w[:, j] * x[src]
    if b is not None:
        y = y + b
    return y


def rotate_interleaved(x, pos, base, dims):
    """x [..., d] at integer position pos: pairs (2i, 2i+1), i < dims/2."""
    out = x.clone()
    for i in range(dims // 2):
        a = pos * (base ** (-2.0 * i / dims))
        c, s = math.cos(a), math.sin(a)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def delta_mixer(h, p, m, eps):
    """Gated delta rule. h [T, W]; p: the mixer's tensors by short name."""
    T = h.shape[0]
    H, KH, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ p["q"].T, p["q.conv"]))
    k = silu(short_conv(h @ p["k"].T, p["k.conv"]))
    v = silu(short_conv(h @ p["v"].T, p["v.conv"]))
    q = q.view(T, KH, d)
    k = k.view(T, KH, d)
    v = v.view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ p["b"].T)                          # [T, H]
    g = torch.exp(-torch.exp(p["A_log"]) * softplus(h @ p["a"].T + p["dt_bias"]))
    gate = silu(h @ p["g"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        kh = hd // (H // KH)
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hd] = S.T @ q[t, kh]
    out = rms_unit(out, eps) * p["norm"] * gate
    return out.reshape(T, H * dv) @ p["o"].T


def mamba2_mixer(h, p, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    zx = h @ p["in"].T
    z = zx[:, :inner]
    xbc = silu(short_conv(zx[:, inner:2 * inner + 2 * G * N], p["conv"], p["conv.b"]))
    dt = softplus(zx[:, 2 * inner + 2 * G * N:] + p["dt_bias"])   # [T, H]
    x = xbc[:, :inner].view(T, H, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    y = torch.zeros(T, H, P, dtype=h.dtype)
    for hd in range(H):
        gi = hd // (H // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        a = torch.exp(p["A_log"][hd])
        for t in range(T):
            S = torch.exp(-a * dt[t, hd]) * S + dt[t, hd] * torch.outer(Bm[t, gi], x[t, hd])
            y[t, hd] = S.T @ Cm[t, gi] + p["D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * p["norm"]
    return y @ p["o"].T


def latent_attention_mixer(h, p, m, eps):
    T = h.shape[0]
    H, d, rd, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    cq = norm_plain(h @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).view(T, H, d + rd)
    dkv = h @ p["dkv"].T
    c = norm_plain(dkv[:, :R], p["dkv.norm"], eps)
    kr = dkv[:, R:]                                        # [T, rd]
    ku = (c @ p["uk"].T).view(T, H, d)
    v = (c @ p["uv"].T).view(T, H, dv)
    qr = torch.stack([rotate_interleaved(q[t, :, d:], t, base, dims) for t in range(T)])
    krr = torch.stack([rotate_interleaved(kr[t], t, base, dims) for t in range(T)])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        s = (q[:, hd, :d] @ ku[:, hd].T + qr[:, hd] @ krr.T) * float(m["scale"])
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), float("-inf"))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, hd]
    return out.reshape(T, H * dv) @ p["o"].T


def moe_ff(h, p, ff):
    E, top = ff["router"]["experts"], ff["router"]["top"]
    s = torch.softmax(h @ p["router"].T, dim=-1)
    out = torch.zeros(h.shape[0], p["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            a = torch.relu(p[f"e{e}.up"] @ h[t]) ** 2
            out[t] += float(ff["router"]["scale"]) * s[t, e] * (p[f"e{e}.down"] @ a)
    return out


MIXERS = {"delta": delta_mixer, "mamba2": mamba2_mixer,
          "latent_attention": latent_attention_mixer}


def layer_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, k = lp["start"], lp["stop"], lp["times"]
    return list(range(a)) + list(range(a, b)) * k + list(range(b, n))


def sub(sd, prefix, dtype):
    return {k[len(prefix):]: v.to(dtype) for k, v in sd.items()
            if k.startswith(prefix)}


def forward(cfg, sd, tokens, dtype=torch.float32, layers_out=None):
    """tokens: list of ints -> logits [T, vocab]. ``layers_out``: a list that
    receives the residual (sum of the streams) after every layer run."""
    eps = cfg["norm"]["eps"]
    emb = sd["embed"].to(dtype)
    x0 = emb[torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    S = cfg.get("streams")
    xs = [x0.clone() for _ in range(S)] if S else None
    x = x0
    for li in layer_order(cfg):
        spec = cfg["layers"][li]
        pre = f"l{li}."
        subs = [(1, lambda u, spec=spec, pre=pre: MIXERS[spec["type"]](
            u, sub(sd, pre + "mix.", dtype), spec["mixer"], eps))]
        if spec.get("mlp") is not None:
            subs.append((2, lambda u, spec=spec, pre=pre: moe_ff(
                u, sub(sd, pre + "mlp.", dtype), spec["mlp"])))
        for qn, fn in subs:
            w = sd[f"{pre}norm{qn}"].to(dtype)
            if S:
                hin = sd[f"{pre}hc{qn}.in"].to(dtype)
                hmix = sd[f"{pre}hc{qn}.mix"].to(dtype)
                hout = sd[f"{pre}hc{qn}.out"].to(dtype)
                u = sum(hin[s] * xs[s] for s in range(S))
                y = fn(norm_centered(u, w, eps))
                xs = [sum(hmix[s, t] * xs[s] for s in range(S)) + hout[t] * y
                      for t in range(S)]
            else:
                x = x + fn(norm_centered(x, w, eps))
        if layers_out is not None:
            layers_out.append(sum(xs) if S else x.clone())
    if S:
        x = sum(xs)
    x = norm_centered(x, sd["final.norm"].to(dtype), eps)
    return x @ emb.T


def make_checkpoint(cfg, seed=0, ff_gain=1.0):
    """Random bf16 tensors under the checkpoint's names for a config dict;
    scales keep every branch of comparable size. ``ff_gain`` scales the
    experts' output: bfloat16 comparisons use a small one, so that a token
    whose router sits on a near-tie that rounding flips moves the logits
    little (input-dependent routing is compared in float32)."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams")

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    def ru(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).to(torch.bfloat16)

    def lin(out, inp):
        return rn(out, inp, std=inp ** -0.5)

    sd = {"embed": rn(cfg["vocab"], W, std=W ** -0.5),
          "final.norm": rn(W, std=0.1)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        sd[p + "norm1"] = rn(W, std=0.1)
        subs = [1] + ([2] if spec.get("mlp") else [])
        if S:
            for q in subs:
                sd[p + f"hc{q}.in"] = ru(S, 0.5, 1.0) / S
                sd[p + f"hc{q}.out"] = ru(S, 0.3, 1.0)
                sd[p + f"hc{q}.mix"] = (torch.eye(S) * 0.8 + torch.randn(
                    S, S, generator=g) * 0.15).to(torch.bfloat16)
        if spec["type"] == "latent_attention":
            H, d, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            R, QR = m["kv_rank"], m["q_rank"]
            sd.update({p + "mix.dq": lin(QR, W),
                       p + "mix.dq.norm": 1 + rn(QR, std=0.1),
                       p + "mix.uq": lin(H * (d + rd), QR) * 2,
                       p + "mix.dkv": lin(R + rd, W),
                       p + "mix.dkv.norm": 1 + rn(R, std=0.1),
                       p + "mix.uk": lin(H * d, R) * 2,
                       p + "mix.uv": lin(H * dv, R),
                       p + "mix.o": lin(W, H * dv)})
        elif spec["type"] == "delta":
            H, KH, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            taps = m["conv"]
            sd.update({p + "mix.q": lin(KH * d, W), p + "mix.k": lin(KH * d, W),
                       p + "mix.v": lin(H * dv, W), p + "mix.g": lin(H * dv, W),
                       p + "mix.b": lin(H, W), p + "mix.a": lin(H, W),
                       p + "mix.q.conv": rn(KH * d, taps, std=0.5),
                       p + "mix.k.conv": rn(KH * d, taps, std=0.5),
                       p + "mix.v.conv": rn(H * dv, taps, std=0.5),
                       p + "mix.A_log": ru(H, -3.0, 0.5),
                       p + "mix.dt_bias": ru(H, -3.0, 0.0),
                       p + "mix.norm": 1 + rn(dv, std=0.1),
                       p + "mix.o": lin(W, H * dv)})
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, C = H * P, H * P + 2 * G * N
            sd.update({p + "mix.in": lin(2 * inner + 2 * G * N + H, W),
                       p + "mix.conv": rn(C, m["conv"], std=0.5),
                       p + "mix.conv.b": rn(C, std=0.1),
                       p + "mix.dt_bias": ru(H, -3.0, 0.0),
                       p + "mix.A_log": ru(H, -1.0, 1.5),
                       p + "mix.D": rn(H),
                       p + "mix.norm": 1 + rn(inner, std=0.1),
                       p + "mix.o": lin(W, inner)})
        ff = spec.get("mlp")
        if ff:
            sd[p + "norm2"] = rn(W, std=0.1)
            sd[p + "mlp.router"] = lin(ff["router"]["experts"], W) * 3
            for e in range(ff["router"]["experts"]):
                sd[p + f"mlp.e{e}.up"] = lin(ff["expert"]["ff"], W)
                sd[p + f"mlp.e{e}.down"] = lin(W, ff["expert"]["ff"]) * ff_gain
    return sd
