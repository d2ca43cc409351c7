"""Plain, slow Lurisun forward pass: one function per mechanism, written from
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


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def silu(x):
    return x / (1.0 + torch.exp(-x))


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def input_conv(h, w):
    """h [T, C]; w [C, taps]; the last column multiplies the current token,
    tokens before the sequence count as zero. Returns h + conv(h)."""
    T, C = h.shape
    taps = w.shape[1]
    y = h.clone()
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] = y[t] + w[:, j] * h[src]
    return y


def hashed_pair_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for each token: a hash of (previous, current);
    the first token of a sequence takes the extra last row."""
    rows = []
    for t, tok in enumerate(tokens):
        if t == 0:
            rows.append(buckets)
        else:
            rows.append((int(tokens[t - 1]) * mul_prev + int(tok) * mul_cur)
                        % buckets)
    return rows


def embed(tokens, sd, cfg):
    x = sd["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        rows = hashed_pair_rows(list(tokens), int(bg["buckets"]),
                                int(bg["mul_prev"]), int(bg["mul_cur"]))
        x = x + sd["bigram"][torch.tensor(rows, dtype=torch.long)]
    return x


def rotate_half(x, pos, base, dims):
    """x [..., d] at integer position pos: channel i pairs with i + dims/2
    for i < dims/2; the channels from dims on pass through."""
    out = x.clone()
    half = dims // 2
    for i in range(half):
        a = pos * (base ** (-2.0 * i / dims))
        c, s = math.cos(a), math.sin(a)
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def lightning_mixer(h, p, m, eps):
    """Linear attention with a constant decay per head. h [T, W]."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ p["q"].T).view(T, H, d)
    k = silu(h @ p["k"].T).view(T, H, d)
    v = silu(h @ p["v"].T).view(T, H, dv)
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    decay = torch.tensor([float(x) for x in m["decay"]], dtype=h.dtype)
    for t in range(T):
        S = decay.view(H, 1, 1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    y = norm_plain(o.reshape(T, H * dv), p["norm"], eps)
    y = y * sigmoid(h @ p["g"].T)
    return y @ p["o"].T


def gated_sigmoid_attention(h, p, m, eps):
    """Grouped-head attention in chunks with element-wise sigmoid weights
    (no normalization over keys); the values are the unnormed, unrotated
    key projections."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    assert d == dv
    q = h @ p["q"].T + p["q.b"]
    k = h @ p["k"].T + p["k.b"]
    v = k.view(T, G, dv)
    q = norm_plain(q, p["q.norm"], eps).view(T, H, d)
    k = norm_plain(k, p["k.norm"], eps).view(T, G, d)
    rot = m.get("rot")
    if rot and int(rot["dims"]) >= 2:
        q = torch.stack([rotate_half(q[t], t, float(rot["base"]),
                                     int(rot["dims"])) for t in range(T)])
        k = torch.stack([rotate_half(k[t], t, float(rot["base"]),
                                     int(rot["dims"])) for t in range(T)])
    size = int(m["mask"]["size"])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for i in range(T):
        lo = (i // size) * size
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hh]) * float(m["scale"])
            w = sigmoid(s + p["pb"][hh])
            out[i, hh] = w @ v[lo:i + 1, g]
    return out.reshape(T, H * dv) @ p["o"].T


def latent_window_attention(h, p, m, eps):
    """Queries and keys/values through low-rank latents, no positions, a
    sliding window, softmax, sigmoid output gate."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    cq = norm_plain(h @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).view(T, H, d)
    c = norm_plain(h @ p["dkv"].T, p["dkv.norm"], eps)
    k = (c @ p["uk"].T).view(T, H, d)
    v = (c @ p["uv"].T).view(T, H, dv)
    size = int(m["mask"]["size"])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - size + 1)
        for hh in range(H):
            s = (k[lo:i + 1, hh] @ q[i, hh]) * float(m["scale"])
            w = torch.softmax(s, dim=0)
            out[i, hh] = w @ v[lo:i + 1, hh]
    y = out.reshape(T, H * dv) * sigmoid(h @ p["g"].T)
    return y @ p["o"].T


def dense_ff(h, p):
    return (silu(h @ p["gate"].T) * (h @ p["up"].T)) @ p["down"].T


MIXERS = {"lightning": lightning_mixer, "attention": gated_sigmoid_attention,
          "latent_attention": latent_window_attention}


def sub(sd, prefix):
    n = len(prefix)
    return {k[n:]: v for k, v in sd.items() if k.startswith(prefix)}


def forward(tokens, sd, cfg, dtype=torch.float32, layers_out=None):
    """Logits [T, vocab] of one whole sequence. ``layers_out`` (a list)
    receives the residual after every layer."""
    sd = {k: (v.to(dtype) if v.is_floating_point() else v)
          for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, sd, cfg)
    for i, spec in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = x
        if f"{pre}canon1" in sd:
            h = input_conv(x, sd[f"{pre}canon1"])
        y = MIXERS[spec["type"]](h, sub(sd, pre + "mix."), spec["mixer"], eps)
        x = x + norm_plain(y, sd[f"{pre}norm1"], eps)
        if spec.get("mlp") is not None:
            y = dense_ff(x, sub(sd, pre + "mlp."))
            x = x + norm_plain(y, sd[f"{pre}norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    y = norm_plain(x, sd["final.norm"], eps)
    return (y @ sd["head"].T) * float(cfg.get("logit_scale", 1.0))


def make_checkpoint(cfg, seed=0, dtype=torch.bfloat16, ff_gain=1.0):
    """Random tensors for a config.json dict, under the checkpoint's names;
    values are rounded to ``dtype`` (so a bfloat16 and a float32 run read the
    same numbers)."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    def lin(out, inp, gain=1.0):
        return rn(out, inp, std=gain * inp ** -0.5)

    sd = {"embed": rn(V, W), "final.norm": 1 + rn(W, std=0.1),
          "head": lin(V, W)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        sd["bigram"] = rn(int(bg["buckets"]) + 1, W, std=0.7)
    taps = int((cfg.get("canon") or {}).get("taps") or 0)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        sd[p + "norm1"] = 1 + rn(W, std=0.1)
        if taps:
            sd[p + "canon1"] = rn(W, taps, std=0.4)
        if spec["type"] == "lightning":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            sd.update({p + "mix.q": lin(H * d, W), p + "mix.k": lin(H * d, W),
                       p + "mix.v": lin(H * dv, W),
                       p + "mix.g": lin(H * dv, W),
                       p + "mix.norm": 1 + rn(H * dv, std=0.1),
                       p + "mix.o": lin(W, H * dv)})
        elif spec["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            sd.update({p + "mix.q": lin(H * d, W), p + "mix.k": lin(G * d, W),
                       p + "mix.q.b": rn(H * d, std=0.2),
                       p + "mix.k.b": rn(G * d, std=0.2),
                       p + "mix.q.norm": 1 + rn(H * d, std=0.1),
                       p + "mix.k.norm": 1 + rn(G * d, std=0.1),
                       p + "mix.pb": rn(H, std=0.5) - 1.5,
                       p + "mix.o": lin(W, H * m["vdim"])})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            R, QR = m["kv_rank"], m["q_rank"]
            sd.update({p + "mix.dq": lin(QR, W),
                       p + "mix.dq.norm": 1 + rn(QR, std=0.1),
                       p + "mix.uq": lin(H * d, QR, 2.0),
                       p + "mix.dkv": lin(R, W),
                       p + "mix.dkv.norm": 1 + rn(R, std=0.1),
                       p + "mix.uk": lin(H * d, R, 2.0),
                       p + "mix.uv": lin(H * dv, R),
                       p + "mix.g": lin(H * dv, W),
                       p + "mix.o": lin(W, H * dv)})
        ff = spec.get("mlp")
        if ff is not None:
            sd.update({p + "norm2": (1 + rn(W, std=0.1)) * ff_gain,
                       p + "mlp.gate": lin(ff["ff"], W),
                       p + "mlp.up": lin(ff["ff"], W),
                       p + "mlp.down": lin(W, ff["ff"])})
    return sd
