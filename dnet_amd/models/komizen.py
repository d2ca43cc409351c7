"""Komizen ring model: heterogeneous sequence mixers on several fp32 residual
streams, with looped layer spans.

A layer is pre-norm, mixer then feed-forward, each sublayer reading from and
writing to S residual streams x_1..x_S (hyper-connections):

    u   = sum_s a_s x_s                        (read weights a  [S])
    y   = sublayer(rmsnorm(u) * (1 + g))       (norm weight stored around 0)
    x_t <- sum_s M[s, t] x_s + b_t y           (mix M [S, S], write b [S])

All streams start as the scaled embedding; the model output norms their sum.
Without streams in the configuration the same code runs one plain residual
(S = 1, a = b = M = 1).

Mixers (``cfg.layer_specs[run]["type"]``):

* ``latent_attention``: queries through a low-rank latent (down, RMS norm,
  up); keys and values share one cached latent per token, [RMS-normed latent
  | rotated key part] (interleaved rotation). Attention runs in the latent
  space: each head's plain query part is carried through its key
  up-projection first, the scores are taken against the cached rows, the
  softmax-weighted sum of the latents is carried through the head's value
  up-projection afterwards. Nothing per head is cached (unless the shared
  row is wider than the attention kernels' key row: then per-head keys and
  values are, see ``_expanded_attention``).
* ``delta``: gated delta rule. q/k/v pass short causal convolutions + SiLU;
  q, k are made unit vectors per head; per value head
  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, then a per-head
  RMS norm, an output gate and the output projection.
* ``mamba2``: selective state-space layer with a scalar decay per head
  (convolution over x, B, C; softplus step size; gate before a grouped norm).

Feed-forward: a mixture of ungated experts (up, squared ReLU, down); the
router takes a softmax over all experts, keeps the largest ``top`` and uses
their probabilities times a constant, not renormalized.

Layer loops: a span of stored layers may run several times in a row. The
configuration is unrolled into layer *runs* (``cfg.layer_weight_ids[run]`` is
the stored layer): runs of one stored layer share one ``LayerWeights`` object
and own separate cache / state entries, so the executor, the pipeline plan
and the cache see an ordinary stack.

Per-slot state lives in the framework's cache object: the latent rows in
``KVCache.k`` (one "kv head", no separate values), convolution tails and fp32
recurrent states in ``KVCache.state``. State is taken as zero at position 0
and never touched by padding or idle rows.

Checkpoint names: ``embed`` (also the output projection), ``final.norm``,
``l<i>.norm{1,2}``, ``l<i>.hc{1,2}.{in,out,mix}``,
``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,o}``,
``l<i>.mix.{q,k,v,q.conv,k.conv,v.conv,b,a,A_log,dt_bias,g,norm,o}``,
``l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o}``,
``l<i>.mlp.{router,e<j>.{up,down}}``.

``cfg.compute_dtype == "float32"`` runs weights, activations, caches and every
product in true fp32.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .. import ops
from .base import KVCache, LayerWeights, Linear, RingModel
from .config import ModelConfig

UNIT_EPS = 1e-6                 # inside the root of the delta rule's unit norms


class KomizenRingModel(RingModel):
    model_type = "komizen"
    model_types = ["komizen"]
    act_dtype = torch.float32          # residual streams / ring hops
    ragged_prefill = True
    supports_float32 = True
    stateful = True                    # idle decode rows must not step
    supports_offload = False           # layer kinds hold different tensors
    DENSE_MOE_MAX_T = 64
    # the attention kernels hold one key row of at most this many entries
    MAX_LATENT_ROW = 256

    def __init__(self, cfg: ModelConfig, layer_ids: Sequence[int], device,
                 is_first: bool, is_last: bool, smax: int = 4096, **kw):
        if kw.get("tp_size", 1) > 1 or kw.get("cp_size", 1) > 1:
            raise NotImplementedError(
                "komizen: tensor/context parallelism inside a stage is not "
                "implemented")
        assert cfg.layer_specs is not None, "komizen needs per-layer specs"
        assert cfg.quant is None, "komizen: bf16 / fp32 weights only"
        super().__init__(cfg, layer_ids, device, is_first, is_last,
                         smax=smax, **kw)
        self.wdtype = (torch.float32 if cfg.compute_dtype == "float32"
                       else torch.bfloat16)
        self.logits_dtype = self.wdtype
        self.streams = max(1, int(cfg.hc_streams))
        self._sum_in = torch.ones(self.streams, dtype=torch.float32,
                                  device=self.device)
        for lid in self.layer_ids:
            s = self._spec(lid)
            if s["type"] == "latent_attention" and not self._latent_fits(
                    s["mixer"]):
                m = s["mixer"]
                if max(m["dim"] + m["rot_dim"], m["vdim"]) \
                        > self.MAX_LATENT_ROW:
                    raise NotImplementedError(
                        f"komizen layer run {lid}: neither the latent row "
                        f"({m['kv_rank'] + m['rot_dim']}) nor the per-head "
                        f"key / value sizes fit the attention kernels' row "
                        f"of {self.MAX_LATENT_ROW}")

    def _init_positional(self):
        pass        # angles are computed from positions inside the kernels

    def _latent_fits(self, m: dict) -> bool:
        """Whether the shared row [latent | rotated key part] fits one key
        row of the attention kernels. If not, the layer caches per-head keys
        and values instead (same kernels, a larger cache)."""
        return m["kv_rank"] + m["rot_dim"] <= self.MAX_LATENT_ROW

    @property
    def hidden_width(self) -> int:
        return self.streams * self.cfg.hidden_size

    # ---------- per-run sizes ----------

    def _spec(self, lid: int) -> dict:
        return self.cfg.layer_specs[lid]

    def _stored(self, lid: int) -> int:
        ids = self.cfg.layer_weight_ids
        return lid if ids is None else ids[lid]

    @staticmethod
    def _ssm_dims(m: dict):
        heads, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
        return heads, P, N, G, heads * P, heads * P + 2 * G * N

    @staticmethod
    def _delta_dims(m: dict):
        H, KH, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        return H, KH, d, dv, 2 * KH * d + H * dv       # conv channels

    def make_kv_cache(self, batch: int, smax: int) -> KVCache:
        dims, states = [], []
        for lid in self.layer_ids:
            s = self._spec(lid)
            m = s["mixer"]
            taps = max(int(m.get("conv") or 1) - 1, 0)
            if s["type"] == "latent_attention":
                if self._latent_fits(m):
                    dims.append((1, m["kv_rank"] + m["rot_dim"], 0))
                else:
                    dims.append((m["heads"], m["dim"] + m["rot_dim"],
                                 m["vdim"]))
                states.append({})
            elif s["type"] == "delta":
                H, KH, d, dv, C = self._delta_dims(m)
                dims.append(None)
                states.append({"conv": ((taps, C), self.wdtype),
                               "S": ((H, d, dv), torch.float32)})
            else:
                heads, P, N, G, inner, C = self._ssm_dims(m)
                dims.append(None)
                states.append({"conv": ((taps, C), self.wdtype),
                               "ssm": ((heads, N, P), torch.float32)})
        return KVCache(self.cfg, self.layer_ids, batch, smax, self.device,
                       layer_dims=dims, dtype=self.wdtype,
                       layer_state=states)

    # ---------- weights ----------

    def _lin(self, w: torch.Tensor, bias=None) -> Linear:
        return Linear(w.to(self.wdtype).to(self.device).contiguous(), bias)

    def _vec(self, t: torch.Tensor) -> torch.Tensor:
        # small per-channel / per-head parameters feed fp32 math directly
        return t.to(torch.float32).to(self.device).contiguous()

    def _build_layer(self, spec: dict, get) -> LayerWeights:
        """Weights of one stored layer. ``get(name)`` returns the tensor
        ``l<i>.<name>``."""
        m = spec["mixer"]
        W = self.cfg.hidden_size
        S = self.streams
        # norm weights are stored around zero: the kernels take 1 + w
        lw = LayerWeights(attn_norm=self._vec(get("norm1")) + 1.0)
        for q in (1, 2):
            if q == 2 and spec.get("mlp") is None:
                continue
            if self.cfg.hc_streams:
                a, b, mx = (self._vec(get(f"hc{q}.{n}"))
                            for n in ("in", "out", "mix"))
                assert a.shape == (S,) and b.shape == (S,) \
                    and mx.shape == (S, S), "stream weights"
            else:
                a = torch.ones(1, dtype=torch.float32, device=self.device)
                b, mx = a.clone(), a.clone().view(1, 1)
            setattr(lw, f"hc{q}_in", a)
            setattr(lw, f"hc{q}_out", b)
            setattr(lw, f"hc{q}_mix", mx)
        if spec["type"] == "latent_attention":
            H, d, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            R, QR = m["kv_rank"], m["q_rank"]
            dq, dkv, uq = get("mix.dq"), get("mix.dkv"), get("mix.uq")
            uk, uv = get("mix.uk"), get("mix.uv")
            assert dq.shape == (QR, W) and dkv.shape == (R + rd, W) \
                and uq.shape == (H * (d + rd), QR) and uk.shape == (H * d, R) \
                and uv.shape == (H * dv, R), "latent attention shapes"
            lw.qkv = self._lin(torch.cat([dq, dkv]))        # [dq ; dkv]
            lw.q_a_norm = self._vec(get("mix.dq.norm"))
            lw.kv_a_norm = self._vec(get("mix.dkv.norm"))
            lw.q_b = self._lin(uq)
            # per-head up-projections as batched operands: keys [H, d, R]
            # (query side: q_h W_uk,h), values [H, R, dv]
            lw.uk = uk.to(self.wdtype).to(self.device).view(H, d, R) \
                .contiguous()
            lw.uv = uv.to(self.wdtype).to(self.device).view(H, dv, R) \
                .transpose(1, 2).contiguous()
            if not self._latent_fits(m):
                lw.kv_b = self._lin(torch.cat([uk, uv]))    # [uk ; uv]
            lw.o = self._lin(get("mix.o"))
            n = int(m["rot"]["dims"])
            f = [float(m["rot"]["base"]) ** (-2.0 * i / n)
                 for i in range(n // 2)]
            lw.rot_freq = torch.tensor(f, dtype=torch.float32,
                                       device=self.device)
        elif spec["type"] == "delta":
            H, KH, d, dv, C = self._delta_dims(m)
            q, k, v, g = (get("mix." + n) for n in "qkvg")
            wb, wa = get("mix.b"), get("mix.a")
            assert q.shape == (KH * d, W) and k.shape == (KH * d, W) \
                and v.shape == (H * dv, W) and g.shape == (H * dv, W) \
                and wb.shape == (H, W) and wa.shape == (H, W), "delta shapes"
            lw.qkv = self._lin(torch.cat([q, k, v, g, wb, wa]))
            lw.conv_w = self._vec(torch.cat(
                [get("mix.q.conv"), get("mix.k.conv"), get("mix.v.conv")]))
            assert lw.conv_w.shape == (C, int(m["conv"]))
            lw.conv_b = torch.zeros(C, dtype=torch.float32,
                                    device=self.device)
            lw.a_log = self._vec(get("mix.A_log"))
            lw.dt_bias = self._vec(get("mix.dt_bias"))
            # one norm weight of size vdim shared by the heads
            lw.delta_norm = self._vec(get("mix.norm")).repeat(H).contiguous()
            lw.o = self._lin(get("mix.o"))
        else:
            heads, P, N, G, inner, C = self._ssm_dims(m)
            win = get("mix.in")
            assert win.shape == (2 * inner + 2 * G * N + heads, W), \
                "state-space projection shape"
            lw.ssm_in = self._lin(win)
            lw.conv_w = self._vec(get("mix.conv"))
            assert lw.conv_w.shape == (C, int(m["conv"]))
            lw.conv_b = self._vec(get("mix.conv.b"))
            lw.dt_bias = self._vec(get("mix.dt_bias"))
            lw.a_log = self._vec(get("mix.A_log"))
            lw.dskip = self._vec(get("mix.D"))
            lw.ssm_norm = self._vec(get("mix.norm"))
            lw.o = self._lin(get("mix.o"))
        ff = spec.get("mlp")
        if ff is not None:
            E = int(ff["router"]["experts"])
            lw.mlp_norm = self._vec(get("norm2")) + 1.0
            # the router runs in fp32 whatever the activation dtype
            lw.router = Linear(self._vec(get("mlp.router")))
            lw.up_w = torch.stack([get(f"mlp.e{e}.up") for e in range(E)]) \
                .to(self.wdtype).to(self.device).contiguous()    # [E, I, W]
            lw.down_w = torch.stack([get(f"mlp.e{e}.down")
                                     for e in range(E)]) \
                .to(self.wdtype).to(self.device).contiguous()    # [E, W, I]
        return lw

    def _bind_runs(self, build) -> None:
        """One LayerWeights per stored layer, shared by all its runs."""
        made: dict = {}
        for lid in self.layer_ids:
            wid = self._stored(lid)
            if wid not in made:
                made[wid] = build(wid, self._spec(lid))
            self.layers[lid] = made[wid]

    def load_state_dict(self, sd: dict):
        self._bind_runs(lambda wid, spec: self._build_layer(
            spec, lambda n, p=f"l{wid}.": sd[p + n]))
        if self.is_first or self.is_last:
            emb = sd["embed"].to(self.wdtype).to(self.device).contiguous()
            if self.is_first:
                self.embed = emb
            if self.is_last:
                self.final_norm = self._vec(sd["final.norm"]) + 1.0
                self.lm_head = Linear(emb)       # tied, without the scale

    def init_random(self, seed: int = 0):
        """Seeded per stored layer id (any sharding of one (model, seed)
        holds the same global weights); scales keep every branch of
        comparable size."""
        c = self.cfg
        W = c.hidden_size
        S = self.streams
        gdev = self.device if self.device.type == "cuda" else "cpu"

        def gen(sub):
            g = torch.Generator(device=gdev)
            g.manual_seed(seed * 100003 + sub)
            return g

        def rn(g, *shape, std=1.0):
            return (torch.randn(*shape, generator=g, device=gdev)
                    * std).to(torch.bfloat16)

        def ru(g, n, lo, hi):
            return (torch.rand(n, generator=g, device=gdev)
                    * (hi - lo) + lo).to(torch.bfloat16)

        def lin(g, out, inp):
            return rn(g, out, inp, std=inp ** -0.5)

        def build(wid, spec):
            g = gen(wid)
            m = spec["mixer"]
            t = {"norm1": rn(g, W, std=0.1), "norm2": rn(g, W, std=0.1)}
            for q in (1, 2):
                t[f"hc{q}.in"] = ru(g, S, 0.5, 1.0) / S
                t[f"hc{q}.out"] = ru(g, S, 0.3, 1.0)
                t[f"hc{q}.mix"] = (torch.eye(S, device=gdev) * 0.8
                                   + rn(g, S, S, std=0.1).float()
                                   ).to(torch.bfloat16)
            if spec["type"] == "latent_attention":
                H, d, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
                R, QR = m["kv_rank"], m["q_rank"]
                t.update({"mix.dq": lin(g, QR, W),
                          "mix.dq.norm": 1 + rn(g, QR, std=0.1),
                          "mix.uq": lin(g, H * (d + rd), QR),
                          "mix.dkv": lin(g, R + rd, W),
                          "mix.dkv.norm": 1 + rn(g, R, std=0.1),
                          "mix.uk": lin(g, H * d, R),
                          "mix.uv": lin(g, H * dv, R),
                          "mix.o": lin(g, W, H * dv)})
            elif spec["type"] == "delta":
                H, KH, d, dv, C = self._delta_dims(m)
                taps = int(m["conv"])
                t.update({"mix.q": lin(g, KH * d, W),
                          "mix.k": lin(g, KH * d, W),
                          "mix.v": lin(g, H * dv, W),
                          "mix.g": lin(g, H * dv, W),
                          "mix.b": lin(g, H, W), "mix.a": lin(g, H, W),
                          "mix.q.conv": rn(g, KH * d, taps, std=0.5),
                          "mix.k.conv": rn(g, KH * d, taps, std=0.5),
                          "mix.v.conv": rn(g, H * dv, taps, std=0.5),
                          "mix.A_log": ru(g, H, -3.0, 0.5),
                          "mix.dt_bias": ru(g, H, -3.0, 0.0),
                          "mix.norm": 1 + rn(g, dv, std=0.1),
                          "mix.o": lin(g, W, H * dv)})
            else:
                heads, P, N, G, inner, C = self._ssm_dims(m)
                t.update({"mix.in": lin(g, 2 * inner + 2 * G * N + heads, W),
                          "mix.conv": rn(g, C, int(m["conv"]), std=0.5),
                          "mix.conv.b": rn(g, C, std=0.1),
                          "mix.dt_bias": ru(g, heads, -3.0, 0.0),
                          "mix.A_log": ru(g, heads, -1.0, 1.5),
                          "mix.D": rn(g, heads),
                          "mix.norm": 1 + rn(g, inner, std=0.1),
                          "mix.o": lin(g, W, inner)})
            ff = spec.get("mlp")
            if ff is not None:
                ef = ff["expert"]["ff"]
                t["mlp.router"] = lin(g, ff["router"]["experts"], W)
                for e in range(ff["router"]["experts"]):
                    t[f"mlp.e{e}.up"] = lin(g, ef, W)
                    t[f"mlp.e{e}.down"] = lin(g, W, ef)
            return self._build_layer(spec, t.__getitem__)

        self._bind_runs(build)
        if self.is_first or self.is_last:
            emb = rn(gen(99991), c.vocab_size, W, std=W ** -0.5).to(
                self.wdtype).to(self.device)
            if self.is_first:
                self.embed = emb
            if self.is_last:
                self.final_norm = self._vec(rn(gen(99993), W, std=0.1)) + 1.0
                self.lm_head = Linear(emb)

    # ---------- forward ----------

    def embed_tokens(self, tokens: torch.Tensor) -> torch.Tensor:
        """Every stream starts as the scaled embedding: [..., S*W] fp32."""
        assert self.embed is not None, "this shard does not own the embedding"
        x = torch.nn.functional.embedding(tokens, self.embed).to(
            torch.float32) * float(self.cfg.embedding_scale)
        if self.streams == 1:
            return x
        return x.repeat(*([1] * (x.dim() - 1)), self.streams)

    def _latent_attention(self, u, lw, m, kv, li, pos, T, lens, slots):
        H, d, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        R, QR = m["kv_rank"], m["q_rank"]
        M = u.shape[0]
        p = lw.qkv(u)                                  # [dq | dkv]
        cq = ops.rmsnorm_rows(p[:, :QR], lw.q_a_norm, self.cfg.rms_eps,
                              self.wdtype)
        q = lw.q_b(cq)                                 # [M, H*(d+rd)]
        if kv.v[li] is not None:
            return self._expanded_attention(p, q, lw, m, kv, li, pos, T,
                                            lens, slots)
        ops.latent_append(p, QR, lw.kv_a_norm, self.cfg.rms_eps, R,
                          lw.rot_freq, kv.k[li], pos, T, lens, slots)
        # plain query part into the latent space, head by head
        qabs = torch.bmm(q.view(M, H, d + rd)[:, :, :d].transpose(0, 1),
                         lw.uk)                        # [H, M, R]
        qf = ops.latent_q_pack(q, qabs, lw.rot_freq, pos, T, H, d)
        ol = ops.attn_mod(qf, kv.k[li], None, pos, T, float(m["scale"]),
                          lens, slots, v_dim=R)        # [M, H*R]
        ov = torch.bmm(ol.view(M, H, R).transpose(0, 1), lw.uv)
        return lw.o(ov.transpose(0, 1).reshape(M, H * dv))

    def _expanded_attention(self, p, q, lw, m, kv, li, pos, T, lens, slots):
        """Latent rows too wide for one key row of the kernels: per-head keys
        [plain | rotated shared part] and values are formed from the latent
        and cached. Padding and idle rows write where their slot's next real
        token is written later, before anything reads it."""
        H, d, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        R, QR = m["kv_rank"], m["q_rank"]
        M = p.shape[0]
        B = M // T
        c = ops.rmsnorm_rows(p[:, QR:QR + R], lw.kv_a_norm, self.cfg.rms_eps,
                             self.wdtype)
        kvu = lw.kv_b(c)                               # [ku (H*d) | v (H*dv)]
        ku = kvu[:, :H * d].reshape(M, H, d)
        kin = torch.cat([ku, p[:, QR + R:QR + R + rd].reshape(M, 1, rd)
                         .expand(M, H, rd)], dim=-1).reshape(M, H * (d + rd))
        # the rotation kernel of the query pack turns the rotated parts and
        # copies the plain ones
        k = ops.latent_q_pack(kin.contiguous(),
                              ku.transpose(0, 1).contiguous(), lw.rot_freq,
                              pos, T, H, d)
        qr = ops.latent_q_pack(
            q, q.view(M, H, d + rd)[:, :, :d].transpose(0, 1).contiguous(),
            lw.rot_freq, pos, T, H, d)
        smax = kv.k[li].shape[2]
        at = (pos.view(B, 1).long()
              + torch.arange(T, device=p.device)).clamp_(max=smax - 1)
        sl = (slots.long() if slots is not None
              else torch.arange(B, device=p.device)).view(B, 1)
        kv.k[li][sl, :, at] = k.view(B, T, H, d + rd)
        kv.v[li][sl, :, at] = kvu[:, H * d:].reshape(B, T, H, dv)
        a = ops.attn_mod(qr, kv.k[li], kv.v[li], pos, T, float(m["scale"]),
                         lens, slots)
        return lw.o(a)

    def _delta(self, u, lw, m, kv, li, pos, T, lens, slots):
        H, KH, d, dv, C = self._delta_dims(m)
        st = kv.state[li]
        p = lw.qkv(u)                          # [q | k | v | g | b | a]
        qkv = ops.causal_conv_silu(p, 0, lw.conv_w, lw.conv_b, st["conv"],
                                   pos, T, lens, slots)
        o = ops.gated_delta_scan(qkv, p, C + H * dv, C + H * dv + H,
                                 lw.a_log, lw.dt_bias, st["S"], pos, T, H,
                                 KH, d, dv, UNIT_EPS, lens, slots)
        og = ops.gated_group_rmsnorm(o, p, C, lw.delta_norm, H,
                                     self.cfg.rms_eps, "silu", False,
                                     self.wdtype)
        return lw.o(og)

    def _ssd(self, u, lw, m, kv, li, pos, T, lens, slots):
        heads, P, N, G, inner, C = self._ssm_dims(m)
        st = kv.state[li]
        zx = lw.ssm_in(u)                      # [z | x B C | dt]
        xbc = ops.causal_conv_silu(zx, inner, lw.conv_w, lw.conv_b,
                                   st["conv"], pos, T, lens, slots)
        y = ops.ssd_scan(xbc, zx, inner + C, lw.dt_bias, lw.a_log, lw.dskip,
                         st["ssm"], pos, T, heads, P, N, G, lens, slots)
        yg = ops.gated_group_rmsnorm(y, zx, 0, lw.ssm_norm,
                                     int(m["norm_groups"]), self.cfg.rms_eps,
                                     "silu", True, self.wdtype)
        return lw.o(yg)

    def _moe(self, u, lw, ff):
        T = u.shape[0]
        W = self.cfg.hidden_size
        E, top = int(ff["router"]["experts"]), int(ff["router"]["top"])
        we = ops.moe_route(lw.router(u.float()), top,
                           float(ff["router"]["scale"]))
        I = lw.up_w.shape[1]
        if (T * top < E and self.wdtype == torch.bfloat16
                and W % 8 == 0 and I % 8 == 0):
            # few rows, most experts idle: grouped expert kernels, two
            # launches, unrouted experts skipped on the device (no host
            # sync: graph-capturable), so only the chosen experts' weights
            # are read
            act = ops.moe_up_act(u, lw.up_w, we)
            return ops.moe_down(act, lw.down_w, None, None, we, 0, False)
        if T <= self.DENSE_MOE_MAX_T:
            # a decode batch that reaches most experts anyway: every expert
            # on every row as two batched products (each expert's weights
            # read once), weighted with zero for the experts a row did not
            # choose; no host sync
            z = torch.bmm(u.unsqueeze(0).expand(E, T, W),
                          lw.up_w.transpose(1, 2))              # [E, T, I]
            a = ops.act_slice(z.view(E * T, I), 0, I, "relu_sq")
            d = torch.bmm(a.view(E, T, I), lw.down_w.transpose(1, 2))
            return ops.moe_weighted_sum(d, we)
        out = torch.zeros(T, W, dtype=torch.float32, device=u.device)
        hit = (we > 0).any(dim=0).tolist()
        for e in range(E):
            if not hit[e]:
                continue
            rows = (we[:, e] > 0).nonzero(as_tuple=True)[0]
            a = ops.act_slice(u[rows] @ lw.up_w[e].t(), 0, I, "relu_sq")
            out.index_add_(0, rows, (a @ lw.down_w[e].t()).float()
                           * we[rows, e:e + 1])
        return out

    def _window(self, xs: torch.Tensor, layer_ids: Sequence[int],
                kv: KVCache, pos: torch.Tensor, T: int, lens, slots) -> None:
        """Run the layer runs of one window over the streams xs [B*T, S*W]
        fp32 (in place). Token (b, t) sits at position pos[b]+t of cache row
        slots[b]."""
        eps, wdt = self.cfg.rms_eps, self.wdtype
        u = None
        layer_ids = list(layer_ids)
        mixers = {"latent_attention": self._latent_attention,
                  "delta": self._delta, "mamba2": self._ssd}
        for i, lid in enumerate(layer_ids):
            lw = self._layer(lid)
            s = self._spec(lid)
            li = kv.local[lid]
            if u is None:
                u = ops.hc_read_norm(xs, lw.hc1_in, lw.attn_norm, eps, wdt)
            a = mixers[s["type"]](u, lw, s["mixer"], kv, li, pos, T, lens,
                                  slots)
            nxt = (self.layers[layer_ids[i + 1]]
                   if i + 1 < len(layer_ids)
                   and layer_ids[i + 1] in self.layers else None)
            n_in = nxt.hc1_in if nxt is not None else None
            n_wn = nxt.attn_norm if nxt is not None else None
            ff = s.get("mlp")
            if ff is not None:
                u2 = ops.hc_write(xs, a, lw.hc1_mix, lw.hc1_out, lw.hc2_in,
                                  lw.mlp_norm, eps, wdt)
                f = self._moe(u2, lw, ff)
                u = ops.hc_write(xs, f, lw.hc2_mix, lw.hc2_out, n_in, n_wn,
                                 eps, wdt)
            else:
                u = ops.hc_write(xs, a, lw.hc1_mix, lw.hc1_out, n_in, n_wn,
                                 eps, wdt)
            if self._obs_sync:
                self._profile_layer_sync(lid)

    def decode_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                      kv: KVCache) -> torch.Tensor:
        """One decode step. h [B, S*W] fp32, modified in place; kv.pos holds
        each row's write position; rows flagged in kv.idle keep their state
        (they run as padding)."""
        if layer_ids:
            self._window(h, layer_ids, kv, kv.pos, 1,
                         (~kv.idle).to(torch.int32), None)
        return h

    def prefill_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                       kv: KVCache, p0, lens: Optional[torch.Tensor] = None,
                       slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Prefill h [B, T, S*W] fp32 in place. ``p0``: first position, an
        int (every row) or an int32 tensor [B]. ``lens`` [B] int32: real
        token count per row (rows are right-padded to T; padding never
        reaches the cache or any state and its outputs are meaningless).
        ``slots`` [B] int32: cache row of each batch row (default: row b)."""
        if not layer_ids:
            return h
        B, T, HW = h.shape
        if not torch.is_tensor(p0):
            p0 = torch.full((B,), int(p0), dtype=torch.int32,
                            device=h.device)
        self._window(h.view(B * T, HW), layer_ids, kv, p0, T, lens, slots)
        return h

    def normalize_project(self, h: torch.Tensor) -> torch.Tensor:
        """Norm of the sum of the streams, then the tied output projection."""
        assert self.final_norm is not None and self.lm_head is not None
        y = ops.hc_read_norm(h, self._sum_in, self.final_norm,
                             self.cfg.rms_eps, self.wdtype)
        return self.lm_head(y)

    def weight_bytes(self) -> int:
        """Bytes of every tensor and linear the resident layers hold (each
        stored layer once, however many runs share it)."""
        def size(v) -> int:
            if isinstance(v, Linear):
                return v.nbytes()
            if torch.is_tensor(v):
                return v.numel() * v.element_size()
            return 0
        seen = {id(lw): lw for lw in self.layers.values()}
        return sum(size(v) for lw in seen.values()
                   for v in vars(lw).values())
