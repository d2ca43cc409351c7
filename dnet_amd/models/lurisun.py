"""Lurisun ring model: three kinds of sequence mixers on an fp32 residual,
each sublayer's OUTPUT normalized before it is added.

    x0 = embed[token] + pair[hash(previous token, token)]
    h  = x + conv(x)          (causal per-channel convolution over time)
    x <- x + rmsnorm(mixer(h)) * g1
    x <- x + rmsnorm(ff(x)) * g2          (ff = down(silu(gate x) * up x))
    logits = head(rmsnorm(x) * g) * logit_scale

The sublayers read the residual itself (no norm in front). The pair table has
``buckets`` hashed rows, (previous * mul_prev + token * mul_cur) mod buckets,
and one more row for a sequence's first token.

Mixers (``cfg.layer_specs[l]["type"]``):

* ``lightning``: linear attention with one constant decay per head,
  q, k, v = silu(projections); S <- decay_h S + k v^T, o = S^T q; the heads
  together are RMS-normalized, gated by sigmoid(W_g h) and projected.
* ``attention``: grouped heads with projection biases; q and k are
  RMS-normalized over their whole projection, then rotated (half-split
  pairs on the first ``rot.dims`` channels of a head); the values are the key
  projections as they come (before norm and rotation). A query sees the keys
  of its own block of ``mask.size`` positions only; a visible key weighs
  sigmoid(score + b_h), without any normalization over the keys.
* ``latent_attention``: queries through a low-rank latent (down, RMS norm,
  up); keys and values from one cached RMS-normed latent per token, no
  positions. Attention runs in the latent space (each head's query is
  carried through its key up-projection, the softmax-weighted latent through
  its value up-projection), over a sliding window of ``mask.size`` tokens,
  then a sigmoid gate from the layer input and the output projection. A
  latent wider than the attention kernels' key row is expanded into per-head
  keys and values in the cache instead.

Per-slot state lives in the framework's cache object: keys/values or the
latent rows in ``KVCache.k`` / ``KVCache.v``, the convolution's input tail
and the fp32 recurrent state in ``KVCache.state``, the sequence's last token
in ``KVCache.model_state``. State is taken as zero at position 0 and never
touched by padding or idle rows, so slots are reused without a reset and a
ragged batch equals each row alone.

Checkpoint names: ``embed``, ``bigram``, ``l<i>.canon1``, ``l<i>.norm{1,2}``,
``l<i>.mix.{q,k,v,g,o,norm}``, ``l<i>.mix.{q,q.b,k,k.b,q.norm,k.norm,pb,o}``,
``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,g,o}``,
``l<i>.mlp.{gate,up,down}``, ``final.norm``, ``head``.

``cfg.compute_dtype == "float32"`` runs weights, activations, caches and every
product in true fp32.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .. import ops
from .base import KVCache, LayerWeights, Linear, RingModel
from .config import ModelConfig


class LurisunRingModel(RingModel):
    model_type = "lurisun"
    model_types = ["lurisun"]
    act_dtype = torch.float32          # residual stream / ring hops
    ragged_prefill = True
    supports_float32 = True
    stateful = True                    # idle decode rows must not step
    supports_offload = False           # layer kinds hold different tensors
    # the embedding reads and advances the slot's last token: the executor
    # hands it the cache and the rows' geometry
    embed_reads_cache = True
    # the attention kernels hold one key row of at most this many entries
    MAX_KEY_ROW = 256

    def __init__(self, cfg: ModelConfig, layer_ids: Sequence[int], device,
                 is_first: bool, is_last: bool, smax: int = 4096, **kw):
        if kw.get("tp_size", 1) > 1 or kw.get("cp_size", 1) > 1:
            raise NotImplementedError(
                "lurisun: tensor/context parallelism inside a stage is not "
                "implemented")
        assert cfg.layer_specs is not None, "lurisun needs per-layer specs"
        assert cfg.quant is None, "lurisun: bf16 / fp32 weights only"
        super().__init__(cfg, layer_ids, device, is_first, is_last,
                         smax=smax, **kw)
        self.wdtype = (torch.float32 if cfg.compute_dtype == "float32"
                       else torch.bfloat16)
        self.logits_dtype = self.wdtype
        self.pair_table: Optional[torch.Tensor] = None
        self._no_rot = torch.zeros(0, dtype=torch.float32,
                                   device=self.device)
        for lid in self.layer_ids:
            s = self._spec(lid)
            m = s["mixer"]
            if s["type"] == "attention" and m["dim"] > self.MAX_KEY_ROW:
                raise NotImplementedError(
                    f"lurisun layer {lid}: head size {m['dim']} exceeds the "
                    f"attention kernels' row of {self.MAX_KEY_ROW}")
            if s["type"] == "latent_attention" and not self._latent_fits(m) \
                    and max(m["dim"], m["vdim"]) > self.MAX_KEY_ROW:
                raise NotImplementedError(
                    f"lurisun layer {lid}: neither the latent row nor the "
                    f"per-head sizes fit the attention kernels' row of "
                    f"{self.MAX_KEY_ROW}")

    def _init_positional(self):
        pass        # angles are computed from positions inside the kernels

    def _spec(self, lid: int) -> dict:
        return self.cfg.layer_specs[lid]

    def _latent_fits(self, m: dict) -> bool:
        return m["kv_rank"] <= self.MAX_KEY_ROW

    def make_kv_cache(self, batch: int, smax: int) -> KVCache:
        W = self.cfg.hidden_size
        conv = int(self.cfg.input_conv_taps)
        dims, states = [], []
        for lid in self.layer_ids:
            s = self._spec(lid)
            m = s["mixer"]
            st = {}
            if conv:                # a one-tap convolution has an empty tail
                st["conv"] = ((conv - 1, W), torch.float32)
            if s["type"] == "attention":
                dims.append((m["kv_heads"], m["dim"], m["vdim"]))
            elif s["type"] == "latent_attention":
                if self._latent_fits(m):
                    dims.append((1, m["kv_rank"], 0))
                else:
                    dims.append((m["heads"], m["dim"], m["vdim"]))
            else:
                dims.append(None)
                st["S"] = ((m["heads"], m["dim"], m["vdim"]), torch.float32)
            states.append(st)
        ms = None
        if self.is_first and self.cfg.pair_embedding:
            ms = {"prev_token": ((), torch.int32)}
        return KVCache(self.cfg, self.layer_ids, batch, smax, self.device,
                       layer_dims=dims, dtype=self.wdtype,
                       layer_state=states, model_state=ms)

    # ---------- weights ----------

    def _lin(self, w: torch.Tensor, bias=None) -> Linear:
        if bias is not None:
            bias = bias.to(self.wdtype).to(self.device).contiguous()
        return Linear(w.to(self.wdtype).to(self.device).contiguous(), bias)

    def _vec(self, t: torch.Tensor) -> torch.Tensor:
        # small per-channel / per-head parameters feed fp32 math directly
        return t.to(torch.float32).to(self.device).contiguous()

    def _build_layer(self, lid: int, get) -> LayerWeights:
        s = self._spec(lid)
        m = s["mixer"]
        W = self.cfg.hidden_size
        lw = LayerWeights(attn_norm=self._vec(get("norm1")))
        assert lw.attn_norm.shape == (W,)
        lw.conv_w = None
        if self.cfg.input_conv_taps:
            lw.conv_w = self._vec(get("canon1"))
            assert lw.conv_w.shape == (W, int(self.cfg.input_conv_taps)), \
                f"layer {lid}: input convolution shape"
        if s["type"] == "lightning":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            q, k, v, g = (get("mix." + n) for n in "qkvg")
            assert q.shape == (H * d, W) and k.shape == (H * d, W) \
                and v.shape == (H * dv, W) and g.shape == (H * dv, W), \
                f"layer {lid}: linear attention shapes"
            lw.qkv = self._lin(torch.cat([q, k, v, g]))     # [q | k | v | g]
            lw.decay = torch.tensor([float(x) for x in m["decay"]],
                                    dtype=torch.float32, device=self.device)
            lw.mix_norm = self._vec(get("mix.norm"))
            assert lw.mix_norm.shape == (H * dv,)
            lw.o = self._lin(get("mix.o"))
        elif s["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            q, k = get("mix.q"), get("mix.k")
            assert q.shape == (H * d, W) and k.shape == (G * d, W), \
                f"layer {lid}: attention shapes"
            lw.qkv = self._lin(torch.cat([q, k]),
                               torch.cat([get("mix.q.b"), get("mix.k.b")]))
            lw.q_norm = self._vec(get("mix.q.norm"))
            lw.k_norm = self._vec(get("mix.k.norm"))
            assert lw.q_norm.shape == (H * d,) and lw.k_norm.shape == (G * d,)
            lw.score_bias = self._vec(get("mix.pb"))
            assert lw.score_bias.shape == (H,)
            rot = m.get("rot")
            lw.rot_freq = None
            if rot and int(rot["dims"]) >= 2:
                n = int(rot["dims"])
                f = [float(rot["base"]) ** (-2.0 * i / n)
                     for i in range(n // 2)]
                lw.rot_freq = torch.tensor(f, dtype=torch.float32,
                                           device=self.device)
            lw.o = self._lin(get("mix.o"))
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            R, QR = m["kv_rank"], m["q_rank"]
            dq, dkv, g = get("mix.dq"), get("mix.dkv"), get("mix.g")
            uq, uk, uv = get("mix.uq"), get("mix.uk"), get("mix.uv")
            assert dq.shape == (QR, W) and dkv.shape == (R, W) \
                and g.shape == (H * dv, W) and uq.shape == (H * d, QR) \
                and uk.shape == (H * d, R) and uv.shape == (H * dv, R), \
                f"layer {lid}: latent attention shapes"
            lw.qkv = self._lin(torch.cat([dq, dkv, g]))     # [dq | dkv | g]
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
        ff = s.get("mlp")
        lw.gateup = None
        if ff is not None:
            gate, up = get("mlp.gate"), get("mlp.up")
            assert gate.shape == (ff["ff"], W) and up.shape == (ff["ff"], W)
            lw.mlp_norm = self._vec(get("norm2"))
            lw.gateup = self._lin(torch.cat([gate, up]))
            lw.down = self._lin(get("mlp.down"))
        return lw

    def _finish_ends(self, embed, pair, final_norm, head):
        if self.is_first:
            self.embed = embed.to(self.wdtype).to(self.device).contiguous()
            if self.cfg.pair_embedding:
                self.pair_table = pair.to(self.wdtype).to(
                    self.device).contiguous()
                assert self.pair_table.shape == (
                    int(self.cfg.pair_embedding["buckets"]) + 1,
                    self.cfg.hidden_size), "pair table shape"
        if self.is_last:
            # the factor on the logits rides on the fp32 norm weight
            self.final_norm = self._vec(final_norm) * float(
                self.cfg.logit_scale)
            self.lm_head = self._lin(head)

    def load_state_dict(self, sd: dict):
        for lid in self.layer_ids:
            self.layers[lid] = self._build_layer(
                lid, lambda n, p=f"l{lid}.": sd[p + n])
        self._finish_ends(sd.get("embed"), sd.get("bigram"),
                          sd.get("final.norm"), sd.get("head"))

    def init_random(self, seed: int = 0):
        """Seeded per layer id (any sharding of one (model, seed) holds the
        same global weights); scales keep every branch of comparable size."""
        c = self.cfg
        W = c.hidden_size
        gdev = self.device if self.device.type == "cuda" else "cpu"

        def gen(sub):
            g = torch.Generator(device=gdev)
            g.manual_seed(seed * 100003 + sub)
            return g

        def rn(g, *shape, std=1.0):
            return (torch.randn(*shape, generator=g, device=gdev)
                    * std).to(torch.bfloat16)

        def lin(g, out, inp):
            return rn(g, out, inp, std=inp ** -0.5)

        for lid in self.layer_ids:
            g = gen(lid)
            s = self._spec(lid)
            m = s["mixer"]
            t = {"norm1": 1 + rn(g, W, std=0.1),
                 "norm2": 1 + rn(g, W, std=0.1)}
            if c.input_conv_taps:
                t["canon1"] = rn(g, W, int(c.input_conv_taps), std=0.3)
            if s["type"] == "lightning":
                H, d, dv = m["heads"], m["dim"], m["vdim"]
                t.update({"mix.q": lin(g, H * d, W), "mix.k": lin(g, H * d, W),
                          "mix.v": lin(g, H * dv, W),
                          "mix.g": lin(g, H * dv, W),
                          "mix.norm": 1 + rn(g, H * dv, std=0.1),
                          "mix.o": lin(g, W, H * dv)})
            elif s["type"] == "attention":
                H, G, d = m["heads"], m["kv_heads"], m["dim"]
                t.update({"mix.q": lin(g, H * d, W), "mix.k": lin(g, G * d, W),
                          "mix.q.b": rn(g, H * d, std=0.1),
                          "mix.k.b": rn(g, G * d, std=0.1),
                          "mix.q.norm": 1 + rn(g, H * d, std=0.1),
                          "mix.k.norm": 1 + rn(g, G * d, std=0.1),
                          "mix.pb": rn(g, H, std=0.5) - 2.0,
                          "mix.o": lin(g, W, H * m["vdim"])})
            else:
                H, d, dv = m["heads"], m["dim"], m["vdim"]
                R, QR = m["kv_rank"], m["q_rank"]
                t.update({"mix.dq": lin(g, QR, W),
                          "mix.dq.norm": 1 + rn(g, QR, std=0.1),
                          "mix.uq": lin(g, H * d, QR),
                          "mix.dkv": lin(g, R, W),
                          "mix.dkv.norm": 1 + rn(g, R, std=0.1),
                          "mix.uk": lin(g, H * d, R),
                          "mix.uv": lin(g, H * dv, R),
                          "mix.g": lin(g, H * dv, W),
                          "mix.o": lin(g, W, H * dv)})
            ff = s.get("mlp")
            if ff is not None:
                t["mlp.gate"] = lin(g, ff["ff"], W)
                t["mlp.up"] = lin(g, ff["ff"], W)
                t["mlp.down"] = lin(g, W, ff["ff"])
            self.layers[lid] = self._build_layer(lid, t.__getitem__)
        pair = None
        if c.pair_embedding:
            pair = rn(gen(99994), int(c.pair_embedding["buckets"]) + 1, W,
                      std=0.5)
        self._finish_ends(rn(gen(99991), c.vocab_size, W), pair,
                          1 + rn(gen(99993), W, std=0.1),
                          lin(gen(99992), c.vocab_size, W))

    # ---------- forward ----------

    def embed_tokens(self, tokens: torch.Tensor, kv: Optional[KVCache] = None,
                     pos=0, lens=None, slots=None) -> torch.Tensor:
        """tokens [B] (one decode step) or [B, T] (a prompt portion whose
        first token sits at position ``pos``, an int or int32 [B]) -> fp32
        residual rows of the same leading shape. With a pair table the
        slot's last token is read from / written to ``kv.model_state``."""
        assert self.embed is not None, "this shard does not own the embedding"
        pe = self.cfg.pair_embedding
        if not pe:
            return torch.nn.functional.embedding(tokens, self.embed).to(
                torch.float32)
        assert kv is not None, "the pair table needs the slot's last token"
        tk = tokens.view(tokens.shape[0], -1)
        if not torch.is_tensor(pos):
            pos = torch.full((tk.shape[0],), int(pos), dtype=torch.int32,
                             device=tk.device)
        x = ops.pair_hash_embed(tk, self.embed, self.pair_table,
                                kv.model_state["prev_token"], pos,
                                int(pe["buckets"]), int(pe["mul_prev"]),
                                int(pe["mul_cur"]), lens, slots)
        return x.view(*tokens.shape, x.shape[-1])

    def _lightning(self, h, lw, m, kv, li, pos, T, lens, slots):
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        p = lw.qkv(h)                          # [q | k | v | g]
        o = ops.decay_scan(p, 0, H * d, 2 * H * d, lw.decay,
                           kv.state[li]["S"], pos, T, H, d, dv, lens, slots)
        og = ops.gated_group_rmsnorm(o, p, 2 * H * d + H * dv, lw.mix_norm,
                                     1, self.cfg.rms_eps, "sigmoid", False,
                                     self.wdtype)
        return lw.o(og)

    def _attention(self, h, lw, m, kv, li, pos, T, lens, slots):
        H, G, d = m["heads"], m["kv_heads"], m["dim"]
        q = ops.qknorm_half_append(lw.qkv(h), lw.q_norm, lw.k_norm,
                                   self.cfg.rms_eps, H, G, d, lw.rot_freq,
                                   kv.k[li], kv.v[li], pos, T, lens, slots)
        a = ops.attn_mod(q, kv.k[li], kv.v[li], pos, T, float(m["scale"]),
                         lens, slots, chunk=int(m["mask"]["size"]),
                         sig_bias=lw.score_bias)
        return lw.o(a)

    def _latent_attention(self, h, lw, m, kv, li, pos, T, lens, slots):
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        R, QR = m["kv_rank"], m["q_rank"]
        size = int(m["mask"]["size"])
        M = h.shape[0]
        p = lw.qkv(h)                                  # [dq | dkv | g]
        cq = ops.rmsnorm_rows(p[:, :QR], lw.q_a_norm, self.cfg.rms_eps,
                              self.wdtype)
        q = lw.q_b(cq)                                 # [M, H*d]
        if kv.v[li] is not None:
            a = self._expanded_attention(p, q, lw, m, kv, li, pos, T, lens,
                                         slots)
        else:
            ops.latent_append(p, QR, lw.kv_a_norm, self.cfg.rms_eps, R,
                              self._no_rot, kv.k[li], pos, T, lens, slots)
            # queries into the latent space, head by head
            qabs = torch.bmm(q.view(M, H, d).transpose(0, 1), lw.uk)
            qf = qabs.transpose(0, 1).reshape(M, H * R)
            ol = ops.attn_mod(qf, kv.k[li], None, pos, T, float(m["scale"]),
                              lens, slots, window=size, v_dim=R)
            a = torch.bmm(ol.view(M, H, R).transpose(0, 1), lw.uv) \
                .transpose(0, 1).reshape(M, H * dv)
        return lw.o(ops.mul_sigmoid(a, p, QR + R))

    def _expanded_attention(self, p, q, lw, m, kv, li, pos, T, lens, slots):
        """Latent rows too wide for one key row of the kernels: per-head keys
        and values are formed from the latent and cached. Padding and idle
        rows write where their slot's next real token is written later,
        before anything reads it."""
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        R, QR = m["kv_rank"], m["q_rank"]
        M = p.shape[0]
        B = M // T
        c = ops.rmsnorm_rows(p[:, QR:QR + R], lw.kv_a_norm, self.cfg.rms_eps,
                             self.wdtype)
        kvu = lw.kv_b(c)                               # [k (H*d) | v (H*dv)]
        smax = kv.k[li].shape[2]
        at = (pos.view(B, 1).long()
              + torch.arange(T, device=p.device)).clamp_(max=smax - 1)
        sl = (slots.long() if slots is not None
              else torch.arange(B, device=p.device)).view(B, 1)
        kv.k[li][sl, :, at] = kvu[:, :H * d].reshape(B, T, H, d)
        kv.v[li][sl, :, at] = kvu[:, H * d:].reshape(B, T, H, dv)
        return ops.attn_mod(q, kv.k[li], kv.v[li], pos, T, float(m["scale"]),
                            lens, slots, window=int(m["mask"]["size"]))

    def _window(self, x: torch.Tensor, layer_ids: Sequence[int], kv: KVCache,
                pos: torch.Tensor, T: int, lens, slots) -> None:
        """Run the layers of one window over x [B*T, W] fp32 (in place).
        Token (b, t) sits at position pos[b]+t of cache row slots[b]."""
        eps, wdt = self.cfg.rms_eps, self.wdtype
        mixers = {"lightning": self._lightning, "attention": self._attention,
                  "latent_attention": self._latent_attention}
        xc = None                  # x in the activation dtype, when current
        for lid in layer_ids:
            lw = self._layer(lid)
            s = self._spec(lid)
            li = kv.local[lid]
            if lw.conv_w is not None:
                h = ops.causal_conv_residual(x, lw.conv_w,
                                             kv.state[li]["conv"], pos, T,
                                             wdt, lens, slots)
            else:
                h = xc if xc is not None else x.to(wdt)
            a = mixers[s["type"]](h, lw, s["mixer"], kv, li, pos, T, lens,
                                  slots)
            ff = lw.gateup is not None
            # x += rmsnorm(a) * g1; the feed-forward reads x as it is then
            _, xc = ops.resid_branches_rmsnorm(
                x, a, lw.attn_norm, None, None, 1.0, None, None, eps, wdt,
                want_cast=ff or self.cfg.input_conv_taps == 0)
            if ff:
                f = lw.down(ops.swiglu(lw.gateup(xc)))
                _, xc = ops.resid_branches_rmsnorm(
                    x, f, lw.mlp_norm, None, None, 1.0, None, None, eps, wdt,
                    want_cast=self.cfg.input_conv_taps == 0)
            if self._obs_sync:
                self._profile_layer_sync(lid)

    def decode_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                      kv: KVCache) -> torch.Tensor:
        """One decode step. h [B, W] fp32, modified in place; kv.pos holds
        each row's write position; rows flagged in kv.idle keep their state
        (they run as padding)."""
        if layer_ids:
            self._window(h, layer_ids, kv, kv.pos, 1,
                         (~kv.idle).to(torch.int32), None)
        return h

    def prefill_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                       kv: KVCache, p0, lens: Optional[torch.Tensor] = None,
                       slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Prefill h [B, T, W] fp32 in place. ``p0``: first position, an int
        (every row) or an int32 tensor [B]. ``lens`` [B] int32: real token
        count per row (rows are right-padded to T; padding never reaches the
        cache or any state and its outputs are meaningless). ``slots`` [B]
        int32: cache row of each batch row (default: row b)."""
        if not layer_ids:
            return h
        B, T, W = h.shape
        if not torch.is_tensor(p0):
            p0 = torch.full((B,), int(p0), dtype=torch.int32,
                            device=h.device)
        self._window(h.view(B * T, W), layer_ids, kv, p0, T, lens, slots)
        return h

    def normalize_project(self, h: torch.Tensor) -> torch.Tensor:
        assert self.final_norm is not None and self.lm_head is not None
        y = ops.rmsnorm_rows(h, self.final_norm, self.cfg.rms_eps,
                             self.wdtype)
        return self.lm_head(y)

    def weight_bytes(self) -> int:
        """Bytes of every tensor and linear the resident layers hold (the
        layer kinds carry different sets of them)."""
        def size(v) -> int:
            if isinstance(v, Linear):
                return v.nbytes()
            if torch.is_tensor(v):
                return v.numel() * v.element_size()
            return 0
        return sum(size(v) for lw in self.layers.values()
                   for v in vars(lw).values())
