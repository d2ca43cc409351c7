"""Lurisun in the framework against the plain oracle (tests/lurisun_oracle.py).

Every test builds its own small configuration and random checkpoint, runs it
through the framework's ops / model / cache / executor (and, for generation,
the shard runtime's slot scheduler and the trace replay CLI) and compares with
the oracle, which is written from the equations, runs whole sequences without
any cache and shares no code with dnet_amd. Tests run on the CPU reference-op
path and, marked ``gpu``, on the HIP kernels.
"""
import copy
import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import lurisun_oracle as O
from dnet_amd.models import ModelConfig
from dnet_amd.models.config import lurisun_config
from dnet_amd.parallel.ring import RingExecutor

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
F64 = torch.float64
V = 83
W = 48


def base_cfg(**kw):
    """Five layers: linear attention, latent attention, chunked sigmoid
    attention, linear attention without a feed-forward, latent attention;
    windows and chunks far shorter than the test prompts."""
    args = dict(pattern="nlanl", layers=5, heads=6, kv_heads=2, dim=12,
                rot_dims=8, chunk=11, latent_heads=3, latent_dim=8,
                latent_vdim=10, kv_rank=20, q_rank=14, window=9, lin_heads=3,
                lin_dim=8, lin_vdim=12, decay=[0.5, 0.96875, 1.0], ff=40,
                taps=3, buckets=37, mul_prev=7, mul_cur=5, logit_scale=0.5,
                rot_base=300.0)
    args.update(kw)
    cfg = lurisun_config(W, V, **args)
    cfg["layers"] = copy.deepcopy(cfg["layers"])
    if len(cfg["layers"]) == 5:
        cfg["layers"][3]["mlp"] = None
    return cfg


def steady_cfg(dtype, **kw):
    """The base stack; for bfloat16 runs a shallower one (every layer of
    these tiny random models multiplies rounding noise)."""
    if dtype == "bfloat16":
        kw = dict(dict(pattern="nla", layers=3), **kw)
    return base_cfg(**kw)


def tokens(n, seed, vocab=V):
    return torch.randint(0, vocab, (n,),
                         generator=torch.Generator().manual_seed(seed))


def executor(cfg, sd, device, dtype="float32", slots=3, smax=160, **kw):
    mc = ModelConfig.from_hf(cfg)
    mc.compute_dtype = dtype
    ex = RingExecutor(mc, 0, 1, torch.device(device), mb_size=slots,
                      smax=smax, init_weights=False,
                      use_graphs=kw.pop("use_graphs", False), **kw)
    ex.model.load_state_dict(sd)
    return ex


def close(got, want, dtype="float32"):
    got, want = got.detach().cpu().to(F64), want.to(F64)
    scale = float(want.pow(2).mean().sqrt())
    # float32 is the sharp comparison. In bfloat16 these tiny random stacks
    # multiply rounding noise layer by layer and single positions stand out,
    # so the bound is on the root mean square, with a loose cap on any entry.
    if dtype == "float32":
        cap, mean = 2e-3, 6e-4
    else:
        cap, mean = 1.0, 0.15
    err = float((got - want).abs().max())
    assert err <= cap * scale, f"max err {err:.3g} vs scale {scale:.3g}"
    rms = float((got - want).pow(2).mean().sqrt())
    assert rms <= mean * scale, f"rms err {rms:.3g} vs {scale:.3g}"


def decode_step(ex, slot_tokens):
    """One slot-batch decode step {slot: token}; other rows sit it out."""
    tb = ex.tokbuf[0].cpu()
    for s, t in slot_tokens.items():
        tb[s] = int(t)
    ex.tokbuf[0].copy_(tb)
    idle = torch.ones(ex.mb_size, dtype=torch.bool)
    idle[list(slot_tokens)] = False
    idle = idle.to(ex.device)
    ex.slot_step_compute(park=idle)
    lg = ex.logits_buf[0].float().cpu().clone()
    ex.kvs[0].pos.add_((~idle).to(torch.int32))
    return lg


def oracle(toks, cfg, sd, **kw):
    return O.forward([int(t) for t in toks], sd, cfg, F64, **kw)


def sub64(sd, prefix):
    return {k: v.to(F64) for k, v in O.sub(sd, prefix).items()}


# ---------- configuration ----------

def test_config_registry_and_cache_layout():
    from dnet_amd.models import LurisunRingModel, get_ring_model
    cfg = base_cfg()
    mc = ModelConfig.from_hf(cfg)
    assert mc.model_type == "lurisun" and mc.num_layers == 5
    assert get_ring_model("lurisun") is LurisunRingModel
    assert mc.input_conv_taps == 3 and mc.logit_scale == 0.5
    assert mc.pair_embedding == {"buckets": 37, "mul_prev": 7, "mul_cur": 5}
    ex = executor(cfg, O.make_checkpoint(cfg, 1), "cpu")
    kv = ex.kvs[0]
    assert kv.k[0] is None and kv.state[0]["S"].shape == (3, 3, 8, 12)
    assert kv.k[1].shape == (3, 1, 160, 20) and kv.v[1] is None
    assert kv.k[2].shape == (3, 2, 160, 12) and kv.v[2].shape == kv.k[2].shape
    assert all(st["conv"].shape == (3, 2, W) for st in kv.state)
    assert kv.model_state["prev_token"].shape == (3,)
    for bad in (dict(pattern="x"), ):
        with pytest.raises(KeyError):
            base_cfg(**bad)
    broken = base_cfg()
    broken["layers"][2]["mixer"]["vdim"] = 10
    with pytest.raises(ValueError):
        ModelConfig.from_hf(broken)
    broken = base_cfg()
    broken["layers"][0]["mixer"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        ModelConfig.from_hf(broken)
    broken = base_cfg()
    broken["layers"][1]["type"] = "mystery"
    with pytest.raises(ValueError):
        ModelConfig.from_hf(broken)


# ---------- mechanisms alone ----------

def _one_layer(kind, **kw):
    return base_cfg(pattern=kind, layers=1, **kw)


def _mixer_alone(device, cfg, sd, u, T0, portion=None):
    """Run the layer's mixer on given inputs u [T, W] through the cache: the
    first T0 rows as one prompt portion (or portions), then row by row."""
    ex = executor(cfg, sd, device)
    m, kv = ex.model, ex.kvs[0]
    lw, spec = m.layers[0], m.cfg.layer_specs[0]
    fn = {"latent_attention": m._latent_attention,
          "attention": m._attention, "lightning": m._lightning}[spec["type"]]
    T = u.shape[0]
    slot = torch.tensor([2], dtype=torch.int32, device=device)
    steps, p = [], 0
    while p < T0:
        n = min(portion or T0, T0 - p)
        steps.append((p, n))
        p += n
    steps += [(t, 1) for t in range(T0, T)]
    outs = []
    for p0, n in steps:
        pos = torch.tensor([p0], dtype=torch.int32, device=device)
        ln = torch.tensor([n], dtype=torch.int32, device=device)
        x = u[p0:p0 + n].to(torch.float32).to(device).contiguous()
        outs.append(fn(x, lw, spec["mixer"], kv, 0, pos, n, ln, slot)
                    .float().cpu())
    return torch.cat(outs)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind,kw", [
    ("n", {}), ("n", dict(lin_heads=1, lin_dim=5, lin_vdim=3, decay=[0.75])),
    ("n", dict(lin_heads=2, lin_dim=32, lin_vdim=16, decay=[1.0, 0.25])),
    ("a", {}), ("a", dict(heads=1, kv_heads=1, dim=4, rot_dims=4, chunk=1)),
    ("a", dict(heads=4, kv_heads=4, dim=10, rot_dims=0, chunk=64)),
    ("a", dict(heads=4, kv_heads=1, dim=16, rot_dims=2, chunk=5)),
    ("l", {}), ("l", dict(latent_heads=1, latent_dim=4, latent_vdim=3,
                          kv_rank=7, q_rank=5, window=1)),
    ("l", dict(latent_heads=4, latent_dim=16, latent_vdim=8, kv_rank=40,
               q_rank=12, window=64)),
])
def test_each_mixer_alone(device, kind, kw):
    """A mixer on its own inputs: prompt portion, then token by token through
    the cache / state, equals the oracle's whole-sequence result."""
    cfg = _one_layer(kind, **kw)
    sd = O.make_checkpoint(cfg, 3)
    T = 41
    u = torch.randn(T, W, generator=torch.Generator().manual_seed(9))
    spec = cfg["layers"][0]
    want = O.MIXERS[spec["type"]](u.to(F64), sub64(sd, "l0.mix."),
                                  spec["mixer"], cfg["norm"]["eps"])
    for T0, portion in ((29, None), (30, 7), (2, 2)):
        got = _mixer_alone(device, cfg, sd, u, T0, portion)
        close(got, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind,key,size", [("l", "window", 9),
                                           ("l", "window", 2),
                                           ("a", "chunk", 11),
                                           ("a", "chunk", 3)])
def test_window_and_chunk_edges_are_sharp(device, kind, key, size):
    """Peaky scores (scaled query and key projections) make single keys carry
    the output, so a window or chunk that is one token off shows: the oracle
    with the size changed by one differs grossly from the true one, while the
    framework, in prompts, portions and decoding, equals the true one."""
    cfg = _one_layer(kind, **{key: size})
    sd = O.make_checkpoint(cfg, 5)
    for n in ("uq", "uk") if kind == "l" else ("q", "k"):
        sd["l0.mix." + n] = sd["l0.mix." + n] * 6.0
    if kind == "a":
        # strongly negative bias: only standout scores open a key
        sd["l0.mix.pb"] = sd["l0.mix.pb"] * 0 - 6.0
        sd["l0.mix.q.norm"] = sd["l0.mix.q.norm"] * 4.0
    T = 45
    u = torch.randn(T, W, generator=torch.Generator().manual_seed(10))
    spec = cfg["layers"][0]
    p64 = sub64(sd, "l0.mix.")
    want = O.MIXERS[spec["type"]](u.to(F64), p64, spec["mixer"],
                                  cfg["norm"]["eps"])
    scale = float(want.pow(2).mean().sqrt())
    for off in (-1, 1):
        if size + off < 1:
            continue
        m2 = copy.deepcopy(spec["mixer"])
        m2["mask"]["size"] = size + off
        other = O.MIXERS[spec["type"]](u.to(F64), p64, m2,
                                       cfg["norm"]["eps"])
        assert float((other - want).abs().max()) > 0.05 * scale
    for T0, portion in ((33, None), (32, 5), (2, 2)):
        close(_mixer_alone(device, cfg, sd, u, T0, portion), want)


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_through_the_recurrent_state(device):
    """A head without decay keeps a token from the far past at full weight:
    one standout key/value early in a long sequence, met by a matching query
    at the end, in a prompt, across portions and in decoding."""
    cfg = _one_layer("n", lin_heads=2, lin_dim=8, lin_vdim=8,
                     decay=[1.0, 0.5])
    sd = O.make_checkpoint(cfg, 6)
    T = 140
    u = torch.randn(T, W, generator=torch.Generator().manual_seed(11)) * 0.2
    u[T - 1] = u[3] * 4             # the query's direction, a modest key
    u[3] = u[3] * 30
    spec = cfg["layers"][0]
    p64 = sub64(sd, "l0.mix.")
    want = O.lightning_mixer(u.to(F64), p64, spec["mixer"],
                             cfg["norm"]["eps"])
    quiet = u.clone()
    quiet[3] = u[4]
    other = O.lightning_mixer(quiet.to(F64), p64, spec["mixer"],
                              cfg["norm"]["eps"])
    assert float((other[-1] - want[-1]).abs().max()) > 0.3
    for T0, portion in ((T, None), (T - 10, 33), (5, None)):
        close(_mixer_alone(device, cfg, sd, u, T0, portion), want)


@pytest.mark.parametrize("device", DEVICES)
def test_pair_embedding_and_input_convolution(device):
    """The hashed pair rows (first token: the extra row; later ones from the
    previous token, also across portions and decode steps) and the input
    convolution's tail, against the oracle's functions."""
    cfg = base_cfg()
    sd = O.make_checkpoint(cfg, 7)
    a = tokens(23, 12)
    want = O.embed(a.tolist(), {k: v.to(F64) for k, v in sd.items()}, cfg)
    rows = O.hashed_pair_rows(a.tolist(), 37, 7, 5)
    assert rows[0] == 37 and all(0 <= r < 37 for r in rows[1:])
    ex = executor(cfg, sd, device)
    m, kv = ex.model, ex.kvs[0]
    slot = torch.tensor([1], dtype=torch.int32, device=device)
    got, p = [], 0
    for n in (1, 6, 2, 9):
        pos = torch.tensor([p], dtype=torch.int32, device=device)
        ln = torch.tensor([n], dtype=torch.int32, device=device)
        got.append(m.embed_tokens(a[p:p + n].view(1, n).to(device), kv=kv,
                                  pos=pos, lens=ln, slots=slot)[0].cpu())
        p += n
    kv.pos[1] = p
    kv.idle.copy_(torch.tensor([True, False, True]))
    while p < 23:
        t = torch.zeros(3, dtype=torch.int64)
        t[1] = a[p]
        got.append(m.embed_tokens(t.to(device), kv=kv, pos=kv.pos,
                                  lens=(~kv.idle).to(torch.int32))[1:2].cpu())
        kv.pos[1] += 1
        p += 1
    close(torch.cat(got), want)
    # convolution: whole, in portions and token by token
    from dnet_amd import ops
    x = torch.randn(23, W, generator=torch.Generator().manual_seed(13))
    want = O.input_conv(x.to(F64), sd["l0.canon1"].to(F64))
    w = sd["l0.canon1"].float().to(device)
    st = torch.full((3, 2, W), 7.0, device=device)      # stale tail
    out, p = [], 0
    for n in (5, 1, 1, 2, 14):
        pos = torch.tensor([p], dtype=torch.int32, device=device)
        out.append(ops.causal_conv_residual(
            x[p:p + n].to(device).contiguous(), w, st, pos, n, torch.float32,
            torch.tensor([n], dtype=torch.int32, device=device), slot).cpu())
        p += n
    close(torch.cat(out), want)


# ---------- the whole model ----------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_logits_first_tokens_and_layers(device, dtype):
    cfg = steady_cfg(dtype)
    sd = O.make_checkpoint(cfg, 6, ff_gain=1.0 if dtype == "float32" else 0.3)
    a = tokens(37, 1)
    layers = []
    want = oracle(a, cfg, sd, layers_out=layers)
    ex = executor(cfg, sd, device, dtype)
    got = ex.prefill_slots([1], [a], want=[list(range(37))])[0]
    close(got, want, dtype)
    if dtype == "float32":
        # the residual after every layer
        m, kv = ex.model, ex.kvs[0]
        ln = torch.tensor([37], dtype=torch.int32, device=device)
        slot = torch.tensor([2], dtype=torch.int32, device=device)
        p0 = torch.zeros(1, dtype=torch.int32, device=device)
        h = m.embed_tokens(a.view(1, -1).to(device), kv=kv, pos=p0, lens=ln,
                           slots=slot).clone()
        for lid in range(len(cfg["layers"])):
            m.prefill_window(h, [lid], kv, 0, lens=ln, slots=slot)
            close(h[0], layers[lid])
    # single-token prompts and the very first positions
    one = ex.prefill_slots([0], [a[:1]])[0]
    close(one, want[:1], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_vs_token_by_token_and_long_decode(device):
    cfg = base_cfg()
    sd = O.make_checkpoint(cfg, 7)
    a = tokens(150, 2)
    want = oracle(a, cfg, sd)
    ex = executor(cfg, sd, device)
    got = [ex.prefill_slots([2], [a[:1]])[0].float().cpu()]
    for t in range(1, 150):                 # decode from the second token on
        got.append(decode_step(ex, {2: a[t]})[2:3])
    close(torch.cat(got), want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("chunk", [2, 3, 16, 33])
def test_portions(device, chunk):
    """A prompt cut into portions (executor chunking and continued requests)
    gives the logits of the whole prompt."""
    cfg = base_cfg()
    sd = O.make_checkpoint(cfg, 8)
    a = tokens(45, 3)
    want = oracle(a, cfg, sd)
    ex = executor(cfg, sd, device)
    got = ex.prefill_slots([1], [a], want=[list(range(45))], chunk=chunk)[0]
    close(got, want)
    # the same through continued calls of unequal size
    rows, p = [], 0
    for n in (chunk, 2, 45):
        n = min(n, 45 - p)
        if n <= 0:
            break
        rows.append(ex.prefill_slots([0], [a[p:p + n]],
                                     want=[list(range(n))], start=[p])[0])
        p += n
    close(torch.cat(rows), want[:p])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_equals_each_alone(device, dtype):
    cfg = steady_cfg(dtype)
    sd = O.make_checkpoint(cfg, 9, ff_gain=1.0 if dtype == "float32" else 0.3)
    a, b, c = tokens(40, 4), tokens(5, 5), tokens(1, 6)
    if dtype == "float32":
        wa, wb, wc = (oracle(t, cfg, sd) for t in (a, b, c))
    else:
        # each request alone through the framework, whole and in one step
        wa, wb, wc = (executor(cfg, sd, device, dtype).prefill_slots(
            [0], [t], want=[list(range(len(t)))])[0].float().cpu()
            for t in (a, b, c))
    ex = executor(cfg, sd, device, dtype, slots=4)
    got = ex.prefill_slots([3, 1, 0], [a[:30], b[:3], c],
                           want=[[0, 29], [2], [0]])
    close(got[0], wa[[0, 29]], dtype)
    close(got[1], wb[2:3], dtype)
    close(got[2], wc, dtype)
    for i in range(2):                      # decoded together
        lg = decode_step(ex, {3: a[30 + i], 1: b[3 + i]})
        close(lg[3:4], wa[30 + i].view(1, -1), dtype)
        close(lg[1:2], wb[3 + i].view(1, -1), dtype)
    for i in range(32, 40):                 # the shorter request has ended
        lg = decode_step(ex, {3: a[i]})
        close(lg[3:4], wa[i].view(1, -1), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_slot_freed_and_used_again(device):
    """A slot that held a long request is taken by a new one without any
    reset: cache rows, recurrent states, convolution tails and the last token
    of the old request do not leak."""
    cfg = base_cfg()
    sd = O.make_checkpoint(cfg, 10)
    a, b = tokens(60, 7), tokens(20, 8)
    ex = executor(cfg, sd, device, slots=2)
    ex.prefill_slots([1], [a[:50]])
    for t in range(50, 60):
        decode_step(ex, {1: a[t]})
    wb = oracle(b, cfg, sd)
    ex.kvs[0].pos[1] = 0
    got = ex.prefill_slots([1], [b[:12]], want=[[0, 5, 11]])[0]
    close(got, wb[[0, 5, 11]])
    for t in range(12, 20):
        close(decode_step(ex, {1: b[t]})[1:2], wb[t].view(1, -1))


OTHER = [
    # no convolution, no pair table, no rotation, no logit factor; one head
    dict(pattern="anl", layers=3, taps=0, buckets=0, rot_dims=0,
         logit_scale=1.0, heads=1, kv_heads=1, dim=6, chunk=4,
         latent_heads=1, latent_dim=5, latent_vdim=5, kv_rank=5, q_rank=5,
         window=3, lin_heads=1, lin_dim=6, lin_vdim=6, decay=[0.875]),
    # every head with its own key head, full rotation, two taps, window and
    # chunk longer than the prompts, a single bucket
    dict(pattern="la", layers=4, taps=2, buckets=1, heads=4, kv_heads=4,
         dim=10, rot_dims=10, chunk=200, window=200, latent_heads=5,
         latent_dim=6, latent_vdim=14, kv_rank=9, q_rank=30, ff=24),
    # many taps, many query heads on one key head, value size above the key
    # size in the linear layer, windows of one token
    dict(pattern="nnal", layers=4, taps=6, heads=8, kv_heads=1, dim=8,
         rot_dims=4, chunk=1, window=1, lin_heads=2, lin_dim=4, lin_vdim=20,
         decay=[0.99, 0.3], mul_prev=1, mul_cur=1, buckets=1000),
    # a one-tap convolution (no tail), odd width-independent sizes, sixteen
    # query heads on one latent (the grouped-heads decode kernel in bf16)
    dict(pattern="lna", layers=3, taps=1, latent_heads=16, latent_dim=6,
         latent_vdim=5, kv_rank=24, q_rank=11, window=7, heads=3, kv_heads=3,
         dim=14, rot_dims=6, chunk=13, lin_heads=5, lin_dim=7, lin_vdim=9,
         decay=[0.9, 0.8, 0.7, 0.6, 1.0], ff=33),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", OTHER)
def test_other_sizes(device, kw):
    cfg = base_cfg(**kw)
    sd = O.make_checkpoint(cfg, 11)
    a, b = tokens(33, 9), tokens(7, 10)
    wa, wb = oracle(a, cfg, sd), oracle(b, cfg, sd)
    ex = executor(cfg, sd, device, slots=2)
    got = ex.prefill_slots([0, 1], [a[:25], b[:4]],
                           want=[list(range(25)), [3]], chunk=9)
    close(got[0], wa[:25])
    close(got[1], wb[3:4])
    for i in range(3):
        lg = decode_step(ex, {0: a[25 + i], 1: b[4 + i]})
        close(lg[0:1], wa[25 + i].view(1, -1))
        close(lg[1:2], wb[4 + i].view(1, -1))


@pytest.mark.parametrize("device", DEVICES)
def test_latent_wider_than_the_kernels_key_row(device, monkeypatch):
    """When the latent does not fit one key row of the attention kernels the
    layer caches per-head keys and values: same logits, through ragged
    prompts, portions, batched decode with an idle row."""
    from dnet_amd.models import LurisunRingModel
    monkeypatch.setattr(LurisunRingModel, "MAX_KEY_ROW", 16)
    cfg = base_cfg()                        # latent 20 > 16
    sd = O.make_checkpoint(cfg, 13)
    a, b = tokens(33, 11), tokens(6, 12)
    wa, wb = oracle(a, cfg, sd), oracle(b, cfg, sd)
    ex = executor(cfg, sd, device, slots=3)
    assert ex.kvs[0].v[1] is not None and ex.kvs[0].k[1].shape[1] == 3
    got = ex.prefill_slots([2, 0], [a[:25], b[:3]],
                           want=[list(range(25)), [2]], chunk=7)
    close(got[0], wa[:25])
    close(got[1], wb[2:3])
    for i in range(3):
        lg = decode_step(ex, {2: a[25 + i], 0: b[3 + i]})
        close(lg[2:3], wa[25 + i].view(1, -1))
        close(lg[0:1], wb[3 + i].view(1, -1))
    for i in range(28, 33):
        close(decode_step(ex, {2: a[i]})[2:3], wa[i].view(1, -1))
    with pytest.raises(NotImplementedError):
        monkeypatch.setattr(LurisunRingModel, "MAX_KEY_ROW", 4)
        executor(cfg, sd, device)


@pytest.mark.gpu
def test_decode_graph_replays_match_eager():
    """Captured decode steps, replayed with eager prefills and host syncs in
    between, equal the eager steps every time (warm-up runs of the capture
    must not advance any slot's state)."""
    cfg = steady_cfg("bfloat16")
    sd = O.make_checkpoint(cfg, 12, ff_gain=0.3)
    a, b = tokens(40, 31), tokens(30, 32)
    runs = []
    for graphs in (False, True):
        ex = executor(cfg, sd, "cuda:0", "bfloat16", use_graphs=graphs)
        out = [ex.prefill_slots([1], [a[:30]], want=[[0, 29]])[0].float().cpu()]
        for t in range(30, 35):
            out.append(decode_step(ex, {1: a[t]})[1:2])
        out.append(ex.prefill_slots([2], [b[:25]],
                                    want=[[3, 24]])[0].float().cpu())
        for t in range(5):
            lg = decode_step(ex, {1: a[35 + t], 2: b[25 + t]})
            out.append(lg[1:3])
            torch.cuda.synchronize()
        runs.append(torch.cat(out))
    torch.testing.assert_close(runs[1], runs[0], atol=2e-2, rtol=2e-2)


# ---------- generation through the scheduler, trace replay ----------

def write_checkpoint(path: Path, cfg, sd):
    from safetensors.torch import save_file
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()},
              str(path / "model.safetensors"))


def oracle_greedy(prompt, n, cfg, sd):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(oracle(seq, cfg, sd)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_slot_scheduler(tmp_path, device,
                                                  monkeypatch):
    """Requests queued at the shard runtime are admitted into slots (more
    requests than slots), prefilled, decoded as one batch with idle rows in
    it and sampled greedily; every token equals the oracle's argmax."""
    if device == "cpu":
        monkeypatch.setattr(torch.cuda, "is_available", lambda: False)
    from dnet_amd.core.types import ShardLoadModelRequest
    from dnet_amd.shard.runtime import ShardRuntime
    cfg = base_cfg()
    cfg["vocab"] = 59
    sd = O.make_checkpoint(cfg, 15)
    write_checkpoint(tmp_path / "m", cfg, sd)
    emitted: dict = {}

    class Cap:
        def send(self, frame):
            emitted.setdefault(frame["nonce"], []).append(
                (frame["token_id"], frame["finished"]))

        def close(self):
            pass

    rt = ShardRuntime("probe")
    monkeypatch.setattr(rt.settings.storage, "repack_on_load", False)
    rt._load(ShardLoadModelRequest(
        model_path=str(tmp_path / "m"), total_layers=5,
        layers=list(range(5)), max_batch=2, max_seq=96, dtype="float32"))
    assert (rt.executor.device.type == "cuda") == device.startswith("cuda")
    rt._callback = Cap()
    prompts = {"a": tokens(9, 1, 59), "b": tokens(2, 2, 59),
               "c": tokens(23, 3, 59)}
    n_new = {"a": 6, "b": 9, "c": 4}
    for name in ("a", "b", "c"):            # c waits for a slot to free up
        rt.infer_q.put({"nonce": name, "prompt_len": len(prompts[name]),
                        "tokens": prompts[name].to(torch.int32).numpy()
                        .tobytes(), "max_tokens": n_new[name],
                        "stop_ids": [], "params": {}})
    for _ in range(60):
        rt._slots_tick()
        if all(emitted.get(k) and emitted[k][-1][1] for k in prompts):
            break
    for name, p in prompts.items():
        got = [t for t, _ in emitted[name]]
        assert got == oracle_greedy(p.tolist(), n_new[name], cfg, sd), name
    rt._unload()


def test_repacked_weights_load(tmp_path, monkeypatch):
    """The per-layer repacked weight cache holds every tensor of the family
    (the pair table with the embedding): a second load reads it and gives the
    same logits."""
    monkeypatch.setattr(torch.cuda, "is_available", lambda: False)
    monkeypatch.setenv("DNET_REPACK_DIR", str(tmp_path / "repack"))
    from dnet_amd.core.types import ShardLoadModelRequest
    from dnet_amd.shard.runtime import ShardRuntime
    cfg = base_cfg()
    sd = O.make_checkpoint(cfg, 17)
    write_checkpoint(tmp_path / "m", cfg, sd)
    a = tokens(12, 5)
    outs = []
    for _ in range(2):
        rt = ShardRuntime("probe")
        rt._load(ShardLoadModelRequest(
            model_path=str(tmp_path / "m"), total_layers=5,
            layers=list(range(5)), max_batch=2, max_seq=64, dtype="float32"))
        outs.append(rt.executor.prefill_slots([0], [a])[0].float().cpu())
        rt._unload()
    close(outs[0], oracle(a, cfg, sd)[-1:])
    assert torch.equal(outs[0], outs[1])


@pytest.mark.gpu
def test_trace_replay_cli_gpu(tmp_path):
    test_trace_replay_cli(tmp_path, "bfloat16")
    test_trace_replay_cli(tmp_path / "f", "float32")


def test_trace_replay_cli(tmp_path, dtype="float32"):
    """bin/trace_run on a tiny checkpoint: a prompt batch of unequal
    requests (more than the initial slot count), decode steps together, a
    request that sits steps out, requests that end early, a slot used
    again by a new request."""
    cfg = steady_cfg(dtype)
    cfg["vocab"] = 53
    sd = O.make_checkpoint(cfg, 16,
                           ff_gain=1.0 if dtype == "float32" else 0.3)
    write_checkpoint(tmp_path / "m", cfg, sd)
    a, b = tokens(14, 1, 53).tolist(), tokens(4, 2, 53).tolist()
    c, d = tokens(12, 3, 53).tolist(), tokens(6, 4, 53).tolist()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:11], "want": [0, 10]},
                                {"id": "b", "tokens": b[:2], "want": []},
                                {"id": "c", "tokens": c[:10], "want": [9]}],
         "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[11:12], "want": [0]},
                                {"id": "b", "tokens": b[2:3], "want": [0]}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[12:13], "want": []},
                                {"id": "b", "tokens": b[3:4], "want": [0]}],
         "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[13:14], "want": [0]}],
         "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": c[10:11], "want": [0]}],
         "end": []},
        {"step": 5, "entries": [{"id": "d", "tokens": d[:5], "want": [4]}],
         "end": []},
        {"step": 6, "entries": [{"id": "c", "tokens": c[11:12], "want": [0]},
                                {"id": "d", "tokens": d[5:6], "want": [0]}],
         "end": ["c", "d"]},
    ]
    root = Path(__file__).resolve().parents[1]
    import os

    import numpy as np

    def replay(out, hide_gpu=False):
        env = dict(os.environ)
        if hide_gpu:
            env["HIP_VISIBLE_DEVICES"] = env["CUDA_VISIBLE_DEVICES"] = ""
        r = subprocess.run(
            [sys.executable, str(root / "bin" / "trace_run"), "--model",
             str(tmp_path / "m"), "--dtype", dtype, "--out", str(out),
             "--max-tokens", "48", "--max-batch", "2"],
            input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
            capture_output=True, timeout=600, env=env)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] \
            == [f"done {i}" for i in range(7)]
        return [torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")
                                 .reshape(-1, 53)) for i in range(7)]

    got = replay(tmp_path / "out")
    if dtype == "float32":
        w = {n: oracle(t, cfg, sd) for n, t in
             (("a", a), ("b", b), ("c", c), ("d", d))}
        want = [torch.cat([w["a"][[0, 10]], w["c"][9:10]]),
                torch.stack([w["a"][11], w["b"][2]]), w["b"][3:4],
                w["a"][13:14], w["c"][10:11], w["d"][4:5],
                torch.stack([w["c"][11], w["d"][5]])]
    else:
        # bfloat16: the same replay on the CPU reference ops
        want = replay(tmp_path / "ref", hide_gpu=True)
    for g, x in zip(got, want):
        close(g, x, dtype)


# ---------- pipeline stages (gloo, two processes) ----------

def _ring_run(rank, world):
    cfg = base_cfg()
    mc = ModelConfig.from_hf(cfg)
    mc.compute_dtype = "float32"
    ex = RingExecutor(mc, rank, world, "cpu", mb_count=1, mb_size=2, smax=64,
                      seed=7, use_graphs=False)
    g = torch.Generator().manual_seed(21)
    first = ex.prefill(torch.randint(0, V, (1, 2, 13), generator=g), chunk=5)
    steps = []
    ex.decode_stream(6, on_token=lambda s, t, last: steps.append(t.clone()))
    if rank:
        return None
    return torch.cat([first.view(2, 1)] + [t.view(2, 1) for t in steps], -1)


def _ring_rank_main(rank, world, port, q):
    import os
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port),
                      LOCAL_RANK=str(rank))
    import torch.distributed as dist
    dist.init_process_group("gloo", rank=rank, world_size=world)
    out = _ring_run(rank, world)
    if rank == 0:
        q.put(out)
    dist.destroy_process_group()


@pytest.mark.timeout(360)
def test_two_stage_ring_matches_single():
    """Layers split over two pipeline stages (the embedding's state lives on
    the first, every later layer's on its own stage): the fp32 residual rides
    the ring hops and the generated tokens equal the single-stage run."""
    import multiprocessing as mp
    import socket
    ctx = mp.get_context("spawn")

    def run(world):
        s = socket.socket()
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
        s.close()
        q = ctx.Queue()
        procs = [ctx.Process(target=_ring_rank_main, args=(r, world, port, q))
                 for r in range(world)]
        for p in procs:
            p.start()
        out = q.get(timeout=200)
        for p in procs:
            p.join(timeout=60)
            assert p.exitcode == 0
        return out

    single, out = run(1), run(2)
    assert single.shape[0] == 2 and single.shape[1] >= 6
    assert torch.equal(out, single)


def test_synthetic_preset_runs():
    """The preset builds with seeded random weights and generates the same
    tokens whatever the slot a prompt sits in."""
    from dnet_amd.models import PRESETS
    mc = ModelConfig.from_hf(dict(PRESETS["lurisun-tiny"]))
    ex = RingExecutor(mc, 0, 1, "cpu", mb_size=2, smax=96, seed=3,
                      use_graphs=False)
    toks = torch.randint(0, 256, (1, 2, 30),
                         generator=torch.Generator().manual_seed(1))
    toks[0, 1] = toks[0, 0]
    first = ex.prefill(toks)
    gen = ex.decode_rounds(6)
    assert torch.equal(first[0, 0], first[0, 1])
    assert torch.equal(gen[0, 0], gen[0, 1])
    with pytest.raises(NotImplementedError):
        RingExecutor(mc, 0, 1, "cpu", mb_size=1, smax=32, residency=2,
                     use_graphs=False)
