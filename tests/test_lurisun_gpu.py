"""GPU numerics of the Lurisun kernels (hashed pair embedding, residual
convolution, constant-decay linear attention, whole-projection q/k norm with
half-split rotation, chunked visibility and sigmoid weights in attn_mod,
sigmoid gate, gated feed-forward activation) against their plain-PyTorch
references (dnet_amd.ops.reference), in bf16 and fp32, with ragged batches,
slot indirection, continued states and sizes that are not multiples of the
kernels' tiles; and the whole model on the GPU (prefill, graph-captured
decode) against the same model on the CPU."""
import pytest
import torch

import dnet_amd.ops as ops
from dnet_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTS = [torch.bfloat16, torch.float32]


def _tol(dt):
    return dict(atol=3e-2, rtol=3e-2) if dt == torch.bfloat16 \
        else dict(atol=3e-5, rtol=3e-5)


def _i32(v):
    return torch.tensor(v, dtype=torch.int32)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("W,buckets", [(64, 127), (36, 5), (1030, 2003)])
def test_pair_hash_embed(dt, W, buckets):
    torch.manual_seed(W)
    V, T, B, Bc = 97, 9, 3, 4
    emb = torch.randn(V, W, device=DEV).to(dt)
    tab = torch.randn(buckets + 1, W, device=DEV).to(dt)
    tok = torch.randint(0, V, (B, T), device=DEV)
    pos, lens, slots = _i32([0, 5, 7]), _i32([9, 2, 0]), _i32([3, 0, 1])
    prev = torch.randint(0, V, (Bc,), dtype=torch.int32, device=DEV)
    pr = prev.cpu().clone()
    out = ops.pair_hash_embed(tok, emb, tab, prev, pos.to(DEV), buckets, 53,
                              29, lens.to(DEV), slots.to(DEV))
    want = ref.pair_hash_embed(tok.cpu(), emb.cpu(), tab.cpu(), pr, pos,
                               buckets, 53, 29, lens, slots)
    for b in range(B):
        n = int(lens[b])
        torch.testing.assert_close(out[b, :n].cpu(), want[b, :n],
                                   atol=1e-6, rtol=1e-6)
    assert torch.equal(prev.cpu(), pr)
    # decode steps read the state the portion left
    for step in range(3):
        t1 = torch.randint(0, V, (B, 1), device=DEV)
        p1 = (pos + lens + step).to(torch.int32)
        idle = _i32([1, 1, 0])
        out = ops.pair_hash_embed(t1, emb, tab, prev, p1.to(DEV), buckets,
                                  53, 29, idle.to(DEV), slots.to(DEV))
        want = ref.pair_hash_embed(t1.cpu(), emb.cpu(), tab.cpu(), pr, p1,
                                   buckets, 53, 29, idle, slots)
        torch.testing.assert_close(out[:2].cpu(), want[:2], atol=1e-6,
                                   rtol=1e-6)
        assert torch.equal(prev.cpu(), pr)


@pytest.mark.parametrize("odt", DTS)
@pytest.mark.parametrize("C,taps", [(64, 3), (36, 4), (1030, 2), (7, 1),
                                    (130, 8), (50, 16)])
def test_causal_conv_residual(odt, C, taps):
    torch.manual_seed(C + taps)
    T, B, Bc = 37, 3, 4
    x = torch.randn(B * T, C, device=DEV)
    w = torch.randn(C, taps, device=DEV) * 0.5
    pos, lens, slots = _i32([40, 0, 1]), _i32([37, 2, 0]), _i32([3, 0, 1])
    st = torch.randn(Bc, taps - 1, C, device=DEV)
    sr = st.cpu().clone()
    y = ops.causal_conv_residual(x, w, st, pos.to(DEV), T, odt, lens.to(DEV),
                                 slots.to(DEV))
    want = ref.causal_conv_residual(x.cpu(), w.cpu(), sr, pos, T, odt, lens,
                                    slots)
    torch.testing.assert_close(y.cpu().float(), want.float(), **_tol(odt))
    torch.testing.assert_close(st.cpu(), sr, atol=1e-6, rtol=1e-6)
    for step in range(taps + 1):
        x1 = torch.randn(B, C, device=DEV)
        p1 = (pos + lens + step).to(torch.int32)
        idle = _i32([1, 1, 0])
        y = ops.causal_conv_residual(x1, w, st, p1.to(DEV), 1, odt,
                                     idle.to(DEV), slots.to(DEV))
        want = ref.causal_conv_residual(x1.cpu(), w.cpu(), sr, p1, 1, odt,
                                        idle, slots)
        torch.testing.assert_close(y.cpu().float(), want.float(), **_tol(odt))
    torch.testing.assert_close(st.cpu(), sr, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,d,dv", [(2, 32, 96), (4, 16, 16), (3, 24, 40),
                                    (2, 128, 72), (2, 5, 3), (1, 96, 300)])
def test_decay_scan(dt, H, d, dv):
    torch.manual_seed(H * 100 + d)
    T, B, Bc = 37, 3, 4
    ld = 5 + 2 * H * d + H * dv + 3
    src = torch.randn(B * T, ld, device=DEV).to(dt)
    decay = torch.rand(H, device=DEV) * 0.5 + 0.5
    decay[0] = 0.999
    pos, lens, slots = _i32([40, 0, 7]), _i32([37, 2, 0]), _i32([3, 0, 1])
    st = torch.randn(Bc, H, d, dv, device=DEV)
    sr = st.cpu().clone()
    q0, k0, v0 = 5, 5 + H * d, 5 + 2 * H * d
    o = ops.decay_scan(src, q0, k0, v0, decay, st, pos.to(DEV), T, H, d, dv,
                       lens.to(DEV), slots.to(DEV))
    want = ref.decay_scan(src.cpu(), q0, k0, v0, decay.cpu(), sr, pos, T, H,
                          d, dv, lens, slots)
    torch.testing.assert_close(o.cpu(), want, atol=3e-4, rtol=3e-4)
    torch.testing.assert_close(st.cpu(), sr, atol=3e-4, rtol=3e-4)
    for step in range(3):
        s1 = torch.randn(B, ld, device=DEV).to(dt)
        p1 = (pos + lens + step).to(torch.int32)
        idle = _i32([1, 1, 0])
        o = ops.decay_scan(s1, q0, k0, v0, decay, st, p1.to(DEV), 1, H, d, dv,
                           idle.to(DEV), slots.to(DEV))
        want = ref.decay_scan(s1.cpu(), q0, k0, v0, decay.cpu(), sr, p1, 1, H,
                              d, dv, idle, slots)
        torch.testing.assert_close(o.cpu(), want, atol=3e-4, rtol=3e-4)
    torch.testing.assert_close(st.cpu(), sr, atol=3e-4, rtol=3e-4)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("nq,nkv,d,rot", [(4, 2, 96, 48), (6, 3, 40, 40),
                                          (2, 2, 17, 4), (8, 1, 64, 0),
                                          (3, 3, 256, 256)])
def test_qknorm_half_append_and_sigmoid_chunks(dt, nq, nkv, d, rot):
    torch.manual_seed(nq * 10 + d)
    T, B, Bc, S = 45, 3, 4, 128
    qk = torch.randn(B * T, (nq + nkv) * d, device=DEV).to(dt)
    qw = 1 + 0.1 * torch.randn(nq * d, device=DEV)
    kw = 1 + 0.1 * torch.randn(nkv * d, device=DEV)
    freq = None
    if rot:
        freq = (50000.0 ** (-2.0 * torch.arange(rot // 2) / rot)).float() \
            .to(DEV)
    pos, lens, slots = _i32([60, 0, 7]), _i32([45, 2, 0]), _i32([3, 0, 1])
    kc = torch.randn(Bc, nkv, S, d, device=DEV).to(dt)
    vc = torch.randn(Bc, nkv, S, d, device=DEV).to(dt)
    kr, vr = kc.cpu().clone(), vc.cpu().clone()
    q = ops.qknorm_half_append(qk, qw, kw, 1e-5, nq, nkv, d, freq, kc, vc,
                               pos.to(DEV), T, lens.to(DEV), slots.to(DEV))
    qr = ref.qknorm_half_append(qk.cpu(), qw.cpu(), kw.cpu(), 1e-5, nq, nkv,
                                d, None if freq is None else freq.cpu(), kr,
                                vr, pos, T, lens, slots)
    torch.testing.assert_close(q.cpu().float(), qr.float(), **_tol(dt))
    torch.testing.assert_close(kc.cpu().float(), kr.float(), **_tol(dt))
    assert torch.equal(vc.cpu(), vr)
    # chunked sigmoid attention: prompt (matrix-core kernel in bf16 when the
    # head size allows) and one decode step, chunk edges inside the range
    bias = torch.randn(nq, device=DEV) - 3.0
    for chunk in (16, 37):
        for Tq, ln in ((T, lens), (1, _i32([1, 1, 0]))):
            qq = q[:B * Tq].contiguous()
            out = ops.attn_mod(qq, kc, vc, pos.to(DEV), Tq, d ** -0.5,
                               ln.to(DEV), slots.to(DEV), chunk=chunk,
                               sig_bias=bias)
            want = ref.attn_mod(qq.cpu(), kc.cpu(), vc.cpu(), pos, Tq,
                                d ** -0.5, ln, slots, chunk=chunk,
                                sig_bias=bias.cpu())
            for b in range(B):
                n = int(ln[b])
                torch.testing.assert_close(
                    out[b * Tq:b * Tq + n].cpu().float(),
                    want[b * Tq:b * Tq + n].float(),
                    **(dict(atol=6e-2, rtol=4e-2) if dt == torch.bfloat16
                       else dict(atol=1e-4, rtol=1e-4)))


@pytest.mark.parametrize("dt", DTS)
def test_sigmoid_chunks_split_decode(dt):
    """Long cache, few rows: the decode kernel splits the keys and the
    partial sums add up without a normalization."""
    torch.manual_seed(5)
    B, H, G, d, S = 2, 4, 2, 64, 4096
    kc = torch.randn(B, G, S, d, device=DEV).to(dt)
    vc = torch.randn(B, G, S, d, device=DEV).to(dt)
    q = torch.randn(B, H * d, device=DEV).to(dt)
    bias = torch.randn(H, device=DEV) - 4.0
    pos = _i32([3000, 2047])
    for chunk in (0, 2048, 700):
        out = ops.attn_mod(q, kc, vc, pos.to(DEV), 1, 0.1, None, None,
                           chunk=chunk, sig_bias=bias)
        want = ref.attn_mod(q.cpu(), kc.cpu(), vc.cpu(), pos, 1, 0.1, None,
                            None, chunk=chunk, sig_bias=bias.cpu())
        torch.testing.assert_close(
            out.cpu().float(), want.float(),
            **(dict(atol=0.15, rtol=4e-2) if dt == torch.bfloat16
               else dict(atol=2e-3, rtol=1e-4)))


@pytest.mark.parametrize("dt", DTS)
def test_softmax_chunks(dt):
    """Chunked visibility with the ordinary softmax (the mask alone)."""
    torch.manual_seed(6)
    T, B, H, G, d, S = 50, 2, 4, 2, 32, 128
    kc = torch.randn(B, G, S, d, device=DEV).to(dt)
    vc = torch.randn(B, G, S, d, device=DEV).to(dt)
    q = torch.randn(B * T, H * d, device=DEV).to(dt)
    pos, lens = _i32([30, 0]), _i32([50, 33])
    out = ops.attn_mod(q, kc, vc, pos.to(DEV), T, 0.2, lens.to(DEV), None,
                       chunk=24)
    want = ref.attn_mod(q.cpu(), kc.cpu(), vc.cpu(), pos, T, 0.2, lens, None,
                        chunk=24)
    for b in range(B):
        n = int(lens[b])
        torch.testing.assert_close(out[b * T:b * T + n].cpu().float(),
                                   want[b * T:b * T + n].float(), **_tol(dt))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("N", [64, 36, 1030, 7])
def test_mul_sigmoid_and_gated_activation(dt, N):
    torch.manual_seed(N)
    M = 5
    a = torch.randn(M, N, device=DEV).to(dt)
    g = torch.randn(M, N + 9, device=DEV).to(dt)
    y = ops.mul_sigmoid(a, g, 4)
    torch.testing.assert_close(y.cpu().float(),
                               ref.mul_sigmoid(a.cpu(), g.cpu(), 4).float(),
                               **_tol(dt))
    gu = torch.randn(M, 2 * N, device=DEV).to(dt)
    torch.testing.assert_close(ops.swiglu(gu).cpu().float(),
                               ref.swiglu(gu.cpu()).float(), **_tol(dt))


def _executors(dtype, kw, mb=4, smax=256, width=96, vocab=200):
    from dnet_amd.models import ModelConfig
    from dnet_amd.models.config import lurisun_config
    from dnet_amd.parallel.ring import RingExecutor
    from lurisun_oracle import make_checkpoint
    # bfloat16: the two paths round differently and every layer of a random
    # stack multiplies that noise, so the bfloat16 stack is shallow
    hf = lurisun_config(width, vocab, "nla",
                        layers=6 if dtype == "float32" else 3, **kw)
    sd = make_checkpoint(hf, seed=11)
    out = []
    for dev, graphs in (("cpu", False), (DEV, True)):
        cfg = ModelConfig.from_hf(hf)
        cfg.compute_dtype = dtype
        ex = RingExecutor(cfg, 0, 1, torch.device(dev), mb_size=mb,
                          smax=smax, use_graphs=graphs, init_weights=False)
        ex.model.load_state_dict(sd)
        out.append(ex)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kw", [
    {}, dict(taps=0, buckets=0, rot_dims=0),
    dict(heads=6, kv_heads=1, dim=24, rot_dims=24, latent_heads=3,
         latent_dim=10, latent_vdim=12, kv_rank=20, q_rank=28, lin_heads=2,
         lin_dim=20, lin_vdim=12, taps=2, chunk=7, window=5, ff=100)])
def test_model_gpu_equals_cpu(dtype, kw):
    """Ragged prompt batch into scattered slots, a second portion, then
    graph-captured decode steps with an idle row: the GPU kernels against the
    CPU reference ops under the same executor."""
    torch.manual_seed(0)
    prompts = [torch.randint(0, 200, (n,)) for n in (41, 3, 17)]
    more = [torch.randint(0, 200, (n,)) for n in (2, 9, 1)]
    steps = [torch.randint(0, 200, (4,)) for _ in range(5)]
    outs = []
    for ex in _executors(dtype, kw):
        rows = [r.float().cpu() for r in ex.prefill_slots(
            [2, 0, 3], prompts, want=[list(range(41)), [2], [0, 16]])]
        rows += [r.float().cpu() for r in ex.prefill_slots(
            [2, 0, 3], more, want=[[0, 1], [8], [0]], start=[41, 3, 17])]
        for i, t in enumerate(steps):
            ex.tokbuf[0].copy_(t)
            idle = torch.tensor([False, True, False, i % 2 == 1])
            ex.slot_step_compute(park=idle.to(ex.device))
            live = [j for j in range(4) if not bool(idle[j]) and j != 1]
            rows.append(ex.logits_buf[0].float().cpu()[live].clone())
            ex.kvs[0].pos.add_((~idle).to(torch.int32).to(ex.device))
        outs.append(torch.cat(rows))
    cpu, gpu = outs
    rel = float((gpu - cpu).pow(2).mean().sqrt() / cpu.pow(2).mean().sqrt())
    assert rel < (2e-4 if dtype == "float32" else 0.1), rel
    worst = float((gpu - cpu).abs().max() / cpu.abs().max())
    assert worst < (1e-3 if dtype == "float32" else 0.3), worst


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_odd_sizes_gpu_matches_cpu(dtype):
    """Sizes that are multiples of nothing (width, vocabulary, ranks, head
    sizes, feed-forward width) and sixteen heads on one latent: every
    kernel's unvectorized path and the linears' fallbacks, prompt and
    decode."""
    kw = dict(heads=3, kv_heads=1, dim=13, rot_dims=6, chunk=9,
              latent_heads=16, latent_dim=7, latent_vdim=5, kv_rank=21,
              q_rank=11, window=6, lin_heads=3, lin_dim=9, lin_vdim=11,
              decay=[0.9, 1.0, 0.3], ff=37, taps=5, buckets=101)
    prompts = [torch.arange(19) % 77, (torch.arange(3) * 7) % 77]
    outs = []
    for ex in _executors(dtype, kw, mb=2, smax=64, width=50, vocab=77):
        rows = [r.float().cpu() for r in ex.prefill_slots(
            [1, 0], prompts, want=[list(range(19)), [2]])]
        for step in range(3):
            ex.tokbuf[0].copy_(torch.tensor([5 + step, 9 + step]))
            ex.slot_step_compute(park=torch.zeros(2, dtype=torch.bool,
                                                  device=ex.device))
            rows.append(ex.logits_buf[0].float().cpu().clone())
            ex.kvs[0].pos.add_(1)
        outs.append(torch.cat(rows))
    cpu, gpu = outs
    rel = float((gpu - cpu).pow(2).mean().sqrt() / cpu.pow(2).mean().sqrt())
    assert rel < (2e-4 if dtype == "float32" else 0.2), rel
