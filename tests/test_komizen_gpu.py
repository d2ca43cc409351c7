"""GPU numerics of the Komizen kernels (residual streams, gated delta rule,
latent-attention append / query pack / shared key-value rows, ungated
experts) against their plain-PyTorch references (dnet_amd.ops.reference), in
bf16 and fp32, with ragged batches, slot indirection, continued states and
sizes that are not multiples of the kernels' tiles; and the whole model on the
GPU (prefill, graph-captured decode) against the same model on the CPU."""
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


@pytest.mark.parametrize("ydt", DTS)
@pytest.mark.parametrize("odt", DTS)
@pytest.mark.parametrize("S,W", [(3, 352), (1, 64), (4, 36), (2, 1030), (8, 7)])
def test_streams_write_read(ydt, odt, S, W):
    torch.manual_seed(S * 1000 + W)
    M = 5
    xs = torch.randn(M, S * W, device=DEV) * 3
    y = torch.randn(M, W, device=DEV).to(ydt)
    mix = torch.randn(S, S, device=DEV)
    wo, wi = torch.randn(S, device=DEV), torch.randn(S, device=DEV)
    wn = 1 + 0.1 * torch.randn(W, device=DEV)
    xr = xs.cpu().clone()
    r0 = ref.hc_read_norm(xr, wi.cpu(), wn.cpu(), 1e-6, odt)
    g0 = ops.hc_read_norm(xs, wi, wn, 1e-6, odt)
    torch.testing.assert_close(g0.cpu().float(), r0.float(), **_tol(odt))
    r1 = ref.hc_write(xr, y.cpu(), mix.cpu(), wo.cpu(), wi.cpu(), wn.cpu(),
                      1e-6, odt)
    g1 = ops.hc_write(xs, y, mix, wo, wi, wn, 1e-6, odt)
    torch.testing.assert_close(xs.cpu(), xr, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(g1.cpu().float(), r1.float(), **_tol(odt))
    assert ops.hc_write(xs, y, mix, wo, None, None, 1e-6, odt) is None
    ref.hc_write(xr, y.cpu(), mix.cpu(), wo.cpu(), None, None, 1e-6, odt)
    torch.testing.assert_close(xs.cpu(), xr, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,KH,d,dv", [(2, 1, 32, 96), (4, 4, 16, 16),
                                       (6, 2, 24, 40), (3, 3, 128, 72),
                                       (2, 2, 5, 3)])
def test_gated_delta_scan(dt, H, KH, d, dv):
    torch.manual_seed(H * 100 + d)
    T, B, Bc = 37, 3, 4
    C = 2 * KH * d + H * dv
    qkv = torch.randn(B * T, C, device=DEV)
    gates = torch.randn(B * T, 7 + 2 * H, device=DEV).to(dt)
    a_log = torch.rand(H, device=DEV) * 2 - 2
    dtb = torch.randn(H, device=DEV)
    pos, lens, slots = _i32([40, 0, 7]), _i32([37, 2, 0]), _i32([3, 0, 1])
    st = torch.randn(Bc, H, d, dv, device=DEV)
    sr = st.cpu().clone()
    o = ops.gated_delta_scan(qkv, gates, 3, 3 + H, a_log, dtb, st,
                             pos.to(DEV), T, H, KH, d, dv, 1e-6,
                             lens.to(DEV), slots.to(DEV))
    want = ref.gated_delta_scan(qkv.cpu(), gates.cpu(), 3, 3 + H,
                                a_log.cpu(), dtb.cpu(), sr, pos, T, H, KH, d,
                                dv, 1e-6, lens, slots)
    torch.testing.assert_close(o.cpu(), want, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(st.cpu(), sr, atol=2e-4, rtol=2e-4)
    # decode steps continue the same state
    for step in range(3):
        q1 = torch.randn(B, C, device=DEV)
        g1 = torch.randn(B, 7 + 2 * H, device=DEV).to(dt)
        p1 = (pos + lens + step).to(torch.int32)
        idle = _i32([1, 1, 0])
        o = ops.gated_delta_scan(q1, g1, 3, 3 + H, a_log, dtb, st, p1.to(DEV),
                                 1, H, KH, d, dv, 1e-6, idle.to(DEV),
                                 slots.to(DEV))
        want = ref.gated_delta_scan(q1.cpu(), g1.cpu(), 3, 3 + H, a_log.cpu(),
                                    dtb.cpu(), sr, p1, 1, H, KH, d, dv, 1e-6,
                                    idle, slots)
        torch.testing.assert_close(o.cpu(), want, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(st.cpu(), sr, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("R,rd,H,d", [(96, 32, 4, 40), (40, 6, 3, 10),
                                      (192, 64, 8, 64), (9, 2, 1, 3)])
def test_latent_append_pack_attend(dt, R, rd, H, d):
    torch.manual_seed(R + rd)
    T, B, Bc, S = 21, 3, 4, 128
    col0 = 5
    src = torch.randn(B * T, col0 + R + rd + 3, device=DEV).to(dt)
    wn = 1 + 0.1 * torch.randn(R, device=DEV)
    freq = (20000.0 ** (-2.0 * torch.arange(rd // 2) / rd)).float().to(DEV)
    pos, lens, slots = _i32([60, 0, 7]), _i32([21, 2, 0]), _i32([3, 0, 1])
    kc = torch.randn(Bc, 1, S, R + rd, device=DEV).to(dt)
    kr = kc.cpu().clone()
    ops.latent_append(src, col0, wn, 1e-6, R, freq, kc, pos.to(DEV), T,
                      lens.to(DEV), slots.to(DEV))
    ref.latent_append(src.cpu(), col0, wn.cpu(), 1e-6, R, freq.cpu(), kr, pos,
                      T, lens, slots)
    torch.testing.assert_close(kc.cpu().float(), kr.float(), **_tol(dt))
    q = torch.randn(B * T, H * (d + rd), device=DEV).to(dt)
    qabs = torch.randn(H, B * T, R, device=DEV).to(dt)
    qf = ops.latent_q_pack(q, qabs, freq, pos.to(DEV), T, H, d)
    qfr = ref.latent_q_pack(q.cpu(), qabs.cpu(), freq.cpu(), pos, T, H, d)
    torch.testing.assert_close(qf.cpu().float(), qfr.float(), **_tol(dt))
    # shared rows: prompt (matrix-core kernel in bf16) and one decode step
    for Tq, ln in ((T, lens), (1, _i32([1, 1, 0]))):
        qq = (qf[:B * Tq] * 0.3).contiguous()
        out = ops.attn_mod(qq, kc, None, pos.to(DEV), Tq, 0.11, ln.to(DEV),
                           slots.to(DEV), v_dim=R)
        want = ref.attn_mod(qq.cpu(), kc.cpu(), None, pos, Tq, 0.11, ln,
                            slots, v_dim=R)
        torch.testing.assert_close(out.cpu().float(), want.float(),
                                   **_tol(dt))


@pytest.mark.parametrize("M", [1, 5, 33, 64])
def test_moe_up_act(M):
    torch.manual_seed(M)
    E, I, K = 6, 40, 72
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(E, I, K, device=DEV) * K ** -0.5).to(torch.bfloat16)
    we = torch.rand(M, E, device=DEV)
    we[:, 2] = 0                                   # an expert nobody chose
    we[we < 0.4] = 0
    act = ops.moe_up_act(x, w, we)
    want = ref.moe_up_act(x.cpu(), w.cpu(), we.cpu())
    # rows of an expert that no row of the kernel's tile chose are skipped
    hit = (we > 0).t().cpu()                       # [E, M]
    torch.testing.assert_close(act.cpu().float()[hit], want.float()[hit],
                               atol=3e-2, rtol=3e-2)
    dw = (torch.randn(E, 56, I, device=DEV) * I ** -0.5).to(torch.bfloat16)
    out = ops.moe_down(act, dw, None, None, we, 0, False)
    wr = ref.moe_down(want, dw.cpu(), None, None, we.cpu(), 0, False)
    torch.testing.assert_close(out.cpu(), wr, atol=5e-2, rtol=5e-2)


def _executors(dtype, mb=3, smax=192):
    from dnet_amd.models import ModelConfig
    from dnet_amd.models.config import komizen_config
    from dnet_amd.parallel.ring import RingExecutor
    # bfloat16: the two paths round differently and every layer of a random
    # stack multiplies that noise, so the bfloat16 stack is shallow
    deep = dtype == "float32"
    hf = komizen_config(96, 160, "ldml" if deep else "ldm",
                        layers=4 if deep else 3,
                        loop=(1, 3, 2) if deep else None, streams=3,
                        heads=3, dim=24, rot_dim=8, vdim=40, kv_rank=48,
                        q_rank=40, delta_heads=4, delta_kv_heads=2,
                        delta_dim=16, delta_vdim=24, ssm_heads=6, ssm_vdim=8,
                        ssm_state=12, ssm_groups=2,
                        norm_groups=2 if deep else 1, conv=3,
                        experts=5, top=2, expert_ff=48, router_scale=1.25,
                        embedding_scale=3.0)
    from komizen_oracle import make_checkpoint
    sd = make_checkpoint(hf, seed=11,
                         ff_gain=1.0 if dtype == "float32" else 0.1)
    out = []
    for dev, graphs in (("cpu", False), (DEV, True)):
        cfg = ModelConfig.from_hf(hf)
        cfg.compute_dtype = dtype
        ex = RingExecutor(cfg, 0, 1, torch.device(dev), mb_size=mb,
                          smax=smax, use_graphs=graphs, init_weights=False)
        ex.model.load_state_dict(sd)
        out.append(ex)
    return out


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_odd_sizes_gpu_matches_cpu(dtype):
    """Sizes that are multiples of nothing (width, vocabulary, ranks, head
    sizes, expert width): every kernel's unvectorized path and the linears'
    fallbacks, prompt and decode."""
    from dnet_amd.models import ModelConfig
    from dnet_amd.models.config import komizen_config
    from dnet_amd.parallel.ring import RingExecutor
    from komizen_oracle import make_checkpoint
    hf = komizen_config(52, 77, "ldm", layers=3, streams=3, heads=3, dim=10,
                        rot_dim=6, vdim=14, kv_rank=18, q_rank=11,
                        delta_heads=3, delta_kv_heads=3, delta_dim=5,
                        delta_vdim=7, ssm_heads=2, ssm_vdim=9, ssm_state=5,
                        ssm_groups=1, norm_groups=1, conv=2, experts=3, top=2,
                        expert_ff=13, router_scale=0.8, embedding_scale=2.0)
    sd = make_checkpoint(hf, seed=21,
                         ff_gain=1.0 if dtype == "float32" else 0.1)
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 77, (n,), generator=g) for n in (19, 3)]
    outs = []
    for dev, graphs in (("cpu", False), (DEV, True)):
        cfg = ModelConfig.from_hf(hf)
        cfg.compute_dtype = dtype
        ex = RingExecutor(cfg, 0, 1, torch.device(dev), mb_size=2, smax=64,
                          use_graphs=graphs, init_weights=False)
        ex.model.load_state_dict(sd)
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


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_model_gpu_matches_cpu(dtype):
    """Ragged prefill into slots, then graph-captured decode steps with one
    row idle, on the GPU kernels against the CPU reference ops."""
    cpu, gpu = _executors(dtype)
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 160, (n,), generator=g) for n in (70, 9)]
    want = [[0, 33, 69], [8]]

    def same(y, x):
        # float32 is the sharp comparison; in bfloat16 the two paths round
        # differently and these random stacks multiply that noise layer by
        # layer, so the bound is on the root mean square
        y, x = y.float().cpu(), x.float()
        if dtype == "float32":
            torch.testing.assert_close(y, x, atol=2e-3, rtol=2e-3)
        else:
            rel = float((y - x).pow(2).mean().sqrt() / x.pow(2).mean().sqrt())
            assert rel < 0.3, rel

    a = cpu.prefill_slots([2, 0], prompts, want=want)
    b = gpu.prefill_slots([2, 0], prompts, want=want)
    for x, y in zip(a, b):
        same(y, x)
    park = torch.tensor([False, True, False])
    for step in range(4):
        toks = torch.randint(0, 160, (3,), generator=g)
        for ex in (cpu, gpu):
            ex.tokbuf[0].copy_(toks)
            ex.slot_step_compute(park=park.to(ex.device))
        same(gpu.logits_buf[0][[0, 2]], cpu.logits_buf[0][[0, 2]])
        for ex in (cpu, gpu):
            ex.kvs[0].pos.add_((~park).to(ex.device).to(torch.int32))


@pytest.mark.parametrize("Hq,Hkv,D,DV,share", [
    (32, 1, 256, 192, True), (20, 1, 160, 128, True), (80, 1, 72, 40, True),
    (32, 2, 64, 64, False), (48, 1, 128, 128, False)])
@pytest.mark.parametrize("window", [0, 50])
def test_decode_heads_on_matrix_cores(Hq, Hkv, D, DV, share, window):
    """bf16 decode with >= 16 heads per kv head: the grouped heads share the
    staged key tiles on the matrix cores; split over the keys, every score
    modifier, idle rows, slot indirection, positions at tile borders."""
    torch.manual_seed(Hq + D)
    B, Bc, S = 5, 6, 320
    dt = torch.bfloat16
    kc = torch.randn(Bc, Hkv, S, D, device=DEV).to(dt)
    vc = None if share else torch.randn(Bc, Hkv, S, DV, device=DEV).to(dt)
    q = (torch.randn(B, Hq * D, device=DEV) * 0.5).to(dt)
    pos = _i32([0, 31, 32, 300, 77])
    lens = _i32([1, 1, 1, 1, 0])
    slots = _i32([5, 0, 3, 1, 2])
    temp = torch.rand(Hq, device=DEV) + 0.5
    r1, r2 = torch.rand(Hq, device=DEV) * 0.3, torch.rand(Hq, device=DEV)
    sinks = torch.randn(Hq, device=DEV)
    for mods in (dict(), dict(temp=temp, softcap=5.0, dist_r1=r1, dist_r2=r2,
                              sinks=sinks)):
        out = ops.attn_mod(q, kc, vc, pos.to(DEV), 1, D ** -0.5,
                           lens.to(DEV), slots.to(DEV), window=window,
                           v_dim=DV if share else 0, **mods)
        cm = {k: (v.cpu() if torch.is_tensor(v) else v)
              for k, v in mods.items()}
        want = ref.attn_mod(q.cpu(), kc.cpu(), None if share else vc.cpu(),
                            pos, 1, D ** -0.5, lens, slots, window=window,
                            v_dim=DV if share else 0, **cm)
        torch.testing.assert_close(out.cpu().float()[:4], want.float()[:4],
                                   atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("T,E,top", [(1, 8, 4), (33, 5, 2), (700, 64, 6),
                                     (4, 3, 3), (9, 16, 1)])
def test_route_and_weighted_sum(T, E, top):
    torch.manual_seed(T + E)
    logits = torch.randn(T, E, device=DEV) * 2
    we = ops.moe_route(logits, top, 1.5)
    want = ref.moe_route(logits.cpu(), top, 1.5)
    torch.testing.assert_close(we.cpu(), want, atol=1e-6, rtol=1e-5)
    assert int((we > 0).sum(1).min()) == top == int((we > 0).sum(1).max())
    for dt in DTS:
        d = torch.randn(E, T, 72, device=DEV).to(dt)
        out = ops.moe_weighted_sum(d, we)
        torch.testing.assert_close(out.cpu(),
                                   ref.moe_weighted_sum(d.cpu(), want),
                                   atol=1e-4, rtol=1e-4)
