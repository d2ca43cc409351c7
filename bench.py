#!/usr/bin/env python3
"""dnet_amd flagship benchmark: Qwen-2.5 32B int8 pipelined-ring decode.

Measures the BASELINE.json headline metric — output tokens/sec (whole node)
plus p50 TTFT — on synthetic data with random-init weights (no network).

Single GPU:   python bench.py --steps 32 --warmup 8
Multi GPU:    python -m torch.distributed.run --nnodes=1 --nproc-per-node N \
                  --master-addr 127.0.0.1 bench.py --gpus N --steps K --warmup W

One rank per GPU; ring hops are RCCL send/recv over xGMI. A "step" = every
sequence in every microbatch advances one token (one full ring round).
Rank 0 prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import logging
import os
import time

import sys as _sys

import dnet_amd

# TunableOp algo cache covers the HEADLINE model's prefill shapes only;
# enabling it globally taxes eager-decode models (see enable_tunableop_cache)
def _bench_model_arg() -> str:
    av = _sys.argv
    for i, a in enumerate(av):
        if a == "--model" and i + 1 < len(av):
            return av[i + 1]
        if a.startswith("--model="):
            return a.split("=", 1)[1]
    return "qwen-2.5-32b"


if _bench_model_arg().startswith("qwen-2.5-32b"):
    dnet_amd.enable_tunableop_cache()
import torch

logging.basicConfig(level=logging.INFO)

from dnet_amd.models import ModelConfig, PRESETS, QuantConfig
from dnet_amd.parallel.comm import init_from_env
from dnet_amd.parallel.ring import RingExecutor


# equal-size family comparison: (name, width, heads, kv_heads, head_dim, ff)
_COMPARE_SIZES = [("2k", 2048, 16, 4, 128, 8192),
                  ("4k", 4096, 32, 8, 128, 12288),
                  ("5k", 5120, 64, 8, 128, 25600)]


def _family_hf(fam, W, H, KV, D, FF, layers, vocab, args):
    """config.json-style description of ``fam`` at the given layer sizes."""
    from dnet_amd.models.config import (gegorax_config, komizen_config,
                                        lurisun_config, posudra_config)
    if fam == "lurisun":
        # constant-decay linear attention, windowed latent attention and
        # chunked sigmoid attention in turn; linear-attention heads of D x D
        # state over the model width, 256 cached latent entries per token,
        # window and chunk half the prompt, a 4-tap input convolution in
        # every layer, a hashed pair table beside the embedding, dense gated
        # feed-forwards
        return lurisun_config(
            W, vocab, "nla", layers=layers, heads=H, kv_heads=KV, dim=D,
            rot_dims=D // 2, chunk=max(64, args.prompt_len // 2),
            latent_heads=H, latent_dim=D, latent_vdim=D, kv_rank=256,
            q_rank=max(256, W // 4), window=max(64, args.prompt_len // 2),
            lin_heads=W // D, lin_dim=D, lin_vdim=D,
            decay=[1.0 - 2.0 ** -(3 + h % 8) for h in range(W // D)], ff=FF,
            taps=4, buckets=100003)
    if fam == "komizen":
        # latent attention (every second layer) with gated delta-rule and
        # mamba2 layers between; 192 + 64 cached entries per token; 4
        # residual streams; delta-rule and state-space heads of 64 channels
        # over the model width as in the gegorax stack; every feed-forward a
        # mixture of ungated experts whose chosen ones together are as wide
        # as the dense feed-forward it stands beside
        E = args.compare_experts or 8
        top = min(2, E)
        return komizen_config(
            W, vocab, "ldlm", layers=layers, heads=H, dim=D, rot_dim=64,
            vdim=D, kv_rank=192, q_rank=max(256, W // 4),
            delta_heads=W // 64, delta_kv_heads=max(1, W // 128),
            delta_dim=64, delta_vdim=64, ssm_heads=W // 64, ssm_vdim=64,
            ssm_state=128, ssm_groups=max(1, W // 512), conv=4, experts=E,
            top=top, expert_ff=FF // top, streams=4)
    if fam == "posudra":
        return posudra_config(W, layers, H, KV, D, D, FF, vocab)
    if fam == "gegorax":
        # attention + state-space layers alternate with delta-rule layers;
        # window half the prompt, 16-position pooled blocks; state-space and
        # delta-rule heads of 64 channels over the model width; a per-layer
        # token input of 256 channels; dense feed-forwards unless
        # --compare-experts asks for a mixture in every second layer
        E = args.compare_experts
        return gegorax_config(
            W, layers, vocab, H, KV, D, D, window=max(64, args.prompt_len // 2),
            pool=16, ssm_heads=W // 64, ssm_vdim=64, ssm_state=128,
            delta_heads=W // 64, delta_dim=64, ff=FF, experts=E,
            top=min(4, E), expert_ff=FF // 8, shared_ff=FF // 8 if E else 0,
            side_dim=256)
    return dict(model_type="qwen3", hidden_size=W,
                num_hidden_layers=layers, num_attention_heads=H,
                num_key_value_heads=KV, head_dim=D,
                intermediate_size=FF, vocab_size=vocab,
                rope_theta=1000000.0, rms_norm_eps=1e-6)


# family -> the closest existing family it is measured beside
_COMPARE_WITH = {"posudra": "qwen3", "gegorax": "posudra",
                 "komizen": "gegorax", "lurisun": "gegorax"}


def compare_family(args, device):
    """Prefill and decode throughput of a family beside the closest existing
    one (posudra: qwen3 — dense, grouped heads, q/k norm; gegorax: posudra —
    one norm feeding parallel branches, fp32 residual, per-layer sizes;
    komizen: gegorax — attention beside state-space and delta-rule layers on
    an fp32 residual with per-slot recurrent state; lurisun: gegorax —
    windowed attention beside linear recurrences with per-slot state, dense
    feed-forwards, fp32 residual) at
    equal layer sizes, bf16, random weights. One JSON line; the default
    workload is untouched."""
    new, old = args.compare_family, _COMPARE_WITH[args.compare_family]
    layers, vocab = args.compare_layers, 32768
    B, T, Bd = args.compare_prefill_batch, args.prompt_len, args.mb_size
    rows = []
    for name, W, H, KV, D, FF in _COMPARE_SIZES:
        if args.compare_sizes and name not in args.compare_sizes.split(","):
            continue
        row = {"size": name, "width": W, "heads": H, "kv_heads": KV,
               "head_dim": D, "ff": FF, "layers": layers}
        for fam in (new, old):
            hf = _family_hf(fam, W, H, KV, D, FF, layers, vocab, args)
            cfg = ModelConfig.from_hf(hf)
            g = torch.Generator().manual_seed(7)
            # prefill: B prompts of T tokens, eager (as serving runs it)
            ex = RingExecutor(cfg, 0, 1, device, mb_count=1, mb_size=B,
                              smax=args.smax, seed=1234, use_graphs=False)
            toks = torch.randint(0, vocab, (1, B, T), generator=g).to(device)
            ts = []
            for _ in range(4):
                ex.reset()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                ex.prefill(toks)
                torch.cuda.synchronize()
                ts.append(time.perf_counter() - t0)
            row[fam + "_prefill_tok_s"] = round(B * T / min(ts[1:]), 1)
            del ex
            torch.cuda.empty_cache()
            # decode: Bd sequences at context ~T, hipGraph steps
            ex = RingExecutor(cfg, 0, 1, device, mb_count=1, mb_size=Bd,
                              smax=args.smax, seed=1234,
                              use_graphs=not args.no_graphs)
            toks = torch.randint(0, vocab, (1, Bd, T), generator=g).to(device)
            ex.prefill(toks)
            ex.decode_rounds(args.warmup, collect=False)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ex.decode_rounds(args.steps, collect=False)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            row[fam + "_decode_tok_s"] = round(Bd * args.steps / dt, 1)
            row[fam + "_decode_ms_step"] = round(dt / args.steps * 1e3, 3)
            del ex
            torch.cuda.empty_cache()
        rows.append(row)
    print(json.dumps({
        "metric": f"{new} vs {old} at equal layer sizes: prefill and "
                  "decode tokens/s (1 GPU, bf16)",
        "dtype": "bf16", "data": "synthetic (random tokens, random-init "
                                 "weights)",
        "prefill": {"batch": B, "prompt_len": T},
        "decode": {"batch": Bd, "context": T, "steps": args.steps,
                   "warmup": args.warmup},
        "rows": rows}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--model", default="qwen-2.5-32b")
    ap.add_argument("--quant", default="int8",
                    choices=["int8", "int4", "bf16", "mxfp4"])
    ap.add_argument("--mb-size", type=int, default=64,
                    help="sequences per microbatch")
    ap.add_argument("--mb-per-rank", type=int, default=0,
                    help="microbatches = mb_per_rank * world (pipeline fill); "
                         "0 = auto (1 on a single GPU, 2 per rank otherwise)")
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--smax", type=int, default=1024)
    ap.add_argument("--layers", type=int, default=0,
                    help="override layer count (debug only; invalid for scoring)")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--kv-bits", type=int, default=16, choices=[8, 16])
    ap.add_argument("--tp", type=int, default=1,
                    help="tensor-parallel degree inside each pipeline stage")
    ap.add_argument("--cp", type=int, default=1,
                    help="context-parallel degree (KV sequence sharding)")
    ap.add_argument("--prefill-chunk", type=int, default=0,
                    help="prefill position-chunk size (bounds activation "
                         "memory for long prompts; 0 = one shot)")
    ap.add_argument("--residency", type=int, default=0,
                    help="GPU-resident layers per rank (0=all; <local layers "
                         "enables host-DRAM weight streaming)")
    ap.add_argument("--compare-family", default="",
                    choices=["", "posudra", "gegorax", "komizen", "lurisun"],
                    help="instead of the default workload: throughput of "
                         "this family beside its closest existing one at "
                         "equal layer sizes")
    ap.add_argument("--compare-layers", type=int, default=8)
    ap.add_argument("--compare-experts", type=int, default=0,
                    help="gegorax: experts of the mixture feed-forward in "
                         "every second layer (0 = dense feed-forwards); "
                         "komizen: experts of every layer (0 = 8)")
    ap.add_argument("--compare-prefill-batch", type=int, default=8)
    ap.add_argument("--compare-sizes", default="",
                    help="comma list out of 2k,4k,5k (default: all)")
    args = ap.parse_args()

    rank, world, device = init_from_env()
    on_gpu = device.type == "cuda"
    if args.compare_family:
        assert world == 1 and on_gpu, "family comparison: one GPU"
        if args.prompt_len == 128:
            args.prompt_len = 1024
        args.smax = max(args.smax, args.prompt_len + args.steps
                        + args.warmup + 64)
        if args.mb_size == 64:
            args.mb_size = 32
        compare_family(args, device)
        return

    quant = None
    if args.quant == "int8":
        quant = QuantConfig(8, 128)
    elif args.quant == "int4":
        quant = QuantConfig(4, 128)
    elif args.quant == "mxfp4":
        quant = QuantConfig(4, 32, fmt="mxfp4")   # expert banks only
    hf = dict(PRESETS[args.model])
    if args.layers:
        hf["num_hidden_layers"] = args.layers
    cfg = ModelConfig.from_hf(hf, quant=quant)

    mb_per_rank = args.mb_per_rank or (1 if world == 1 else 2)
    mb_count = max(mb_per_rank * world, 1)
    ex = RingExecutor(cfg, rank, world, device, mb_count=mb_count,
                      mb_size=args.mb_size, smax=args.smax, seed=1234,
                      use_graphs=on_gpu and not args.no_graphs and args.tp == 1,
                      residency=args.residency, tp=args.tp,
                      cp=args.cp,
                      kv_bits=args.kv_bits)

    g = torch.Generator().manual_seed(7)
    tokens = torch.randint(0, cfg.vocab_size,
                           (mb_count, args.mb_size, args.prompt_len),
                           generator=g).to(device)

    def barrier_sync():
        if world > 1:
            torch.distributed.barrier()
        if on_gpu:
            torch.cuda.synchronize()

    # TTFT: p50 over >= 5 prefills (a single measurement is
    # not a p50); each prefill resets the ring KV first
    ttft_samples = []
    n_prefills = max(1, int(os.environ.get("DNET_BENCH_PREFILLS", "5")))
    for i in range(n_prefills):
        ex.reset()
        barrier_sync()
        t0 = time.perf_counter()
        ex.prefill(tokens, chunk=args.prefill_chunk)
        barrier_sync()
        ttft_samples.append((time.perf_counter() - t0) * 1e3)
    ttft_samples.sort()
    ttft_ms = ttft_samples[len(ttft_samples) // 2]

    # warmup decode
    ex.decode_rounds(args.warmup, collect=False)
    barrier_sync()

    t0 = time.perf_counter()
    ex.decode_rounds(args.steps, collect=False)
    barrier_sync()
    elapsed = time.perf_counter() - t0

    # self-corroboration: a few individually timed steps AFTER the timed
    # region (sync per step), so the record shows per-step times without
    # cross-referencing profiles/
    step_samples = []
    for _ in range(3):
        barrier_sync()
        t1 = time.perf_counter()
        ex.decode_rounds(1, collect=False)
        barrier_sync()
        step_samples.append(round((time.perf_counter() - t1) * 1e3, 2))

    # max over ranks
    if world > 1:
        t = torch.tensor([elapsed], device=device if on_gpu else "cpu")
        torch.distributed.all_reduce(t, op=torch.distributed.ReduceOp.MAX)
        elapsed = float(t[0])

    total_seqs = mb_count * args.mb_size
    tokens_generated = total_seqs * args.steps
    toks_per_s = tokens_generated / elapsed
    ms_per_step = elapsed / args.steps * 1e3

    if rank == 0:
        result = {
            "metric": f"output tokens/sec (whole node), {args.model} "
                      f"{args.quant} pipelined ring",
            "value": round(toks_per_s, 2),
            "unit": "tokens/s",
            "n_gpus": world,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(ms_per_step, 3),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": ("bf16" if quant is None else
                      ("mxfp4 experts (bf16 attention/compute)"
                       if quant.fmt == "mxfp4" else
                       f"int{quant.bits}-g{quant.group} weights (bf16 compute)")),
            "data": "synthetic (random tokens, random-init weights)",
            "ttft_ms": round(ttft_ms, 1),
            "ttft_samples_ms": [round(t, 1) for t in ttft_samples],
            "step_samples_ms": step_samples,
            "config": {
                "model": args.model,
                "global_batch": total_seqs,
                "seq_len": args.prompt_len,
                "gen_len": args.steps,
                "parallelism": (f"ring-pp{world // (args.tp * args.cp)}"
                                + (f"xtp{args.tp}" if args.tp > 1 else "")
                                + (f"xcp{args.cp}" if args.cp > 1 else ""))
                               + (f"+offload(res={args.residency})"
                                  if args.residency else ""),
                "microbatches": mb_count,
                "mb_size": args.mb_size,
                "layers": cfg.num_layers,
            },
        }
        print(json.dumps(result))
    if world > 1:
        torch.distributed.destroy_process_group()


if __name__ == "__main__":
    main()
