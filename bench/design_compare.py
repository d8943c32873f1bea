#!/usr/bin/env python3
"""
Datatar beside the framework's closest existing model (Mixtral: MoE feed-forward, paged GQA attention) at equal
size, random weights, one GPU (``python bench.py --design-compare`` runs this; the default bench is unchanged).

Per size, for both models through the same engine (scheduler, paged cache, runner, hipGraph decode, sampling):

* prefill throughput: ``batch`` prompts of ``prompt`` tokens, prompt tokens / s of the prefill steps;
* decode throughput: ``gen`` tokens per sequence, generated tokens / s of the decode steps;

and for the attention kernels alone at the same rows / context (events around the op, median of ``iters``):

* prefill (compute-bound): achieved matrix FLOP/s over the 2.5 PFLOP/s dense bf16 peak; FLOPs counted over
  the causal triangle (window = context), 2 * pairs * (score width + value width) per head;
* decode (memory-bound): cache bytes read / time over the 8 TB/s HBM3E peak.

Prints one JSON line per measurement and a final summary line.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16 = 2.5e15
PEAK_HBM = 8.0e12

# name: (hidden, layers, heads, experts, top, expert ff, vocab | Datatar: dim, rot_dim, vdim, kv_rank, q_rank, shared ff)
SIZES = {
    "2k-moe8": dict(hidden=2048, layers=4, heads=16, experts=8, top=2, ff=2048, vocab=32000,
                    dim=96, rot_dim=32, vdim=128, kv_rank=256, q_rank=768, shared_ff=2048),
    "4k-moe8": dict(hidden=4096, layers=2, heads=32, experts=8, top=2, ff=4096, vocab=32000,
                    dim=96, rot_dim=32, vdim=128, kv_rank=256, q_rank=1536, shared_ff=4096),
}


def datatar_arch(z, window):
    from src.models.datatar import DatatarArch, LatentAttnSpec, LayerSpec, MlpSpec

    m = LatentAttnSpec(heads=z["heads"], dim=z["dim"], rot_dim=z["rot_dim"], vdim=z["vdim"], kv_rank=z["kv_rank"],
                       q_rank=z["q_rank"], scale=1.0 / math.sqrt(z["dim"] + z["rot_dim"]), window=window,
                       rot_base=10000.0, rot_dims=z["rot_dim"])
    f = MlpSpec("moe", experts=z["experts"], top=z["top"], expert_ff=z["ff"], shared_ff=z["shared_ff"])
    return DatatarArch("datatar-bench", z["vocab"], z["hidden"], tuple(LayerSpec("latent_attention", m, f)
                                                                         for _ in range(z["layers"])),
                       logit_scale=1.0)


def mixtral_arch(z):
    from src.models.presets import ArchConfig

    return ArchConfig("mixtral-bench", z["hidden"], z["layers"], z["heads"], max(1, z["heads"] // 4), z["ff"],
                      z["vocab"], rope_theta=1e6, max_position=8192, num_experts=z["experts"], top_k=z["top"])


def serve(model, a, label, size):
    from src.config import EngineConfig
    from src.engine import LLMEngine
    from src.preproc import SamplingParams

    cfg = EngineConfig(max_num_seqs=a.batch, max_num_batched_tokens=a.batch * a.prompt, num_kv_blocks=None,
                       enable_prefix_caching=False, graph_batch_sizes=[a.batch], mixed_batching="off",
                       gpu_memory_fraction=0.5, tuned_gemm_table=False)
    eng = LLMEngine(model, cfg, a.prompt + a.gen + 16, eos_token_id=None)
    eng.runner.capture_graphs()
    g = torch.Generator().manual_seed(0)
    out = None
    for it in range(a.warmup + a.steps):
        if it == a.warmup:
            eng.stats.update(prefill_time=0.0, decode_time=0.0, prompt_tokens=0, generated_tokens=0)
        prompts = [torch.randint(0, model.arch.vocab_size, (a.prompt,), generator=g).tolist() for _ in range(a.batch)]
        eng.generate(prompts, SamplingParams(max_tokens=a.gen, ignore_eos=True))
    st = eng.stats
    dec_tokens = st["generated_tokens"] - a.steps * a.batch  # each prompt's first token comes from its prefill step
    out = {"bench": "design_compare", "model": label, "size": size, "batch": a.batch, "prompt": a.prompt,
           "gen": a.gen, "prefill_tok_s": round(st["prompt_tokens"] / st["prefill_time"], 1),
           "decode_tok_s": round(dec_tokens / st["decode_time"], 1), "graphs": list(eng.runner.graph_sizes),
           "kv_bytes_per_token": model.arch.kv_bytes_per_token()}
    print(json.dumps(out), flush=True)
    del eng
    torch.cuda.empty_cache()
    return out


def _time(fn, iters):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e-3)
    return statistics.median(ts)


def attention_kernels(z, a, size):
    """The two designs' attention kernels alone: ``batch`` sequences, prompt rows (prefill) / one row (decode)."""
    from src import ops

    dev, bf = "cuda", torch.bfloat16
    bs, S, L, H = 16, a.batch, a.prompt, z["heads"]
    nb = S * (L // bs)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(S, L // bs)
    ctx = torch.full((S,), L, dtype=torch.int32, device=dev)
    cu = (torch.arange(S + 1, dtype=torch.int32, device=dev) * L)
    pairs = S * L * (L + 1) / 2
    res = []
    # latent attention: score width kv_rank + rot_dim, value width kv_rank, keys shared by all heads
    R, rot = z["kv_rank"], z["rot_dim"]
    inv = ops.rope_inv_freq(10000.0, rot, dev)
    cache = (torch.randn(nb, bs, R + rot, device=dev) * 0.5).to(bf)
    sink = torch.zeros(H, device=dev)
    scale = 1.0 / math.sqrt(z["dim"] + rot)
    for mode, T, pos, cuq, mq in (("prefill", S * L, torch.arange(L, device=dev).repeat(S), cu, L),
                                  ("decode", S, torch.full((S,), L - 1, device=dev), None, 1)):
        q_lat = (torch.randn(H, T, R, device=dev) * 0.1).to(bf)
        q = (torch.randn(T, H * (z["dim"] + rot), device=dev) * 0.1).to(bf)
        for impl in (0, 1):
            if impl == 1 and mode == "prefill" and T * L > 2 ** 24:
                continue  # the FMA form is the fp32 / odd-shape path: timed at decode only for large prompts
            t = _time(lambda: ops.latent_attn(q_lat, q, z["dim"], cache, bt, cuq, ctx, pos, sink, mq, 0, scale, rot, inv,
                                              impl=impl), a.iters)
            r = {"bench": "attn_kernel", "design": "datatar", "kernel": "latent_attn" + ("_fma" if impl else "_mfma"),
                 "mode": mode, "size": size, "ms": round(t * 1e3, 4)}
            if mode == "prefill":
                r["flops_frac_of_peak"] = round(2 * pairs * H * (2 * R + rot) / t / PEAK_BF16, 4)
            else:
                r["hbm_frac_of_peak"] = round(S * L * (R + rot) * 2 / t / PEAK_HBM, 4)
            res.append(r)
            print(json.dumps(r), flush=True)
    # paged GQA attention of the Llama / Mixtral path: head_dim 128, heads / 4 KV heads
    hkv, d = max(1, H // 4), 128
    kc = (torch.randn(nb, hkv, bs, d, device=dev) * 0.5).to(bf)
    vc = (torch.randn(nb, hkv, bs, d, device=dev) * 0.5).to(bf)
    q = (torch.randn(S * L, H * d, device=dev) * 0.1).to(bf)
    t = _time(lambda: ops.attn_prefill(q, kc, vc, bt, cu, ctx, L, H, hkv, 1.0 / math.sqrt(d)), a.iters)
    r = {"bench": "attn_kernel", "design": "mixtral", "kernel": "attn_prefill", "mode": "prefill", "size": size,
         "ms": round(t * 1e3, 4), "flops_frac_of_peak": round(2 * pairs * H * 2 * d / t / PEAK_BF16, 4)}
    res.append(r)
    print(json.dumps(r), flush=True)
    maxp = ops.decode_partials(L)
    part_o = torch.empty(S * H * maxp * 128, dtype=torch.float32, device=dev)
    part_ml = torch.empty(S * H * maxp * 2, dtype=torch.float32, device=dev)
    cnt = torch.zeros(S * hkv, dtype=torch.int32, device=dev)
    qd = (torch.randn(S, H * d, device=dev) * 0.1).to(bf)
    t = _time(lambda: ops.attn_decode(qd, kc, vc, bt, ctx, L, H, hkv, 1.0 / math.sqrt(d), part_o=part_o,
                                      part_ml=part_ml, counters=cnt), a.iters)
    r = {"bench": "attn_kernel", "design": "mixtral", "kernel": "attn_decode", "mode": "decode", "size": size,
         "ms": round(t * 1e3, 4), "hbm_frac_of_peak": round(S * L * hkv * d * 2 * 2 / t / PEAK_HBM, 4)}
    res.append(r)
    print(json.dumps(r), flush=True)
    return res


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--sizes", default=",".join(SIZES))
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--gen", type=int, default=64)
    ap.add_argument("--steps", type=int, default=2)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--window", type=int, default=0, help="Datatar's sliding window (0: full context, as the GQA path)")
    ap.add_argument("--skip-serving", action="store_true")
    ap.add_argument("--skip-kernels", action="store_true")
    ap.add_argument("--models", default="datatar,mixtral", help="which models to serve")
    a = ap.parse_args(argv)
    assert torch.cuda.is_available(), "needs a GPU"
    from src.models.datatar import DatatarLM
    from src.models.llama import CausalLM

    t0 = time.time()
    summary = []
    for size in a.sizes.split(","):
        z = SIZES[size]
        if not a.skip_kernels:
            summary += attention_kernels(z, a, size)
        if a.skip_serving:
            continue
        if "datatar" in a.models.split(","):
            summary.append(serve(DatatarLM(datatar_arch(z, a.window), "cuda:0", seed=1, init_std=0.02), a, "datatar",
                                 size))
        if "mixtral" in a.models.split(","):
            summary.append(serve(CausalLM(mixtral_arch(z), "cuda:0", seed=1), a, "mixtral", size))
    print(json.dumps({"bench": "design_compare_summary", "seconds": round(time.time() - t0, 1), "rows": summary}),
          flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
