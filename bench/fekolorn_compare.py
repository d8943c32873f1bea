#!/usr/bin/env python3
"""
Fekolorn beside the framework's closest existing model (Llama: dense feed-forward, paged GQA attention) at equal
size, random weights, one GPU (``python bench.py --fekolorn-compare`` runs this; the default bench is unchanged).

Per size, for both models through the same engine (scheduler, paged cache, state slots, runner, hipGraph decode,
sampling):

* prefill throughput: ``batch`` prompts of ``prompt`` tokens, prompt tokens / s of the prefill steps;
* decode throughput: ``gen`` tokens per sequence, generated tokens / s of the decode steps;

and for the new design's kernels alone beside their like in the Llama path (events around the op, median of
``iters``):

* attention, prefill (compute-bound): achieved matrix FLOP/s over the 2.5 PFLOP/s dense bf16 peak, FLOPs counted
  over the causal triangle, 2 * pairs * (dim + vdim) per head;
* attention, decode (memory-bound): cache bytes read / time over the 8 TB/s HBM3E peak;
* residual-stream update + pre-norm, polynomial activation, qkv preparation (memory-bound): bytes moved / time
  over the HBM peak, beside the Llama path's fused residual-add + RMS norm;
* gated delta rule (a sequential recurrence on the vector ALUs): FLOP/s over the 157 TFLOP/s fp32 vector peak.

Prints one JSON line per measurement and a final summary line.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)



def _sibling(name):
    """A module of this folder by file (the folder shares its name with bench.py and is no package)."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(name, os.path.join(ROOT, "bench", name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_dc = _sibling("design_compare")
PEAK_BF16, PEAK_HBM, _time, serve = _dc.PEAK_BF16, _dc.PEAK_HBM, _dc._time, _dc.serve

PEAK_FP32_VALU = 157.3e12

# hidden, layers (a "parallel" and an "attention" layer alternate), heads, kv heads, head dims, feed-forward widths
SIZES = {
    "2k": dict(hidden=2048, layers=4, heads=16, kv_heads=4, dim=128, vdim=128, ff=8192, llama_ff=5504, vocab=32000,
               streams=4, window=1024, conv=4),
    "4k": dict(hidden=4096, layers=2, heads=32, kv_heads=8, dim=128, vdim=128, ff=16384, llama_ff=11008, vocab=32000,
               streams=4, window=1024, conv=4),
}


def fekolorn_arch(z):
    from src.models.fekolorn import (FekLayerSpec, FekolornArch, GatedDeltaSpec, ParallelSpec, PolyMlpSpec,
                                     SinkAttnSpec)

    scale = 1.0 / math.sqrt(z["dim"])
    left = SinkAttnSpec(z["heads"], z["kv_heads"], z["dim"], z["vdim"], scale, rot_dims=z["dim"] // 2, v_unit=True)
    right = GatedDeltaSpec(z["heads"], z["kv_heads"], z["dim"], z["vdim"], z["conv"])
    att = SinkAttnSpec(z["heads"], z["kv_heads"], z["dim"], z["vdim"], scale, window=z["window"], qk_norm=True,
                       v_mix=True, bias_max=128.0)
    mlp = PolyMlpSpec(z["ff"])
    layers = []
    for i in range(z["layers"]):
        layers.append(FekLayerSpec("parallel", ParallelSpec(left, right, 0.6, 0.9), mlp) if i % 2 == 0
                      else FekLayerSpec("attention", att, mlp))
    return FekolornArch("fekolorn-bench", z["vocab"], z["hidden"], tuple(layers), streams=z["streams"],
                        bigram_buckets=65521, bigram_mul_prev=31, bigram_mul_cur=7)


def llama_arch(z):
    from src.models.presets import ArchConfig

    return ArchConfig("llama-bench", z["hidden"], z["layers"], z["heads"], z["kv_heads"], z["llama_ff"], z["vocab"],
                      rope_theta=1e6, max_position=8192)


def kernels(z, a, size):
    from src import ops
    from src.ops import seq

    dev, bf = "cuda", torch.bfloat16
    bs, S, L = 16, a.batch, a.prompt
    H, G, D, DV, W = z["heads"], z["kv_heads"], z["dim"], z["vdim"], z["hidden"]
    nb = S * (L // bs)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(S, L // bs)
    ctx = torch.full((S,), L, dtype=torch.int32, device=dev)
    cu = (torch.arange(S + 1, dtype=torch.int32, device=dev) * L)
    pairs = S * L * (L + 1) / 2
    res = []

    def emit(r):
        r.update(bench="kernel", size=size)
        res.append(r)
        print(json.dumps(r), flush=True)

    cache = (torch.randn(nb, bs, G * (D + DV), device=dev) * 0.5).to(bf)
    sink = torch.zeros(H, device=dev)
    bias = torch.zeros(130, H, device=dev)   # distances up to 128 have their own bias, the rest share one
    scale = 1.0 / math.sqrt(D)
    for mode, T, pos, cuq, mq in (("prefill", S * L, torch.arange(L, device=dev).repeat(S), cu, L),
                                  ("decode", S, torch.full((S,), L - 1, device=dev), None, 1)):
        q = (torch.randn(T, H * D, device=dev) * 0.1).to(bf)
        for label, b in (("sink_attn", None), ("sink_attn+bias", bias)):
            t = _time(lambda: seq.sink_attn(q, cache, bt, cuq, ctx, pos, sink, b, mq, H, G, D, DV, 0, scale), a.iters)
            r = {"design": "fekolorn", "kernel": label, "mode": mode, "ms": round(t * 1e3, 4)}
            if mode == "prefill":
                r["flops_frac_of_peak"] = round(2 * pairs * H * (D + DV) / t / PEAK_BF16, 4)
            else:
                r["hbm_frac_of_peak"] = round(S * L * G * (D + DV) * 2 / t / PEAK_HBM, 4)
            emit(r)
    if ops.native_available() and D == 128 and DV == 128:
        kc = (torch.randn(nb, G, bs, D, device=dev) * 0.5).to(bf)
        vc = (torch.randn(nb, G, bs, D, device=dev) * 0.5).to(bf)
        q = (torch.randn(S * L, H * D, device=dev) * 0.1).to(bf)
        t = _time(lambda: ops.attn_prefill(q, kc, vc, bt, cu, ctx, L, H, G, scale), a.iters)
        emit({"design": "llama", "kernel": "attn_prefill", "mode": "prefill", "ms": round(t * 1e3, 4),
              "flops_frac_of_peak": round(2 * pairs * H * 2 * D / t / PEAK_BF16, 4)})
        maxp = ops.decode_partials(L)
        part_o = torch.empty(S * H * maxp * 128, dtype=torch.float32, device=dev)
        part_ml = torch.empty(S * H * maxp * 2, dtype=torch.float32, device=dev)
        cnt = torch.zeros(S * G, dtype=torch.int32, device=dev)
        qd = (torch.randn(S, H * D, device=dev) * 0.1).to(bf)
        t = _time(lambda: ops.attn_decode(qd, kc, vc, bt, ctx, L, H, G, scale, part_o=part_o, part_ml=part_ml,
                                          counters=cnt), a.iters)
        emit({"design": "llama", "kernel": "attn_decode", "mode": "decode", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(S * L * G * D * 2 * 2 / t / PEAK_HBM, 4)})

    # memory-bound row kernels at prompt size
    T = S * L
    Sn = z["streams"]
    xs = torch.randn(T, Sn, W, device=dev)
    y = torch.randn(T, W, device=dev).to(bf)
    mixw, outw, inw = torch.eye(Sn, device=dev), torch.ones(Sn, device=dev), torch.ones(Sn, device=dev) / Sn
    gain = torch.ones(1, device=dev)
    t = _time(lambda: seq.stream_mix_norm(xs, y, None, 1.0, 1.0, mixw, outw, inw, gain, 1e-6, bf), a.iters)
    emit({"design": "fekolorn", "kernel": "stream_mix_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * W * (8 * Sn + 4) / t / PEAK_HBM, 4)})
    if ops.native_available():
        r32 = torch.randn(T, W, device=dev).to(bf)
        wn = torch.ones(W, device=dev).to(bf)
        t = _time(lambda: ops.fused_add_rms_norm(y, r32, wn, 1e-6), a.iters)
        emit({"design": "llama", "kernel": "fused_add_rms_norm", "mode": "prefill", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T * W * 8 / t / PEAK_HBM, 4)})
    zf = torch.randn(T, z["ff"], device=dev).to(bf)
    coef = torch.tensor([0.5, 0.3, 0.2, 0.1], device=dev)
    t = _time(lambda: seq.poly_norm_act(zf, coef, 1e-6), a.iters)
    emit({"design": "fekolorn", "kernel": "poly_norm_act", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * z["ff"] * 4 / t / PEAK_HBM, 4)})
    if ops.native_available():
        gu = torch.randn(T, 2 * z["llama_ff"], device=dev).to(bf)
        t = _time(lambda: ops.silu_and_mul(gu), a.iters)
        emit({"design": "llama", "kernel": "silu_and_mul", "mode": "prefill", "ms": round(t * 1e3, 4),
              "hbm_frac_of_peak": round(T * z["llama_ff"] * 6 / t / PEAK_HBM, 4)})
    p = torch.randn(T, (H + 2 * G) * D, device=dev).to(bf)
    nq, nk = H * D, G * D
    slots = torch.arange(T, device=dev)
    pos = torch.arange(L, device=dev).repeat(S)
    from src.ops import mix as mixops

    inv = mixops.rope_inv_freq(10000.0, D // 2, dev)
    t = _time(lambda: seq.qkv_prep(p[:, :nq], p[:, nq: nq + nk], p[:, nq + nk:], cache, H, G, D, DV, pos, slots, 1e-6,
                                   rot_dims=D // 2, inv_freq=inv, v_unit=True), a.iters)
    emit({"design": "fekolorn", "kernel": "qkv_prep", "mode": "prefill", "ms": round(t * 1e3, 4),
          "hbm_frac_of_peak": round(T * ((H + 2 * G) * D * 2 + (H + 2 * G) * D * 2) / t / PEAK_HBM, 4)})

    # gated delta rule: prompt and decode
    C = 2 * G * D + H * DV
    state = torch.zeros(S + 1, H, D, DV, device=dev)
    sl = torch.arange(S, dtype=torch.int32, device=dev)
    nw = torch.ones(DV, device=dev)
    for mode, T2, rag in (("prefill", S * L, seq.Ragged(torch.arange(L, device=dev).repeat(S), cu, sl)),
                          ("decode", S, seq.Ragged(torch.full((S,), L - 1, device=dev), None, sl))):
        qkv32 = torch.randn(T2, C, device=dev) * 0.1
        bg = torch.rand(T2, 2 * H, device=dev)
        gate = torch.randn(T2, H * DV, device=dev).to(bf)
        t = _time(lambda: seq.gated_delta(qkv32, bg, gate, nw, 1e-6, state, H, G, D, DV, rag), a.iters)
        r = {"design": "fekolorn", "kernel": "gated_delta", "mode": mode, "ms": round(t * 1e3, 4),
             "valu_fp32_frac_of_peak": round(T2 * H * 6 * D * DV / t / PEAK_FP32_VALU, 4)}
        if mode == "decode":
            r["hbm_frac_of_peak"] = round(S * H * D * DV * 8 / t / PEAK_HBM, 4)
        emit(r)
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
    ap.add_argument("--skip-serving", action="store_true")
    ap.add_argument("--skip-kernels", action="store_true")
    ap.add_argument("--models", default="fekolorn,llama", help="which models to serve")
    a = ap.parse_args(argv)
    assert torch.cuda.is_available(), "needs a GPU"
    from src.models.fekolorn import FekolornLM
    from src.models.llama import CausalLM

    t0 = time.time()
    summary = []
    for size in a.sizes.split(","):
        z = SIZES[size]
        if not a.skip_kernels:
            summary += kernels(z, a, size)
        if a.skip_serving:
            continue
        if "fekolorn" in a.models.split(","):
            summary.append(serve(FekolornLM(fekolorn_arch(z), "cuda:0", seed=1, init_std=0.02), a, "fekolorn", size))
        if "llama" in a.models.split(","):
            summary.append(serve(CausalLM(llama_arch(z), "cuda:0", seed=1), a, "llama", size))
    print(json.dumps({"bench": "fekolorn_compare_summary", "seconds": round(time.time() - t0, 1), "rows": summary}),
          flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
