"""
Fekolorn on the serving engine against the plain float64 oracle (tests/fekolorn_oracle.py).

Every test makes its own small configuration and random weights, writes them as a checkpoint directory, loads it
through ``LLMEngine.from_pretrained`` (registry -> model class -> loader) and steps it with
``LLMEngine.replay_step`` (scheduler, block manager with state slots, runner, kernels). The CPU cases run the
engine's control flow on the plain-PyTorch op semantics; the ``gpu`` cases run the HIP kernels. Structural faults
(a window one token off, a lost state, a missing sink) are far above the fp32 tolerance, so those cases run in
fp32; bf16 cases check the served precision.
"""

import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fekolorn_oracle as orc  # noqa: E402

F64 = torch.float64
CPU = pytest.param("cpu", id="cpu")
GPU = pytest.param("cuda:0", marks=pytest.mark.gpu, id="gpu")
DEVICES = [CPU, GPU]
TOL = {torch.float32: 3e-4, torch.bfloat16: 6e-2}


def _need(device):
    if device != "cpu":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        from src.ops import mix

        assert mix.mix_available(), "HIP extension src/_Cmix not loaded"


def save_checkpoint(path, config, weights):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))


def make_engine(tmp_path, config, weights, device, dtype, max_tokens=512, max_seqs=4, block_size=16, name="ckpt",
                **cfg_kw):
    from src.config import EngineConfig
    from src.engine import LLMEngine

    path = str(tmp_path / name)
    save_checkpoint(path, config, weights)
    nb = (max_tokens + block_size - 1) // block_size
    kw = dict(max_num_seqs=max_seqs, max_num_batched_tokens=nb * block_size, block_size=block_size, num_kv_blocks=nb,
              enable_prefix_caching=False, use_cuda_graph=False, preemption_mode="recompute", tuned_gemm_table=False,
              decode_window=1)
    kw.update(cfg_kw)
    return LLMEngine.from_pretrained(path, device=device, cfg=EngineConfig(**kw), max_model_len=nb * block_size,
                                     capture=False, dtype=dtype)


def row_errs(got, want):
    """Per row: rms of the logit difference (mean taken off) over the rms of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def rel_err(got, want):
    return float(row_errs(got, want).max())


def tokens_for(config, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, config["vocab"], (n,), generator=g).tolist()


def replay(eng, steps):
    """steps: list of lists of (request id, tokens, wanted places[, ends]). Returns {rid: {position: logits row}}."""
    got, at = {}, {}
    for step in steps:
        entries, end = [], []
        for e in step:
            rid, toks, want = e[:3]
            entries.append((rid, toks, want))
            if len(e) > 3 and e[3]:
                end.append(rid)
        logits = eng.replay_step(entries, end)
        r = 0
        for rid, toks, want in entries:
            base = at.get(rid, 0)
            for w in want:
                got.setdefault(rid, {})[base + w] = logits[r]
                r += 1
            at[rid] = base + len(toks)
        for rid in end:
            at.pop(rid, None)
        assert r == logits.shape[0]
    return got


def cut(rid, toks, sizes, end=True):
    """One request alone, cut into portions of the given sizes (the rest one token at a time)."""
    steps, lo = [], 0
    sizes = list(sizes)
    while lo < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - lo)
        hi = lo + n
        steps.append([(rid, toks[lo:hi], list(range(n)), end and hi == len(toks))])
        lo = hi
    return steps


def check_against_oracle(got, weights, config, toks, tol):
    want = orc.forward(toks, weights, config)
    pos = sorted(got)
    g = torch.stack([got[p] for p in pos])
    assert torch.isfinite(g).all()
    e = row_errs(g, want[pos])
    if tol >= 1e-2:
        # bf16 on models this narrow: the typical row is held to the tolerance and no row may be far off (a
        # structural fault moves rows by O(1))
        assert float(e.median()) < tol / 2 and float(e.max()) < 4 * tol, f"median {float(e.median()):.3e} max {float(e.max()):.3e}"
    else:
        assert float(e.max()) < tol, f"relative error {float(e.max()):.3e} >= {tol}"


def std_config(**kw):
    """parallel, attention, attention (values mixed with the first one's), parallel without feed-forward."""
    return orc.make_config([("parallel", orc.parallel_cfg(), 24), ("attention", orc.attn_cfg(), 40),
                            ("attention", orc.attn_cfg(window=9), None), ("parallel", orc.parallel_cfg(conv=2), 24)],
                           **kw)


CONFIGS = {
    "std": lambda: std_config(),
    # one stream / no hyper-connection tensors, no bigram, attention first, feed-forward missing in places
    "plain": lambda: orc.make_config([("attention", orc.attn_cfg(heads=2, kv_heads=2, dim=8, vdim=8, window=0,
                                                                bias_max=16, v_mix=False), None),
                                      ("parallel", orc.parallel_cfg(heads=2, kv_heads=1, dim=8, vdim=12, rot_dims=8,
                                                                    r_heads=1, r_kv_heads=1, r_dim=4, r_vdim=4,
                                                                    conv=1), 16)],
                                     width=16, vocab=23, streams=0, buckets=0, embed_scale=1.0),
    # four streams, odd sizes, taps 4, heads == kv_heads on one side, kv_heads 1 on the other
    "odd": lambda: orc.make_config([("parallel", orc.parallel_cfg(heads=3, kv_heads=3, dim=10, vdim=6, rot_dims=4,
                                                                  rot_base=17.0, r_heads=4, r_kv_heads=2, r_dim=6,
                                                                  r_vdim=10, conv=4), 20),
                                    ("attention", orc.attn_cfg(heads=6, kv_heads=1, dim=12, vdim=20, window=5,
                                                               bias_max=30.0), 28),
                                    ("attention", orc.attn_cfg(heads=2, kv_heads=1, dim=12, vdim=20, window=17,
                                                               bias_max=7.5, v_mix=True), None)],
                                   width=24, vocab=31, streams=4, buckets=11, eps=1e-3),
    "one_stream": lambda: orc.make_config([("parallel", orc.parallel_cfg(), 24)], streams=1),
}


# ------------------------------------------------------------------------------------------- mechanisms
def test_distance_buckets():
    from src.ops import seq

    for B, D, window in ((32, 120.0, 136), (12, 10.0, 0), (8, 100.0, 40), (9, 7.5, 0), (2, 5.0, 0)):
        rel = torch.arange(B * 3, dtype=torch.float32).view(B, 3)
        tab = seq.distance_bias_table(rel, D, window)
        top = window if window else 400
        for n in range(top):
            assert torch.equal(tab[min(n, tab.shape[0] - 1)], rel[orc.distance_bucket(n, B, D)]), (B, D, n)


@pytest.mark.parametrize("device", DEVICES)
def test_embedding_with_previous_token_state(device):
    _need(device)
    from src.ops import seq

    g = torch.Generator().manual_seed(3)
    V, W, buckets = 19, 12, 7
    cfg = {"embedding": {"scale": 0.3, "bigram": {"buckets": buckets, "mul_prev": 5, "mul_cur": 11}}}
    w = {"embed": torch.randn(V, W, generator=g), "bigram": torch.randn(buckets + 1, W, generator=g)}
    a, b = tokens_for({"vocab": V}, 9, 1), tokens_for({"vocab": V}, 5, 2)
    wa, wb = orc.embedding(a, {k: v.double() for k, v in w.items()}, cfg), orc.embedding(b, {k: v.double() for k, v in w.items()}, cfg)
    prev = torch.full((4,), 17, dtype=torch.int64, device=device)   # stale content of the slots
    dw = {k: v.to(device) for k, v in w.items()}

    def step(ids, pos, cu, slots):
        ids_t = torch.tensor(ids, device=device)
        rag = seq.Ragged(torch.tensor(pos, device=device), None if cu is None else torch.tensor(cu, dtype=torch.int32, device=device),
                         torch.tensor(slots, dtype=torch.int32, device=device))
        x = seq.embed_hash(ids_t, dw["embed"], dw["bigram"], rag, prev, 0.3, buckets, 5, 11, 3)
        seq.store_last_token(prev, ids_t, rag)
        assert torch.equal(x[:, 0], x[:, 1]) and torch.equal(x[:, 0], x[:, 2])
        return x[:, 0].cpu().double()

    # a: 4 tokens, b: 2 tokens; then a: 5 more beside one of b; then single rows (decode form)
    x = step(a[:4] + b[:2], [0, 1, 2, 3, 0, 1], [0, 4, 6], [2, 0])
    assert torch.allclose(x, torch.cat([wa[:4], wb[:2]]), atol=1e-5)
    x = step(a[4:9] + b[2:3], [4, 5, 6, 7, 8, 2], [0, 5, 6], [2, 0])
    assert torch.allclose(x, torch.cat([wa[4:9], wb[2:3]]), atol=1e-5)
    x = step(b[3:4], [3], None, [0])
    assert torch.allclose(x, wb[3:4], atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,W", [(1, 37), (3, 37), (8, 37), (3, 64), (2, 8448)])
def test_stream_mixing_and_norm(device, dtype, S, W):
    """Narrow rows (scalar accesses), rows of a multiple of 4 columns (16-byte accesses), and rows wider than what
    the kernel keeps in registers between its two passes."""
    _need(device)
    from src.ops import seq

    g = torch.Generator().manual_seed(S)
    T, eps = 5, 1e-4
    xs = torch.randn(T, S, W, generator=g)
    y1, y2 = torch.randn(T, W, generator=g).to(dtype), torch.randn(T, W, generator=g).to(dtype)
    mixw, outw, inw = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    gain = torch.tensor([1.3])
    y = 0.6 * y1.double() + 0.9 * y2.double()
    new = torch.einsum("sq,tsw->tqw", mixw.double(), xs.double()) + outw.double()[None, :, None] * y[:, None, :]
    u = torch.einsum("s,tsw->tw", inw.double(), new)
    want_h = orc.rms(u, eps) * 1.3
    d = lambda t: t.to(device)  # noqa: E731
    xs_d = d(xs.clone())
    h = seq.stream_mix_norm(xs_d, d(y1), d(y2), 0.6, 0.9, d(mixw), d(outw), d(inw), d(gain), eps, dtype)
    assert torch.allclose(xs_d.cpu().double(), new, atol=1e-4)
    assert torch.allclose(h.cpu().double(), want_h, atol=2e-2 if dtype == torch.bfloat16 else 1e-4)
    # no update, plain sum (the final norm); and the ordinary residual sum of one stream
    h2 = seq.stream_mix_norm(xs_d, None, None, 1.0, 1.0, None, None, None, d(gain), eps, torch.float32)
    assert torch.allclose(h2.cpu().double(), orc.rms(new.sum(1), eps) * 1.3, atol=1e-4)
    if S == 1:
        x1 = d(xs.clone())
        seq.stream_mix_norm(x1, d(y1), None, 1.0, 1.0, None, None, None, None, eps, None)
        assert torch.allclose(x1.cpu().double(), xs.double() + y1.double()[:, None, :], atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [7, 300])
def test_polynomial_norm_activation(device, n):
    _need(device)
    from src.ops import seq

    g = torch.Generator().manual_seed(n)
    z = torch.randn(4, n, generator=g) * 2
    coef = torch.tensor([0.7, -0.3, 0.2, 0.05])
    zz = z.double()
    want = 0.7 * orc.rms(zz, 1e-5) - 0.3 * orc.rms(zz ** 2, 1e-5) + 0.2 * orc.rms(zz ** 3, 1e-5) + 0.05
    got = seq.poly_norm_act(z.to(device), coef.to(device), 1e-5)
    assert torch.allclose(got.cpu().double(), want, atol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [64, 4096, 8200])
def test_polynomial_norm_activation_bf16_rows(device, n):
    """bf16 rows: 16-byte accesses with the row kept in registers, and rows too wide for that."""
    _need(device)
    from src.ops import seq

    g = torch.Generator().manual_seed(n)
    z = (torch.randn(3, n, generator=g) * 1.5).bfloat16()
    coef = torch.tensor([0.7, -0.3, 0.2, 0.05])
    zz = z.double()
    want = 0.7 * orc.rms(zz, 1e-5) - 0.3 * orc.rms(zz ** 2, 1e-5) + 0.2 * orc.rms(zz ** 3, 1e-5) + 0.05
    got = seq.poly_norm_act(z.to(device), coef.to(device), 1e-5)
    assert got.dtype == torch.bfloat16
    assert float((got.cpu().double() - want).abs().max()) < 2e-2 * max(1.0, float(want.abs().max()))


def _delta_weights(H, G, d, dv, taps, W, seed):
    cfg = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": taps}
    full = orc.make_config([("parallel", dict(orc.parallel_cfg(), right=cfg), None)], width=W)
    w = orc.make_weights(full, seed=seed)
    return cfg, {k[len("l0.mix.right."):]: v.double() for k, v in w.items() if k.startswith("l0.mix.right.")}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", [(2, 1, 8, 16, 3), (4, 4, 5, 7, 4), (3, 1, 40, 70, 1), (1, 1, 64, 128, 2),
                                   (2, 1, 128, 128, 4), (1, 1, 200, 256, 2)])
def test_gated_delta_rule_in_portions_and_slots(device, shape):
    """The recurrence with its convolution, cut into portions (down to one token), two sequences sharing steps, in
    slots that held another sequence before."""
    _need(device)
    from src.ops import seq

    H, G, d, dv, taps = shape
    W, eps = 12, 1e-5
    cfg, w = _delta_weights(H, G, d, dv, taps, W, seed=sum(shape))
    g = torch.Generator().manual_seed(5)
    hs = {"a": torch.randn(11, W, generator=g).double(), "b": torch.randn(6, W, generator=g).double()}
    C = 2 * G * d + H * dv
    f = lambda t: t.float().to(device)  # noqa: E731
    conv_w = f(torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]], 0))
    w_in = torch.cat([w["q"], w["k"], w["v"], w["b"], w["a"], w["g"]], 0)
    state = {"delta": torch.randn(3, H, d, dv, generator=g).to(device), "conv": torch.randn(3, taps - 1, C, generator=g).to(device)}
    got = {k: [] for k in hs}
    at = {k: 0 for k in hs}
    slot = {"a": 2, "b": 0}
    for step in ([("a", 4), ("b", 1)], [("b", 2)], [("a", 1), ("b", 1)], [("a", 1)], [("a", 5), ("b", 2)]):
        rows, pos, cu, slots = [], [], [0], []
        for k, n in step:
            rows.append(hs[k][at[k]: at[k] + n])
            pos += list(range(at[k], at[k] + n))
            cu.append(cu[-1] + n)
            slots.append(slot[k])
        single = all(n == 1 for _, n in step)
        p = (torch.cat(rows) @ w_in.T).float().to(device)
        rag = seq.Ragged(torch.tensor(pos, device=device), None if single else torch.tensor(cu, dtype=torch.int32, device=device),
                         torch.tensor(slots, dtype=torch.int32, device=device))
        x, b, a, gt = p[:, :C], p[:, C: C + H], p[:, C + H: C + 2 * H], p[:, C + 2 * H:]
        qkv32, bg = seq.delta_prep(x, b, a, conv_w, state["conv"], f(w["A_log"]), f(w["dt_bias"]), H, G, d, dv, rag)
        if not single:   # the tap-major weights (16-byte path of bf16 prompt steps) give the same as the plain ones
            xb, bb, ab = x.bfloat16(), b.bfloat16(), a.bfloat16()
            pad = xb.new_zeros(xb.shape[0], (-(C + 2 * H)) % 8)   # a row stride that allows 16-byte loads
            pb = torch.cat([xb, bb, ab, pad], 1)
            xb, bb, ab = pb[:, :C], pb[:, C: C + H], pb[:, C + H: C + 2 * H]
            ref32, _ = seq.delta_prep(xb, bb, ab, conv_w, state["conv"], f(w["A_log"]), f(w["dt_bias"]), H, G, d, dv, rag)
            got32, _ = seq.delta_prep(xb, bb, ab, conv_w, state["conv"], f(w["A_log"]), f(w["dt_bias"]), H, G, d, dv, rag,
                                      conv_wt=conv_w.t().contiguous())
            assert torch.allclose(ref32, got32, atol=1e-6), float((ref32 - got32).abs().max())
        seq.conv_state_update(state["conv"], x, H, G, d, dv, rag)
        o = seq.gated_delta(qkv32, bg, gt, f(w["norm"]), eps, state["delta"], H, G, d, dv, rag).cpu().double()
        r = 0
        for k, n in step:
            got[k].append(o[r: r + n])
            r += n
            at[k] += n
    for k in hs:
        full = orc.gated_delta_rule(hs[k], {"." + n: t for n, t in w.items()}, ".", cfg, eps)
        assert torch.allclose(torch.cat(got[k]) @ w["o"].T, full, atol=2e-4), k


def _paged(device, dtype, n_blocks, bs, width, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n_blocks, bs, width, generator=g) * 3).to(dtype).to(device)   # stale rows everywhere


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ["rotary", "biased", "wide", "mc_rotary", "mc_biased", "served_rotary", "served_biased", "mc_far_bias"])
def test_attention_ops_with_standout_keys(device, dtype, case):
    """qkv_prep + sink_attn over scattered pages, prompt portion and single decode rows: one key far back, one on a
    page border, and the keys just inside and just outside the window are made to stand out (their scores lead by
    a wide margin), so a mask that is one token off or a lost page changes the output by O(1)."""
    _need(device)
    from src.ops import seq

    eps = 1e-5
    if case == "rotary":
        H, G, d, dv, window, rot, bias_max = 4, 2, 16, 8, 0, 8, 0
    elif case == "biased":
        H, G, d, dv, window, rot, bias_max = 6, 2, 12, 20, 21, 0, 15.0
    elif case == "mc_rotary":     # shapes the matrix-core kernel takes in bf16 (forced there: impl 2)
        H, G, d, dv, window, rot, bias_max = 8, 2, 80, 32, 0, 48, 0
    elif case == "mc_biased":
        H, G, d, dv, window, rot, bias_max = 6, 2, 32, 96, 37, 0, 15.0
    elif case == "mc_far_bias":    # a window several times the bias table's reach: whole tiles share its last row
        H, G, d, dv, window, rot, bias_max = 4, 2, 32, 32, 80, 0, 6.0
    elif case == "served_rotary":  # default dispatch at a served shape: 8 query heads on one key/value head
        H, G, d, dv, window, rot, bias_max = 8, 1, 128, 128, 0, 64, 0
    elif case == "served_biased":  # default dispatch, one query head per key/value head
        H, G, d, dv, window, rot, bias_max = 2, 2, 64, 32, 50, 0, 15.0
    else:
        H, G, d, dv, window, rot, bias_max = 2, 1, 96, 160, 40, 0, 0
    impl = 2 if case.startswith("mc_") and dtype == torch.bfloat16 and device != "cpu" else 0
    rotary, biased = case.endswith("rotary"), case.endswith("biased") or case.endswith("bias")
    T, bs = 90, 8
    g = torch.Generator().manual_seed(len(case))
    q = torch.randn(T, H, d, generator=g) * 0.3
    k = torch.randn(T, G, d, generator=g) * 0.3
    v = torch.randn(T, G, dv, generator=g)
    # the last query, and one mid-prompt, point at chosen keys
    marks = {T - 1: [T - 1 - (window - 1 if window else 80), 63, 64] + ([T - 1 - window] if window else []),
             50: [50 - (window - 1 if window else 47), 48] + ([50 - window] if window else [])}
    for qi, keys in marks.items():
        for n, kj in enumerate(keys):
            dirn = torch.randn(d, generator=g)
            dirn = dirn / dirn.norm()
            q[qi, :, :] += 6.0 * dirn
            k[kj, :, :] += (3.0 + n) * dirn
    sink = torch.randn(H, generator=g)
    scale = d ** -0.5
    rel = torch.randn(10, H, generator=g) if bias_max else None
    qn = (torch.rand(H * d, generator=g) + 0.5) if biased else None
    kn = (torch.rand(G * d, generator=g) + 0.5) if biased else None
    v_first = torch.randn(T, G * dv, generator=g) if biased else None
    lam = torch.tensor([0.35]) if biased else None
    qd, kd, vd = q.to(dtype).double(), k.to(dtype).double(), v.to(dtype).double()
    # oracle
    oq, ok_, ov = qd, kd, vd
    if qn is not None:
        oq = (orc.rms(qd.reshape(T, -1), eps) * qn.double()).view(T, H, d)
        ok_ = (orc.rms(kd.reshape(T, -1), eps) * kn.double()).view(T, G, d)
        ov = ((1 - 0.35) * vd.reshape(T, -1) + 0.35 * v_first.to(dtype).double()).view(T, G, dv)
    if rot:
        oq, ok_ = orc.rotate_half(oq, rot, 50.0), orc.rotate_half(ok_, rot, 50.0)
    if rotary:
        ov = orc.rms(ov, eps)
    bias = None
    if rel is not None:
        bias = torch.zeros(T, T, H, dtype=F64)
        for i in range(T):
            for j in range(i + 1):
                bias[i, j] = rel[orc.distance_bucket(i - j, 10, bias_max)].double()
    want = orc.sink_attention(oq, ok_, ov, scale, sink.double(), window or None, bias).reshape(T, H * dv)
    # engine ops over scattered pages: a 70-token portion, then single rows
    nblk = (T + bs - 1) // bs
    perm = torch.randperm(nblk + 5, generator=g)[:nblk].tolist()
    cache = _paged(device, dtype, nblk + 5, bs, G * (d + dv), 3)
    bt = torch.tensor([perm], dtype=torch.int32, device=device)
    dev = lambda t: None if t is None else t.to(device)  # noqa: E731
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).to(dtype).to(device)
    nq, nk = H * d, G * d
    inv_freq = torch.tensor([50.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=device) if rot else None
    table = seq.distance_bias_table(rel, bias_max, window).to(device) if rel is not None else None
    outs = []
    for lo, hi in [(0, 70)] + [(t, t + 1) for t in range(70, T)]:
        pos = torch.arange(lo, hi, device=device)
        slots = torch.tensor([perm[t // bs] * bs + t % bs for t in range(lo, hi)], device=device)
        p = proj[lo:hi]
        qr = seq.qkv_prep(p[:, :nq], p[:, nq: nq + nk], p[:, nq + nk:], cache, H, G, d, dv, pos, slots, eps,
                          q_norm=dev(qn), k_norm=dev(kn), rot_dims=rot, inv_freq=inv_freq, v_unit=rotary,
                          v_lambda=dev(lam), v_first=None if v_first is None else v_first[lo:hi].to(dtype).to(device))
        single = hi - lo == 1
        o = seq.sink_attn(qr, cache, bt, None if single else torch.tensor([0, hi - lo], dtype=torch.int32, device=device),
                          torch.tensor([hi], dtype=torch.int32, device=device), pos, sink.to(device), table,
                          hi - lo, H, G, d, dv, window, scale, impl=impl)
        outs.append(o.cpu().double())
    got = torch.cat(outs)
    tol = 3e-4 if dtype == torch.float32 else 4e-2
    assert float((got - want).abs().max()) < tol * max(1.0, float(want.abs().max()))
    # the marked keys matter: dropping the one just inside the window moves the oracle's output by far more
    if window:
        other = orc.sink_attention(oq, ok_, ov, scale, sink.double(), window - 1, bias).reshape(T, H * dv)
        assert float((other[T - 1] - want[T - 1]).abs().max()) > 0.05
        other = orc.sink_attention(oq, ok_, ov, scale, sink.double(), window + 1, bias).reshape(T, H * dv)
        assert float((other[T - 1] - want[T - 1]).abs().max()) > 0.05


# ------------------------------------------------------------------------------------------- whole model
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt(tmp_path, device, dtype, name):
    _need(device)
    cfg = CONFIGS[name]()
    wts = orc.make_weights(cfg, seed=len(name), rel_rows=12 if name != "odd" else 9)
    eng = make_engine(tmp_path, cfg, wts, device, dtype)
    toks = tokens_for(cfg, 45, 3)
    got = replay(eng, cut("r", toks, [45]))["r"]
    check_against_oracle(got, wts, cfg, toks, TOL[dtype])
    assert eng.blocks.num_available() == eng.blocks.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_layer_outputs(tmp_path, device):
    """The sum of the streams after every layer, against the oracle's."""
    _need(device)
    from src.engine.scheduler import PrefillChunk

    cfg = std_config()
    wts = orc.make_weights(cfg, seed=2)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    toks = tokens_for(cfg, 20, 4)
    want = []
    orc.forward(toks, wts, cfg, want)
    seen = []
    model = eng.model
    orig = model.forward
    model.forward = lambda *a, **k: orig(*a, layer_hook=lambda i, r: seen.append(r.cpu().double()), **k)
    replay(eng, cut("r", toks, [20]))
    assert len(seen) == len(want)
    for i, (a, b) in enumerate(zip(seen, want)):
        assert torch.allclose(a, b, atol=2e-4 * float(b.abs().max())), i


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_request(tmp_path, device):
    _need(device)
    cfg = std_config()
    wts = orc.make_weights(cfg, seed=5)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    for n in (1, 2, 3):
        toks = tokens_for(cfg, n, n)
        check_against_oracle(replay(eng, cut(f"r{n}", toks, [n]))[f"r{n}"], wts, cfg, toks, TOL[torch.float32])
    toks = tokens_for(cfg, 4, 9)
    check_against_oracle(replay(eng, cut("d", toks, [1]))["d"], wts, cfg, toks, TOL[torch.float32])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 2, 16, 2, 7], [1], [30, 2], [15, 16, 17]])
@pytest.mark.parametrize("name", ["std", "odd"])
def test_portions_and_decode_equal_whole(tmp_path, device, sizes, name):
    """Portions of several sizes down to two tokens (cut inside pages, windows and convolution tails), the rest one
    token at a time."""
    _need(device)
    cfg = CONFIGS[name]()
    wts = orc.make_weights(cfg, seed=7)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    toks = tokens_for(cfg, 58, 11)
    got = replay(eng, cut("r", toks, sizes))["r"]
    assert sorted(got) == list(range(58))
    check_against_oracle(got, wts, cfg, toks, TOL[torch.float32])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_bf16(tmp_path, device):
    _need(device)
    cfg = std_config()
    wts = orc.make_weights(cfg, seed=8)
    eng = make_engine(tmp_path, cfg, wts, device, torch.bfloat16)
    toks = tokens_for(cfg, 120, 12)
    got = replay(eng, cut("r", toks, [5]))["r"]
    check_against_oracle(got, wts, cfg, toks, TOL[torch.bfloat16])


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone_and_slots_are_reused(tmp_path, device):
    """Four unequal requests live at once in a pool too small for all six, requests sitting out steps; the blocks
    and the state slots of finished requests go to new ones, whose first tokens must not see what was left there."""
    _need(device)
    cfg = std_config()
    wts = orc.make_weights(cfg, seed=9)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32, max_tokens=160, max_seqs=4, block_size=8)
    T = {"a": 40, "b": 7, "c": 50, "d": 21, "e": 33, "f": 12}
    toks = {k: tokens_for(cfg, n, ord(k)) for k, n in T.items()}
    at = {k: 0 for k in T}

    def ent(k, n):
        lo = at[k]
        hi = min(lo + n, T[k])
        at[k] = hi
        return (k, toks[k][lo:hi], list(range(hi - lo)), hi == T[k])

    steps = [[ent("a", 10), ent("b", 3)],
             [ent("a", 1), ent("b", 2), ent("c", 17)],
             [ent("b", 2), ent("c", 2), ent("d", 21)],          # b and d end: two slots and their blocks free
             [ent("a", 9), ent("c", 1), ent("e", 2), ent("f", 5)],   # e and f take them
             [ent("a", 1), ent("c", 1), ent("e", 1), ent("f", 1)],   # a step of single tokens (decode form)
             [ent("a", 19), ent("e", 30), ent("f", 6)],
             [ent("c", 29)]]
    slots_seen = {}
    got = {}
    orig = eng.scheduler.schedule_forced

    def spy(plan):
        out = orig(plan)
        for c in out.prefill:
            slots_seen.setdefault(c.seq.request_id, c.seq.state_slot)
        return out

    eng.scheduler.schedule_forced = spy
    got = replay(eng, steps)
    assert all(at[k] == T[k] for k in T)
    assert {slots_seen["e"], slots_seen["f"]} == {slots_seen["b"], slots_seen["d"]}, "freed slots were not reused"
    for k in T:
        assert sorted(got[k]) == list(range(T[k]))
        check_against_oracle(got[k], wts, cfg, toks[k], TOL[torch.float32])
    assert eng.blocks.num_available() == eng.blocks.num_blocks
    assert sorted(eng.blocks._free_slots) == [0, 1, 2, 3]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_medium_model_long_prompts_in_mixed_steps(tmp_path, device, dtype):
    """A model at the scale of a real small one (width 192, head dims 48 - 96, window 100, 24 distance buckets,
    attention first): prompts several windows and pages long, run as a whole, in portions, token by token and
    beside each other with slots reused. bf16 on the GPU takes the matrix-core kernel where the shapes allow
    (dim 64 / vdim 96, dim 80), the FMA kernel elsewhere (vdim 48) and the decode-step kernel for single tokens."""
    _need(device)
    att = orc.attn_cfg(heads=6, kv_heads=2, dim=64, vdim=96, window=100, bias_max=70.0)
    par = orc.parallel_cfg(heads=6, kv_heads=3, dim=80, vdim=48, rot_dims=40, rot_base=5000.0, r_heads=6, r_kv_heads=2,
                           r_dim=48, r_vdim=32, conv=3, left_scale=1.2, right_scale=0.5)
    cfg = orc.make_config([("attention", att, 320), ("parallel", par, None), ("attention", att, 256)], width=192,
                          vocab=211, streams=2, buckets=97)
    wts = orc.make_weights(cfg, seed=33, rel_rows=24)
    eng = make_engine(tmp_path, cfg, wts, device, dtype, max_tokens=448, max_seqs=3, block_size=32)
    a, b, c = tokens_for(cfg, 230, 1), tokens_for(cfg, 150, 2), tokens_for(cfg, 40, 3)
    at = {"a": 0, "b": 0, "c": 0}
    toks = {"a": a, "b": b, "c": c}

    def ent(k, n, want=None):
        lo = at[k]
        hi = min(lo + n, len(toks[k]))
        at[k] = hi
        w = list(range(hi - lo)) if want is None else want
        return (k, toks[k][lo:hi], w, hi == len(toks[k]))

    steps = [[ent("a", 130)], [ent("a", 1), ent("b", 97)], [ent("a", 1), ent("b", 2)], [ent("a", 1), ent("b", 1)],
             [ent("a", 64), ent("b", 50), ent("c", 33)], [ent("a", 33), ent("c", 7)]]
    got = replay(eng, steps)
    for k in ("a", "b", "c"):
        assert at[k] == len(toks[k])
        check_against_oracle(got[k], wts, cfg, toks[k], TOL[dtype])
    assert eng.blocks.num_available() == eng.blocks.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_window_edges_sink_state_and_far_keys_show_in_logits(tmp_path, device):
    """The engine agrees with the oracle where the oracle itself is sensitive: a window one token longer or shorter,
    no sink, no bias, a decay of one, a convolution without its oldest tap and a far key all move the oracle's
    logits by far more than the tolerance."""
    _need(device)
    cfg = orc.make_config([("parallel", orc.parallel_cfg(), 24), ("attention", orc.attn_cfg(window=12, bias_max=9), 24)])
    wts = orc.make_weights(cfg, seed=10)
    wts["l0.mix.left.sink"] = (wts["l0.mix.left.sink"].float() + 4.0).bfloat16()   # a sink that outweighs many keys
    toks = tokens_for(cfg, 70, 13)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    got = replay(eng, cut("r", toks, [33, 2, 20]))["r"]
    check_against_oracle(got, wts, cfg, toks, TOL[torch.float32])
    want = orc.forward(toks, wts, cfg)
    tol = 30 * TOL[torch.float32]

    def moved(change_cfg=None, change_w=None):
        c2 = json.loads(json.dumps(cfg))
        w2 = dict(wts)
        if change_cfg:
            change_cfg(c2)
        if change_w:
            change_w(w2)
        return rel_err(orc.forward(toks, w2, c2)[40:], want[40:])

    assert moved(lambda c: c["layers"][1]["mixer"]["mask"].update(size=13)) > tol
    assert moved(lambda c: c["layers"][1]["mixer"]["mask"].update(size=11)) > tol
    assert moved(change_w=lambda w: w.update({"l1.mix.sink": w["l1.mix.sink"] - 30})) > tol
    assert moved(change_w=lambda w: w.update({"l0.mix.left.sink": w["l0.mix.left.sink"] - 30})) > tol
    assert moved(change_w=lambda w: w.update({"l1.mix.rel": torch.zeros_like(w["l1.mix.rel"])})) > tol
    assert moved(change_w=lambda w: w.update({"l0.mix.right.A_log": w["l0.mix.right.A_log"] - 30})) > tol
    assert moved(change_w=lambda w: w.update({"l0.mix.right.q.conv": torch.cat(
        [torch.zeros_like(w["l0.mix.right.q.conv"][:, :1]), w["l0.mix.right.q.conv"][:, 1:]], 1)})) > tol
    assert moved(lambda c: c["embedding"]["bigram"].update(mul_prev=6)) > tol

    # the first tokens matter to the last ones (the causal attention and the recurrence reach back to them)
    short = orc.forward(toks[25:], wts, cfg)
    assert rel_err(short[-10:], want[-10:]) > tol


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_engine(tmp_path, device):
    """LLMEngine.generate (scheduler, continuous batching, paged cache, state slots, sampling) on prompts of unequal
    length, more prompts than sequence slots: every generated token is the oracle's argmax given the tokens before
    it, or within the served precision of it."""
    _need(device)
    from src.preproc import SamplingParams

    cfg = std_config(vocab=48)
    wts = orc.make_weights(cfg, seed=18)
    eng = make_engine(tmp_path, cfg, wts, device, torch.bfloat16, max_tokens=512, max_seqs=3, mixed_batching="auto")
    eng.eos_token_id = None
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 23, 40, 9, 17)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10))
    assert [len(o) for o in outs] == [10] * 5
    for p, o in zip(prompts, outs):
        lg = orc.forward(p + o, wts, cfg)
        for i, tok in enumerate(o):
            row = lg[len(p) + i - 1]
            spread = float(row.max() - row.min())
            assert float(row.max() - row[tok]) <= 0.05 * spread, (i, tok, int(row.argmax()))
    assert eng.blocks.num_available() == eng.blocks.num_blocks
    assert len(eng.blocks._free_slots) == 3


def test_preempted_sequence_recomputes_its_state(tmp_path):
    """A pool too small for both sequences' generations: the scheduler preempts one (recompute), which re-prefills
    from position 0 into whatever slot it gets and still generates the oracle's tokens."""
    from src.preproc import SamplingParams

    cfg = std_config(vocab=48)
    wts = orc.make_weights(cfg, seed=19)
    eng = make_engine(tmp_path, cfg, wts, "cpu", torch.float32, max_tokens=64, max_seqs=2, block_size=8)
    eng.eos_token_id = None
    prompts = [tokens_for(cfg, 20, 1), tokens_for(cfg, 18, 2)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=20))
    assert eng.scheduler.num_preemptions >= 1
    for p, o in zip(prompts, outs):
        assert len(o) == 20
        lg = orc.forward(p + o, wts, cfg)
        for i, tok in enumerate(o):
            row = lg[len(p) + i - 1]
            assert float(row.max() - row[tok]) <= 1e-3 * float(row.max() - row.min()), (i, tok, int(row.argmax()))


def test_registry_config_roundtrip_and_options(tmp_path):
    from src.models.fekolorn import FekolornLM
    from src.models.registry import family_of, resolve

    cfg = CONFIGS["odd"]()
    save_checkpoint(str(tmp_path / "m"), cfg, orc.make_weights(cfg, rel_rows=9))
    assert family_of(str(tmp_path / "m")) == "fekolorn"
    _, arch, cls = resolve(str(tmp_path / "m"))
    assert cls is FekolornLM and arch.streams == 4 and arch.layers[1].mixer.window == 5
    assert arch.layers[0].mixer.right.conv == 4 and arch.layers[2].mixer.v_mix and arch.bigram_buckets == 11
    assert arch.to_config()["layers"] == cfg["layers"]
    # a model's own save() loads back to the same logits
    model = FekolornLM(arch, "cpu", dtype=torch.float32, seed=3)
    model.save(str(tmp_path / "s"))
    from src.config import EngineConfig
    from src.engine import LLMEngine

    kw = dict(max_num_seqs=2, max_num_batched_tokens=64, block_size=16, num_kv_blocks=4, enable_prefix_caching=True,
              use_cuda_graph=False, tuned_gemm_table=False)
    eng = LLMEngine.from_pretrained(str(tmp_path / "s"), device="cpu", cfg=EngineConfig(**kw), max_model_len=64,
                                    capture=False, dtype=torch.float32)
    assert not eng.blocks.prefix_caching, "a cached prefix does not hold the recurrent state after it"
    from safetensors.torch import load_file

    wts = load_file(str(tmp_path / "s" / "model.safetensors"))
    toks = tokens_for(cfg, 20, 1)
    check_against_oracle(replay(eng, cut("r", toks, [20]))["r"], wts, arch.to_config(), toks, TOL[torch.float32])


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run end to end on the CPU: steps on stdin, logits files and 'done' lines out."""
    import subprocess

    import numpy as np

    cfg = std_config()
    wts = orc.make_weights(cfg, seed=19)
    save_checkpoint(str(tmp_path / "m"), cfg, wts)
    toks = tokens_for(cfg, 40, 7)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[30:32], "want": []},
                                     {"id": "y", "tokens": toks[:3], "want": [2]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[32:40], "want": [7]}], "end": ["x"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path / "m"),
                        "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "128", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = orc.forward(toks, wts, cfg)
    a = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1))
    assert rel_err(a, want[[0, 29]]) < TOL[torch.float32]
    b = torch.from_numpy(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4").reshape(1, -1))
    assert rel_err(b, orc.forward(toks[:3], wts, cfg)[[2]]) < TOL[torch.float32]
    c = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(1, -1))
    assert rel_err(c, want[[39]]) < TOL[torch.float32]


@pytest.mark.gpu
def test_generation_with_decode_graphs(tmp_path):
    """Served configuration at sizes the matrix-core attention takes (dim 64 / 32, vdim 64): decode steps replayed
    from captured hipGraphs in multi-step windows (padded rows write the spare state slot). Every token is checked
    against the oracle, and the same tokens teacher-forced give the oracle's logits."""
    _need("cuda:0")
    from src.preproc import SamplingParams

    par = orc.parallel_cfg(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, r_heads=4, r_kv_heads=2, r_dim=32,
                           r_vdim=64, conv=4)
    att = orc.attn_cfg(heads=4, kv_heads=1, dim=32, vdim=64, window=24, bias_max=20)
    cfg = orc.make_config([("parallel", par, 256), ("attention", att, 256), ("attention", att, None)], vocab=128,
                          width=256, streams=3)
    wts = orc.make_weights(cfg, seed=21)
    eng = make_engine(tmp_path, cfg, wts, "cuda:0", torch.bfloat16, max_tokens=1024, max_seqs=4, use_cuda_graph=True,
                      graph_batch_sizes=[1, 2, 4], decode_window=4)
    eng.eos_token_id = None
    eng.runner.capture_graphs()
    assert eng.runner.graph_sizes == [1, 2, 4]
    prompts = [tokens_for(cfg, n, 30 + n) for n in (7, 33, 20)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=40))
    assert [len(o) for o in outs] == [40, 40, 40]
    assert eng.stats.get("decode_windows", 0) >= 5
    for p, o in zip(prompts, outs):
        lg = orc.forward(p + o, wts, cfg)
        for i, tok in enumerate(o):
            row = lg[len(p) + i - 1]
            assert float(row.max() - row[tok]) <= 0.05 * float(row.max() - row.min()), (i, tok, int(row.argmax()))
    got = replay(eng, cut("z", prompts[1] + outs[1], [len(prompts[1])]))["z"]
    check_against_oracle(got, wts, cfg, prompts[1] + outs[1], TOL[torch.bfloat16])
    assert eng.blocks.num_available() == eng.blocks.num_blocks


def test_worker_serves_a_fekolorn_checkpoint(tmp_path):
    """The serving path end to end on the CPU: client -> coordinator -> worker -> LLMBackend -> from_pretrained
    (the registry picks FekolornLM from config.json) -> continuous-batching engine with state slots -> sampled token
    ids, which are the oracle's greedy continuation of each prompt. More prompts than sequence slots."""
    import asyncio

    from src.client import InferenceClient
    from src.config import ModelConfig
    from src.coordinator import Coordinator
    from src.worker import Worker

    cfg = std_config(vocab=300)
    wts = orc.make_weights(cfg, seed=22)
    path = str(tmp_path / "served")
    save_checkpoint(path, cfg, wts)
    mc = ModelConfig(model_name="fk", model_path=path, arch="llama", max_batch_size=2, max_model_len=128,
                     max_num_batched_tokens=128, num_kv_blocks=64, use_cuda_graph=False, max_latency_ms=1.0,
                     overrides={"device": "cpu"})

    async def main():
        w = Worker("w0", host="127.0.0.1", install_signal_handlers=False)
        assert w.load_model(mc)
        wport = await w.start()
        coord = Coordinator(port=0, max_batch_size=4, max_latency_ms=2)
        cport = await coord.start()
        await coord.add_static_worker(f"127.0.0.1:{wport}")
        c = InferenceClient(f"127.0.0.1:{cport}")
        prompts = [tokens_for(cfg, n, 40 + n) for n in (4, 19, 11, 7)]
        rs = await asyncio.wait_for(asyncio.gather(*(c.infer("fk", {"prompt_token_ids": p, "max_tokens": 6,
                                                                    "ignore_eos": True}) for p in prompts)), 120)
        c.close()
        await coord.stop()
        await w.shutdown()
        return prompts, rs

    prompts, rs = asyncio.run(main())
    assert all(r["success"] for r in rs), rs
    for p, r in zip(prompts, rs):
        out = r["outputs"]["token_ids"]
        assert len(out) == 6
        lg = orc.forward(p + out, wts, cfg)
        for i, tok in enumerate(out):
            row = lg[len(p) + i - 1]
            assert float(row.max() - row[tok]) <= 0.05 * float(row.max() - row.min())
