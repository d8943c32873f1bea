"""
Datatar on the serving engine against the plain float64 oracle (tests/datatar_oracle.py).

Every test makes its own small configuration and random weights, writes them as a checkpoint directory,
loads it through ``LLMEngine.from_pretrained`` (registry -> model class -> loader) and steps it with
``LLMEngine.replay_step`` (scheduler, block manager, runner, kernels). The CPU cases run the engine's control
flow on the plain-PyTorch op semantics; the ``gpu`` cases run the HIP kernels. Structural faults (a window one
token off, a lost cache row, a missing sink) are far above the fp32 tolerance, so those cases run in fp32;
bf16 cases check the served precision.
"""

import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import datatar_oracle as orc  # noqa: E402

CPU = pytest.param("cpu", id="cpu")
GPU = pytest.param("cuda:0", marks=pytest.mark.gpu, id="gpu")
DEVICES = [CPU, GPU]
TOL = {torch.float32: 3e-4, torch.bfloat16: 6e-2}


def _need(device):
    if device != "cpu":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        from src import ops

        assert ops.mix_available(), "HIP extension src/_Cmix not loaded"


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
    """steps: list of lists of (request id, tokens, wanted places). Returns {rid: {position: logits row}}."""
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


def cut(rid, toks, sizes, want_all=True, end=True):
    """One request alone, cut into portions of the given sizes (the rest one token at a time)."""
    steps, lo = [], 0
    sizes = list(sizes)
    while lo < len(toks):
        n = min(sizes.pop(0) if sizes else 1, len(toks) - lo)
        hi = lo + n
        steps.append([(rid, toks[lo:hi], list(range(n)) if want_all else [], end and hi == len(toks))])
        lo = hi
    return steps


def check_against_oracle(got, weights, config, toks, tol):
    want = orc.forward(weights, config, toks)
    pos = sorted(got)
    g = torch.stack([got[p] for p in pos])
    assert torch.isfinite(g).all()
    e = row_errs(g, want[pos])
    if tol >= 1e-2:
        # bf16 on models this narrow: a few rows of a long sequence round unluckily; the typical row is held to
        # the tolerance and no row may be far off (a structural fault moves rows by O(1))
        assert float(e.median()) < tol / 2 and float(e.max()) < 4 * tol, f"median {float(e.median()):.3e} max {float(e.max()):.3e}"
    else:
        assert float(e.max()) < tol, f"relative error {float(e.max()):.3e} >= {tol}"


def two_layer_config(**kw):
    return orc.make_config([(orc.mixer_cfg(), orc.dense_cfg()), (orc.mixer_cfg(heads=2, window=5), orc.moe_cfg())], **kw)


# ------------------------------------------------------------------------------------------- mechanisms
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norms(device, dtype):
    _need(device)
    from src import ops

    g = torch.Generator().manual_seed(0)
    x = (torch.randn(5, 40, generator=g) * 3).to(dtype)
    w = (torch.randn(24, generator=g) * 0.3).to(dtype)
    xs = x.to(device)[:, 8:32]  # a strided view: rows of 24 inside rows of 40
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for unit, fn in ((False, orc.norm_plain), (True, orc.norm_around_zero)):
        y = ops.rms_norm_ext(xs, w.to(device), 1e-3, unit_offset=unit)
        want = fn(x[:, 8:32].double(), w.double(), 1e-3)
        assert (y.cpu().double() - want).abs().max() < tol * want.abs().max()
    # norm on a sublayer's output, added into an fp32 residual; the bf16 copy follows it
    r0 = torch.randn(5, 24, generator=g)
    resid = r0.clone().to(device)
    act = torch.empty(5, 24, dtype=torch.bfloat16, device=device)
    ops.post_norm_residual(resid, xs, w.to(device), 1e-3, True, act=act)
    want = r0.double() + orc.norm_around_zero(x[:, 8:32].double(), w.double(), 1e-3)
    assert resid.dtype == torch.float32
    assert (resid.cpu().double() - want).abs().max() < 1e-5 * want.abs().max()
    assert torch.equal(act.cpu(), resid.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("device", DEVICES)
def test_gated_activations(device):
    _need(device)
    from src import ops

    g = torch.Generator().manual_seed(1)
    gu = torch.randn(7, 2 * 13, generator=g) * 3   # well beyond the clamp on both sides
    a, b = gu[:, :13].double(), gu[:, 13:].double()
    y = ops.gated_act(gu.to(device), ops.ACT_SILU).cpu().double()
    assert (y - a * torch.sigmoid(a) * b).abs().max() < 1e-5
    lim = 1.25
    y = ops.gated_act(gu.to(device), ops.ACT_CLAMPED, lim, 1.702).cpu().double()
    ac, bc = a.clamp(max=lim), b.clamp(-lim, lim)
    assert (y - ac * torch.sigmoid(1.702 * ac) * (bc + 1)).abs().max() < 1e-5
    assert float(a.min()) < -lim and float(a.max()) > lim   # the gate is clamped above only
    # bf16 rows of a multiple of 8 columns (the 16-byte path on the GPU)
    gb = (torch.randn(5, 2 * 16, generator=g) * 2).to(torch.bfloat16)
    ab, bb = gb[:, :16].double(), gb[:, 16:].double()
    for kind, want in ((ops.ACT_SILU, ab * torch.sigmoid(ab) * bb),
                       (ops.ACT_CLAMPED, ab.clamp(max=lim) * torch.sigmoid(1.702 * ab.clamp(max=lim)) * (bb.clamp(-lim, lim) + 1))):
        y = ops.gated_act(gb.to(device), kind, lim, 1.702).cpu().double()
        assert (y - want).abs().max() < 1e-2 * want.abs().max()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("top", [1, 2, 5])
@pytest.mark.parametrize("tokens", [9, 300])   # fused logits + selection / library fp32 logits + selection kernel
def test_routing_scores_not_renormalised(device, top, tokens):
    _need(device)
    from src import ops

    g = torch.Generator().manual_seed(2)
    x, wr = torch.randn(tokens, 16, generator=g), torch.randn(5, 16, generator=g)
    w, ids = ops.route_sigmoid_topk(x.to(device), wr.to(device), top)
    ws, is_ = orc.route(x.double(), wr.double(), top)
    assert torch.equal(ids.cpu().long(), is_)
    assert (w.cpu().double() - ws).abs().max() < 1e-6
    if top > 1:
        assert float((w.sum(-1) - 1).abs().min()) > 1e-3  # scores are used as they are


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("tokens,shared", [(6, True), (50, True), (50, False)])
def test_experts_scale_their_input(device, tokens, shared):
    """Both expert paths (per-row gathered weights below ops.mix.MOE_BMM_MAX_ROWS rows, per-expert groups above)."""
    _need(device)
    from src import ops

    cfg = orc.make_config([(orc.mixer_cfg(), orc.moe_cfg(experts=4, top=2, ff=8, shared=12 if shared else 0))], width=16)
    wts = orc.make_weights(cfg, seed=3, dtype=torch.float32)
    p = "l0.mlp."
    g = torch.Generator().manual_seed(4)
    x = torch.randn(tokens, 16, generator=g)
    want = orc.moe(x.double(), {k: v.double() for k, v in wts.items()}, p, cfg["layers"][0]["mlp"])
    w13 = torch.stack([torch.cat([wts[p + f"e{e}.gate"], wts[p + f"e{e}.up"]]) for e in range(4)]).to(device)
    w2 = torch.stack([wts[p + f"e{e}.down"] for e in range(4)]).to(device)
    xd = x.to(device)
    w, ids = ops.route_sigmoid_topk(xd, wts[p + "router"].to(device), 2)
    extra = None
    if shared:
        sgu = torch.cat([wts[p + "shared.gate"], wts[p + "shared.up"]]).to(device)
        extra = torch.nn.functional.linear(ops.gated_act(torch.nn.functional.linear(xd, sgu), ops.ACT_SILU),
                                           wts[p + "shared.down"].to(device))
    y = ops.moe_input_scaled(xd, w13, w2, w, ids, extra=extra)
    assert y.dtype == torch.float32
    assert (y.cpu().double() - want).abs().max() < 2e-5 * want.abs().max()


def _dense_latent_attn(q_lat, q_rot, rows, p, sink, window, scale):
    """Absorbed form on one sequence, dense: q_lat [H, n, R], q_rot [H, n, r] (rotated), rows [ctx, R + r]."""
    rank = q_lat.shape[-1]
    sc = (torch.einsum("hqr,jr->hqj", q_lat, rows[:, :rank]) + torch.einsum("hqd,jd->hqj", q_rot, rows[:, rank:])) * scale
    j = torch.arange(rows.shape[0])
    ok = (p[:, None] - j[None]) >= 0
    if window:
        ok &= (p[:, None] - j[None]) < window
    pr = orc.softmax_with_sink(sc, ok, sink)
    return torch.einsum("hqj,jr->hqr", pr, rows[:, :rank])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rank,rot,heads,window", [(12, 4, 3, 37), (40, 8, 5, 0), (130, 6, 2, 129), (8, 2, 1, 1),
                                                   (64, 16, 6, 37), (96, 0, 2, 0), (256, 32, 7, 129), (32, 16, 1, 16),
                                                   (128, 64, 9, 0), (256, 64, 2, 200)])
def test_latent_cache_and_attention_ops(device, dtype, rank, rot, heads, window):
    """latent_kv_write + latent_attn over scattered pages, against a dense computation: one standout key per
    query placed far back, on a page border, just inside and just outside the window (the outside one must be
    ignored however large its score), for a prompt portion that starts mid-page and for single decode rows."""
    _need(device)
    from src import ops

    g = torch.Generator().manual_seed(5)
    bs, ctx, nq, eps, scale, base = 16, 300, 23, 1e-5, 0.3, 500.0
    kv = torch.randn(ctx, rank + rot, generator=g).to(dtype)
    wn = (1 + 0.2 * torch.randn(rank, generator=g)).to(dtype)
    pos = torch.arange(ctx)
    inv = ops.rope_inv_freq(base, rot, device)
    nb = (ctx + bs - 1) // bs
    perm = torch.randperm(2 * nb, generator=g)[:nb]           # pages scattered over a larger pool
    cache = torch.zeros(2 * nb, bs, rank + rot, dtype=dtype, device=device)
    slots = perm[pos // bs] * bs + pos % bs
    slots_w = slots.clone()
    slots_w[7] = -1                                            # a row that is not written stays as it was
    ops.latent_kv_write(cache, kv.to(device), wn.to(device), pos.to(device), slots_w.to(device), rank, rot, inv, eps)
    c = orc.norm_plain(kv[:, :rank].double(), wn.double(), eps)
    kr = orc.rotate_interleaved(kv[:, None, rank:].double(), pos, base, rot)[:, 0]
    rows = torch.cat([c, kr], -1)
    rows[7] = 0
    got_rows = cache.view(-1, rank + rot)[slots.to(device)].cpu().double()
    assert (got_rows - rows).abs().max() < (1e-5 if dtype == torch.float32 else 2e-2) * rows.abs().max()
    rows = got_rows                                            # attention is checked on what the cache holds

    qh = 5 + rot                                               # 5 unrotated dims before the rotary part
    p = torch.arange(ctx - nq, ctx)
    q = torch.randn(nq, heads * qh, generator=g).to(dtype)
    q_lat = torch.randn(heads, nq, rank, generator=g)
    # standout keys: query i looks hard at one key chosen by its index
    w_eff = window if window else ctx
    for i in range(nq):
        pi = int(p[i])
        target = [pi - w_eff + 1, pi - w_eff, (pi // bs) * bs, (pi // bs) * bs - 1, 0, pi][i % 6]
        target = max(0, target)
        q_lat[:, i] = rows[target, :rank].float() * (6.0 / max(1e-3, float(rows[target, :rank].norm()) ** 2) / scale)
    q_lat = q_lat.to(dtype)
    sink = 6.0 + torch.randn(heads, generator=g)   # comparable to the standout scores: it takes real weight
    bt = perm[None].to(torch.int32).to(device)
    ctx_t = torch.tensor([ctx], dtype=torch.int32, device=device)
    cu = torch.tensor([0, nq], dtype=torch.int32, device=device)
    # on the GPU in bf16 the shapes the matrix-core kernel takes must really run on it (impl 2 fails otherwise),
    # and the FMA kernel (impl 1) must agree on the same inputs
    mfma = device != "cpu" and dtype == torch.bfloat16 and rank % 32 == 0 and rank <= 256 and rot % 16 == 0
    out = ops.latent_attn(q_lat.to(device), q.to(device), 5, cache, bt, cu, ctx_t, p.to(device), sink.to(device), nq,
                          window, scale, rot, inv, impl=2 if mfma else 0)
    if mfma:
        out1 = ops.latent_attn(q_lat.to(device), q.to(device), 5, cache, bt, cu, ctx_t, p.to(device), sink.to(device),
                               nq, window, scale, rot, inv, impl=1)
        assert (out.float() - out1.float()).abs().max() < 2e-2 * out1.float().abs().max()
        # impl 3: the matrix-core kernel that keeps the queries in LDS (the one decode-sized steps and other
        # rotary widths use), on the same prompt-sized step
        out3 = ops.latent_attn(q_lat.to(device), q.to(device), 5, cache, bt, cu, ctx_t, p.to(device), sink.to(device),
                               nq, window, scale, rot, inv, impl=3)
        assert (out3.float() - out1.float()).abs().max() < 2e-2 * out1.float().abs().max()
    q_rot = orc.rotate_interleaved(q.view(nq, heads, qh)[:, :, 5:].double(), p, base, rot).transpose(0, 1)
    want = _dense_latent_attn(q_lat.double(), q_rot, rows, p, sink, window, scale)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert (out.cpu().double() - want).abs().max() < tol * want.abs().max()
    # the sink takes weight: without it the outputs differ
    no_sink = _dense_latent_attn(q_lat.double(), q_rot, rows, p, None, window, scale)
    assert (no_sink - want).abs().max() > 0.03 * want.abs().max()
    # decode form: one row per sequence, three "sequences" sharing the pages at different lengths
    lens = [ctx, ctx - 9, 17]
    qd = q[:3].to(device)
    qld = q_lat[:, :3].contiguous().to(device)
    pd = torch.tensor([n - 1 for n in lens])
    outd = ops.latent_attn(qld, qd, 5, cache, bt.expand(3, -1).contiguous(), None,
                           torch.tensor(lens, dtype=torch.int32, device=device), pd.to(device), sink.to(device), 1,
                           window, scale, rot, inv)
    for i, n in enumerate(lens):
        qr = orc.rotate_interleaved(q[i:i + 1].view(1, heads, qh)[:, :, 5:].double(), pd[i:i + 1], base, rot).transpose(0, 1)
        w1 = _dense_latent_attn(q_lat[:, i:i + 1].double(), qr, rows[:n], pd[i:i + 1], sink, window, scale)
        assert (outd[:, i:i + 1].cpu().double() - w1).abs().max() < tol * max(1e-6, float(w1.abs().max()))


# ------------------------------------------------------------------------------------------ whole model
CONFIGS = {
    "dense+moe": lambda: two_layer_config(),
    "top1-noshared-nomlp": lambda: orc.make_config(
        [(orc.mixer_cfg(heads=1, dim=4, rot_dim=2, vdim=9, kv_rank=5, q_rank=3, window=3), None),
         (orc.mixer_cfg(heads=4, window=0), orc.moe_cfg(experts=3, top=1, ff=6, shared=0)),
         (orc.mixer_cfg(heads=2, dim=6, rot_dim=6, vdim=6, kv_rank=70, window=20), orc.moe_cfg(experts=6, top=3))],
        vocab=37, width=20, logit_scale=1.3),
    "wide": lambda: orc.make_config([(orc.mixer_cfg(heads=5, dim=16, rot_dim=8, vdim=12, kv_rank=136, q_rank=24,
                                                    window=33), orc.dense_cfg(ff=40, limit=0.8))] * 2,
                                    vocab=91, width=48, logit_scale=0.25),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt(tmp_path, device, dtype, name):
    _need(device)
    cfg = CONFIGS[name]()
    wts = orc.make_weights(cfg, seed=11)
    toks = tokens_for(cfg, 70, 0)
    eng = make_engine(tmp_path, cfg, wts, device, dtype)
    got = replay(eng, cut("a", toks, [len(toks)]))["a"]
    # positions whose routing rests on a close call (at the compared precision) are not compared
    gaps = orc.routing_margins(wts, cfg, toks)
    got = {p: v for p, v in got.items() if float(gaps[p]) > (1e-5 if dtype == torch.float32 else 5e-3)}
    assert len(got) >= 10
    check_against_oracle(got, wts, cfg, toks, TOL[dtype])
    assert eng.blocks.num_available() == eng.blocks.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_request(tmp_path, device):
    _need(device)
    cfg = two_layer_config()
    wts = orc.make_weights(cfg, seed=12)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    toks = tokens_for(cfg, 4, 2)
    got = replay(eng, [[("one", toks[:1], [0], True)]] + cut("a", toks, [1, 1, 2]))
    check_against_oracle(got["one"], wts, cfg, toks[:1], TOL[torch.float32])
    check_against_oracle(got["a"], wts, cfg, toks, TOL[torch.float32])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2] * 40, [3, 2, 17, 2, 5, 31, 2], [1] * 5 + [16, 16, 15, 1, 17], [37]])
def test_portions_and_decode_equal_whole(tmp_path, device, sizes):
    """Portions of many sizes down to two tokens, cut inside pages and windows; the rest decodes one by one,
    far enough that the windows (5 and 7) slide over decoded tokens and decode crosses page borders."""
    _need(device)
    cfg = two_layer_config()
    wts = orc.make_weights(cfg, seed=13)
    toks = tokens_for(cfg, 90, 3)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    got = replay(eng, cut("a", toks, sizes))["a"]
    assert sorted(got) == list(range(len(toks)))
    check_against_oracle(got, wts, cfg, toks, TOL[torch.float32])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_bf16(tmp_path, device):
    _need(device)
    cfg = orc.make_config([(orc.mixer_cfg(window=40), orc.dense_cfg())] * 2)
    wts = orc.make_weights(cfg, seed=14)
    toks = tokens_for(cfg, 200, 4)
    eng = make_engine(tmp_path, cfg, wts, device, torch.bfloat16)
    got = replay(eng, cut("a", toks, [20]))["a"]
    check_against_oracle(got, wts, cfg, toks, TOL[torch.bfloat16])


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone_and_blocks_are_reused(tmp_path, device):
    """Four live requests of unequal lengths, prompt portions beside single decode tokens, requests sitting out
    steps, in a pool too small for all requests at once: finished requests' blocks are taken by later ones."""
    _need(device)
    cfg = two_layer_config()
    wts = orc.make_weights(cfg, seed=15)
    lens = {"a": 75, "b": 21, "c": 50, "d": 33, "e": 64, "f": 18}
    toks = {r: tokens_for(cfg, n, 10 + i) for i, (r, n) in enumerate(lens.items())}
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32, max_tokens=208, max_seqs=4)
    total = eng.blocks.num_blocks
    at = {r: 0 for r in lens}

    def take(r, n):
        lo = at[r]
        hi = min(len(toks[r]), lo + n)
        at[r] = hi
        return (r, toks[r][lo:hi], list(range(hi - lo)), hi == len(toks[r]))

    steps = [[take("a", 30), take("b", 2)],
             [take("a", 1), take("b", 17), take("c", 16), take("d", 33)],          # d whole and gone
             [take("a", 1), take("b", 1), take("c", 2)],
             [take("b", 1), take("c", 31), take("e", 5)],                          # a sits out; b ends; e takes d's slot
             [take("a", 43), take("c", 1), take("e", 27)],                         # a ends (75); c ends
             [take("e", 1), take("f", 18)],                                        # f reuses freed blocks
             [take("e", 31)]]
    got = replay(eng, steps)
    assert all(at[r] == lens[r] for r in lens)
    for r in lens:
        assert sorted(got[r]) == list(range(lens[r]))
        check_against_oracle(got[r], wts, cfg, toks[r], TOL[torch.float32])
    assert eng.blocks.num_available() == total
    assert eng.scheduler.steps_mixed >= 3 and not eng.scheduler.running
    assert sum(-(-n // 16) for n in lens.values()) > total  # the pool could not hold them all at once


@pytest.mark.parametrize("device", DEVICES)
def test_window_edges_sink_and_far_keys_show_in_logits(tmp_path, device):
    """A one-layer model whose attention is made sharp (large scale): the oracle's logits move by far more than
    the tolerance when the window is one token longer or shorter or the sink is dropped, and the engine agrees
    with the right one — at prompt positions and at decoded ones, around the window's edge and a page border."""
    _need(device)
    win = 19
    cfg = orc.make_config([(orc.mixer_cfg(window=win, scale=2.5), None)], width=16)
    wts = orc.make_weights(cfg, seed=16, dtype=torch.float32)
    toks = tokens_for(cfg, 60, 5)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    got = replay(eng, cut("a", toks, [26]))["a"]        # 26 in the prompt, the rest decoded
    want = orc.forward(wts, cfg, toks)
    g = torch.stack([got[p] for p in range(len(toks))])
    assert rel_err(g, want) < TOL[torch.float32]
    for delta in (-1, 1):
        c2 = json.loads(json.dumps(cfg))
        c2["layers"][0]["mixer"]["mask"]["size"] = win + delta
        other = orc.forward(wts, c2, toks)
        for lo, hi in ((win - 1, 26), (30, 60)):          # prompt rows past the window, decoded rows
            assert rel_err(other[lo:hi], want[lo:hi]) > 30 * TOL[torch.float32]
    w2 = dict(wts)
    w2.pop("l0.mix.sink")
    assert rel_err(orc.forward(w2, cfg, toks), want) > 30 * TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_without_window(tmp_path, device):
    """No window: a key hundreds of tokens and many pages back keeps its weight (decode and prompt rows)."""
    _need(device)
    cfg = orc.make_config([(orc.mixer_cfg(window=0, scale=2.0), orc.dense_cfg())], width=16)
    wts = orc.make_weights(cfg, seed=17, dtype=torch.float32)
    toks = tokens_for(cfg, 330, 6)
    eng = make_engine(tmp_path, cfg, wts, device, torch.float32)
    got = replay(eng, [[("a", toks[:300], [0, 299])]] + cut("a", toks[300:], []))["a"]
    # cut() restarted its positions at 0 for the tail: shift them
    tail = {300 + p: v for p, v in got.items() if p < 30 and p not in (0,)}
    full = {0: got[0], 299: got[299], **{p: v for p, v in tail.items()}}
    full.pop(300, None)
    want = orc.forward(wts, cfg, toks)
    pos = sorted(full)
    assert rel_err(torch.stack([full[p] for p in pos]), want[pos]) < TOL[torch.float32]
    # dropping the first 100 keys changes the late rows: far keys matter in this model
    c2 = json.loads(json.dumps(cfg))
    c2["layers"][0]["mixer"]["mask"] = {"size": 200}
    assert rel_err(orc.forward(wts, c2, toks)[310:], want[310:]) > 30 * TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_engine(tmp_path, device):
    """LLMEngine.generate (scheduler, continuous batching, paged cache, sampling) on three prompts of unequal
    length: every generated token is the oracle's argmax given the tokens before it, or within the served
    precision of it."""
    _need(device)
    from src.preproc import SamplingParams

    cfg = orc.make_config([(orc.mixer_cfg(), orc.dense_cfg()), (orc.mixer_cfg(heads=2, window=9), orc.dense_cfg())],
                          vocab=48)
    wts = orc.make_weights(cfg, seed=18)
    dtype = torch.bfloat16
    eng = make_engine(tmp_path, cfg, wts, device, dtype, max_tokens=512, max_seqs=4, mixed_batching="auto")
    eng.eos_token_id = None
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 23, 40)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12))
    assert [len(o) for o in outs] == [12, 12, 12]
    for p, o in zip(prompts, outs):
        lg = orc.forward(wts, cfg, p + o)
        for i, tok in enumerate(o):
            row = lg[len(p) + i - 1]
            spread = float(row.max() - row.min())
            assert float(row.max() - row[tok]) <= 0.05 * spread, (i, tok, int(row.argmax()))
    assert eng.blocks.num_available() == eng.blocks.num_blocks


def test_registry_picks_the_model_class_from_config(tmp_path):
    from src.models.datatar import DatatarLM
    from src.models.registry import family_of, resolve

    cfg = two_layer_config()
    save_checkpoint(str(tmp_path / "d"), cfg, orc.make_weights(cfg))
    assert family_of(str(tmp_path / "d")) == "datatar"
    name, arch, cls = resolve(str(tmp_path / "d"))
    assert cls is DatatarLM and arch.num_layers == 2 and arch.layers[1].mixer.window == 5
    assert arch.to_config()["layers"] == cfg["layers"]
    os.makedirs(tmp_path / "h")
    with open(tmp_path / "h" / "config.json", "w") as f:
        json.dump({"model_type": "llama", "hidden_size": 64, "num_attention_heads": 2, "num_hidden_layers": 1,
                   "intermediate_size": 128, "vocab_size": 100}, f)
    assert family_of(str(tmp_path / "h")) == "llama"
    with open(tmp_path / "h" / "config.json", "w") as f:
        json.dump({"architecture": "Unknown"}, f)
    with pytest.raises(ValueError):
        family_of(str(tmp_path / "h"))


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run end to end on the CPU: steps on stdin, logits files and 'done' lines out."""
    import subprocess
    import sys

    import numpy as np

    cfg = two_layer_config()
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
    assert not os.path.exists(tmp_path / "o" / "1.f32") or True
    want = orc.forward(wts, cfg, toks)
    a = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1))
    assert rel_err(a, want[[0, 29]]) < TOL[torch.float32]
    b = torch.from_numpy(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4").reshape(1, -1))
    assert rel_err(b, orc.forward(wts, cfg, toks[:3])[[2]]) < TOL[torch.float32]
    c = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(1, -1))
    assert rel_err(c, want[[39]]) < TOL[torch.float32]


@pytest.mark.gpu
def test_generation_with_decode_graphs_and_decode_gemms(tmp_path):
    """Served configuration: shapes that the weight-streaming decode GEMM and the expert-streaming grouped GEMM
    tile (width 256, expert width 64), the matrix-core attention (rank 64, rot 16), decode steps replayed from
    captured hipGraphs in multi-step windows. Every replay's token is checked against the oracle."""
    _need("cuda:0")
    from src.preproc import SamplingParams

    mixer = orc.mixer_cfg(heads=4, dim=48, rot_dim=16, vdim=32, kv_rank=64, q_rank=96, window=24)
    cfg = orc.make_config([(mixer, orc.dense_cfg(ff=256)), (mixer, orc.moe_cfg(experts=4, top=2, ff=64, shared=64))],
                          vocab=128, width=256)
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
        lg = orc.forward(wts, cfg, p + o)
        for i, tok in enumerate(o):
            row = lg[len(p) + i - 1]
            assert float(row.max() - row[tok]) <= 0.05 * float(row.max() - row.min()), (i, tok, int(row.argmax()))
    # the same prompts teacher-forced through replay_step (eager, no graphs) give the oracle's logits
    got = replay(eng, cut("z", prompts[1] + outs[1], [len(prompts[1])]))["z"]
    check_against_oracle(got, wts, cfg, prompts[1] + outs[1], TOL[torch.bfloat16])
    assert eng.blocks.num_available() == eng.blocks.num_blocks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fused_launches_equal_their_parts(device, dtype):
    """latent_qkv_prep = rms_norm_ext + latent_kv_write; moe_input_scaled(post_norm=...) = the expert sum followed
    by post_norm_residual. On narrow (scalar path) and 8-aligned (16-byte path) widths."""
    _need(device)
    from src import ops

    g = torch.Generator().manual_seed(7)
    for q_rank, rank, rot in ((10, 12, 4), (16, 32, 16)):
        t, bs = 9, 4
        p = torch.randn(t, q_rank + rank + rot, generator=g).to(dtype).to(device)
        wq = (1 + 0.1 * torch.randn(q_rank, generator=g)).to(dtype).to(device)
        wkv = (1 + 0.1 * torch.randn(rank, generator=g)).to(dtype).to(device)
        pos = torch.arange(3, 3 + t).to(device)
        slots = torch.tensor([5, 0, -1, 7, 2, 11, 3, 9, 1]).to(device)
        inv = ops.rope_inv_freq(100.0, rot, device)
        c1 = torch.zeros(3, bs, rank + rot, dtype=dtype, device=device)
        c2 = torch.zeros_like(c1)
        cq = ops.latent_qkv_prep(p, q_rank, wq, wkv, c1, pos, slots, rank, rot, inv, 1e-5)
        ops.latent_kv_write(c2, p[:, q_rank:], wkv, pos, slots, rank, rot, inv, 1e-5)
        assert torch.equal(c1, c2) and float(c1.float().abs().sum()) > 0
        assert torch.equal(cq, ops.rms_norm_ext(p[:, :q_rank], wq, 1e-5))
    for h, f, tokens in ((12, 6, 5), (16, 8, 70)):
        e, k = 4, 2
        x = torch.randn(tokens, h, generator=g).to(dtype).to(device)
        w13 = (torch.randn(e, 2 * f, h, generator=g) * 0.3).to(dtype).to(device)
        w2 = (torch.randn(e, h, f, generator=g) * 0.3).to(dtype).to(device)
        router = torch.randn(e, h, generator=g).to(dtype).to(device)
        extra = torch.randn(tokens, h, generator=g).to(dtype).to(device)
        nw = (0.2 * torch.randn(h, generator=g)).to(dtype).to(device)
        w, ids = ops.route_sigmoid_topk(x, router, k)
        r0 = torch.randn(tokens, h, generator=g).to(device)
        want = r0.clone()
        ops.post_norm_residual(want, ops.moe_input_scaled(x, w13, w2, w, ids, extra=extra), nw, 1e-5, True)
        got = r0.clone()
        act = torch.empty(tokens, h, dtype=torch.bfloat16, device=device)
        assert ops.moe_input_scaled(x, w13, w2, w, ids, extra=extra, post_norm=(got, nw, 1e-5, True, act)) is None
        assert (got - want).abs().max() < 1e-5 * want.abs().max()
        assert torch.equal(act, got.to(torch.bfloat16))


def test_worker_serves_a_datatar_checkpoint(tmp_path):
    """The serving path end to end on the CPU: client -> coordinator -> worker -> LLMBackend -> from_pretrained
    (the registry picks DatatarLM from config.json) -> continuous-batching engine -> sampled token ids, which are
    the oracle's greedy continuation of each prompt."""
    import asyncio

    from src.client import InferenceClient
    from src.config import ModelConfig
    from src.coordinator import Coordinator
    from src.worker import Worker

    cfg = orc.make_config([(orc.mixer_cfg(), orc.dense_cfg()), (orc.mixer_cfg(heads=2, window=6), orc.dense_cfg(ff=16))],
                          vocab=300, width=16)
    wts = orc.make_weights(cfg, seed=22, dtype=torch.float32)
    path = str(tmp_path / "served")
    save_checkpoint(path, cfg, wts)
    mc = ModelConfig(model_name="dt", model_path=path, arch="llama", max_batch_size=4, max_model_len=128,
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
        prompts = [tokens_for(cfg, n, 40 + n) for n in (4, 19, 11)]
        rs = await asyncio.wait_for(asyncio.gather(*(c.infer("dt", {"prompt_token_ids": p, "max_tokens": 6,
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
        lg = orc.forward(wts, cfg, p + out)
        for i, tok in enumerate(out):
            row = lg[len(p) + i - 1]
            assert float(row.max() - row[tok]) <= 0.05 * float(row.max() - row.min())
