"""
Slow, plain float64 implementation of the Datatar design, one function per mechanism, written from the
design's equations and sharing no code with ``src/``: the tests compare the engine against it.

Notation: x_t is the residual stream of token t (position t, counted from 0), W tensors are [out, in] and
applied as W x. ``weights`` maps checkpoint names to tensors, ``config`` is the checkpoint's config dict.
Everything runs on whole sequences with dense [T, T] masks — no cache, no chunks, no batching.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return rms(x, eps) * w


def norm_around_zero(x, w, eps):
    """the stored weight is an offset from one: the gain is 1 + w."""
    return rms(x, eps) * (1.0 + w)


def rotate_interleaved(x: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., n]: of its first ``dims`` entries, entry 2i pairs with 2i + 1; the pair (u, v) at position p
    turns by the angle p * base^(-2i / dims). Later entries pass unchanged."""
    out = x.clone()
    for i in range(dims // 2):
        ang = pos.to(F64) * (base ** (-2.0 * i / dims))
        c = torch.cos(ang).reshape(-1, *([1] * (x.dim() - 2)))
        s = torch.sin(ang).reshape(-1, *([1] * (x.dim() - 2)))
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def window_mask(t: int, size: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (size 0: every j <= i)."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    ok = (i - j) >= 0
    if size:
        ok = ok & ((i - j) < size)
    return ok


def softmax_with_sink(scores: torch.Tensor, ok: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """scores [H, T, T]; the denominator has one extra term exp(sink_h) per head, attached to no position and
    left out of the score scaling."""
    e = torch.where(ok[None], torch.exp(scores - scores.masked_fill(~ok[None], -1e300).amax(-1, keepdim=True)), 0.0)
    # redo with an explicit common shift so that the sink enters on the same scale
    shift = scores.masked_fill(~ok[None], -1e300).amax(-1, keepdim=True)
    if sink is not None:
        shift = torch.maximum(shift, sink.to(F64)[:, None, None])
    e = torch.where(ok[None], torch.exp(scores - shift), 0.0)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.to(F64)[:, None, None] - shift)
    return e / den


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The mixer on a whole sequence h [T, width], keys and values expanded per head (nothing absorbed)."""
    t = h.shape[0]
    hh, d, r, vd, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(t)
    cq = norm_plain(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).view(t, hh, d + r)
    dkv = h @ w[p + "dkv"].T
    c = norm_plain(dkv[:, :kr], w[p + "dkv.norm"], eps)
    k_shared = dkv[:, kr:].view(t, 1, r)
    k_nope = (c @ w[p + "uk"].T).view(t, hh, d)
    v = (c @ w[p + "uv"].T).view(t, hh, vd)
    rot = m["rot"]
    q_rot = rotate_interleaved(q[..., d:], pos, rot["base"], rot["dims"])
    k_rot = rotate_interleaved(k_shared, pos, rot["base"], rot["dims"])[:, 0]
    scores = (torch.einsum("ihd,jhd->hij", q[..., :d], k_nope) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    ok = window_mask(t, int((m.get("mask") or {}).get("size") or 0))
    pr = softmax_with_sink(scores, ok, w.get(p + "sink"))
    o = torch.einsum("hij,jhv->ihv", pr, v).reshape(t, hh * vd)
    return o @ w[p + "o"].T


def ff_clamped(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def ff_silu(h, w, p):
    g = h @ w[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w_router, top) -> Tuple[torch.Tensor, torch.Tensor]:
    s = torch.sigmoid(h @ w_router.T)
    return torch.topk(s, top, dim=-1)


def moe(h, w, p, m) -> torch.Tensor:
    """Each token's chosen experts see the token scaled by its score; a shared expert sees it as it is."""
    wt, ids = route(h, w[p + "router"], m["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(ids.shape[1]):
            out[t] += ff_silu(wt[t, k] * h[t], w, p + f"e{int(ids[t, k])}.")
    if m.get("shared"):
        out = out + ff_silu(h, w, p + "shared.")
    return out


def forward(weights: Dict[str, torch.Tensor], config: dict, tokens: List[int], layers_out: Optional[list] = None):
    """Logits [T, vocab] (float64) of one whole sequence."""
    w = {k: v.detach().to("cpu", F64) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    for i, lc in enumerate(config["layers"]):
        assert lc["type"] == "latent_attention"
        x = x + norm_around_zero(latent_attention(x, w, f"l{i}.mix.", lc["mixer"], eps), w[f"l{i}.norm1"], eps)
        f = lc.get("mlp")
        if f is not None:
            y = ff_clamped(x, w, f"l{i}.mlp.", f["limit"]) if f["kind"] == "dense" else moe(x, w, f"l{i}.mlp.", f)
            x = x + norm_around_zero(y, w[f"l{i}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (norm_around_zero(x, w["final.norm"], eps) @ w["head"].T) * config["logit_scale"]


# ----------------------------------------------------------------------------- test models
def mixer_cfg(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=12, q_rank=10, window=7, base=1000.0, scale=None):
    c = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "rot": {"base": base, "dims": rot_dim}, "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}
    if window:
        c["mask"] = {"size": window}
    return c


def dense_cfg(ff=24, limit=1.25):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe_cfg(experts=5, top=2, ff=8, shared=12):
    c = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        c["shared"] = {"ff": shared}
    return c


def make_config(layers, vocab=50, width=16, logit_scale=0.7, eps=1e-5) -> dict:
    return {"architecture": "Datatar", "layers": [{"type": "latent_attention", "mixer": m, "mlp": f} for m, f in layers],
            "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def make_weights(config: dict, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random weights under the checkpoint names, rounded to ``dtype`` (so that the engine and the oracle read
    the same numbers) and sized so that activations stay O(1) and routing / softmax are not degenerate."""
    g = torch.Generator().manual_seed(seed)
    wd, out = config["width"], {}

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    out["embed"] = rnd(config["vocab"], wd, std=1.0)
    out["head"] = rnd(config["vocab"], wd, std=wd ** -0.5)
    out["final.norm"] = rnd(wd, std=0.2)
    for i, lc in enumerate(config["layers"]):
        m, p = lc["mixer"], f"l{i}."
        hh, d, r, vd, kr, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        out[p + "norm1"] = rnd(wd, std=0.2)
        out[p + "mix.dq"] = rnd(qr, wd, std=wd ** -0.5)
        out[p + "mix.dq.norm"] = 1.0 + rnd(qr, std=0.2)
        out[p + "mix.uq"] = rnd(hh * (d + r), qr, std=2.0 * qr ** -0.5)
        out[p + "mix.dkv"] = rnd(kr + r, wd, std=wd ** -0.5)
        out[p + "mix.dkv.norm"] = 1.0 + rnd(kr, std=0.2)
        out[p + "mix.uk"] = rnd(hh * d, kr, std=2.0 * kr ** -0.5)
        out[p + "mix.uv"] = rnd(hh * vd, kr, std=kr ** -0.5)
        out[p + "mix.sink"] = rnd(hh, std=1.0)
        out[p + "mix.o"] = rnd(wd, hh * vd, std=(hh * vd) ** -0.5)
        f = lc.get("mlp")
        if f is None:
            continue
        out[p + "norm2"] = rnd(wd, std=0.2)
        if f["kind"] == "dense":
            out[p + "mlp.gate"] = rnd(f["ff"], wd, std=2.0 * wd ** -0.5)
            out[p + "mlp.up"] = rnd(f["ff"], wd, std=2.0 * wd ** -0.5)
            out[p + "mlp.down"] = rnd(wd, f["ff"], std=f["ff"] ** -0.5)
        else:
            ef = f["expert"]["ff"]
            out[p + "mlp.router"] = rnd(f["router"]["experts"], wd, std=2.0 * wd ** -0.5)
            for e in range(f["router"]["experts"]):
                out[p + f"mlp.e{e}.gate"] = rnd(ef, wd, std=2.0 * wd ** -0.5)
                out[p + f"mlp.e{e}.up"] = rnd(ef, wd, std=2.0 * wd ** -0.5)
                out[p + f"mlp.e{e}.down"] = rnd(wd, ef, std=ef ** -0.5)
            if f.get("shared"):
                sf = f["shared"]["ff"]
                out[p + "mlp.shared.gate"] = rnd(sf, wd, std=wd ** -0.5)
                out[p + "mlp.shared.up"] = rnd(sf, wd, std=wd ** -0.5)
                out[p + "mlp.shared.down"] = rnd(wd, sf, std=sf ** -0.5)
    return out


def routing_margins(weights, config, tokens) -> torch.Tensor:
    """[T]: for each position, the smallest gap between the last chosen and the first rejected router score that
    its logits depend on (of the float64 forward): a MoE layer below another layer counts for every earlier
    position too (attention reads them), the last layer's only for the position itself. Tests do not compare
    positions whose routing rests on a close call."""
    w = {k: v.detach().to("cpu", F64) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    out = torch.full((len(tokens),), float("inf"), dtype=F64)
    last = len(config["layers"]) - 1
    for i, lc in enumerate(config["layers"]):
        x = x + norm_around_zero(latent_attention(x, w, f"l{i}.mix.", lc["mixer"], eps), w[f"l{i}.norm1"], eps)
        f = lc.get("mlp")
        if f is None:
            continue
        if f["kind"] == "moe":
            s = torch.sort(torch.sigmoid(x @ w[f"l{i}.mlp.router"].T), dim=-1, descending=True).values
            top = f["router"]["top"]
            if top < s.shape[1]:
                gap = s[:, top - 1] - s[:, top]
                out = torch.minimum(out, gap if i == last else torch.cummin(gap, 0).values)
            y = moe(x, w, f"l{i}.mlp.", f)
        else:
            y = ff_clamped(x, w, f"l{i}.mlp.", f["limit"])
        x = x + norm_around_zero(y, w[f"l{i}.norm2"], eps)
    return out
