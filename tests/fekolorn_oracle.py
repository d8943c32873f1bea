"""
A plain, slow float64 implementation of the Fekolorn design, written from its equations: dense masks, explicit
loops over time for everything recurrent, no cache, no paging, no batching. One function per mechanism. It shares
no code with ``src/``; the tests compare the engine against it.

Notation: T tokens of ONE sequence, positions 0 .. T-1. ``w`` maps checkpoint tensor names to float64 tensors.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dim."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------------------ embedding
def embedding(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    e = cfg["embedding"]
    x = w["embed"][tokens] * float(e.get("scale", 1.0))
    bg = e.get("bigram")
    if bg:
        rows = []
        for i, t in enumerate(tokens):
            rows.append(bg["buckets"] if i == 0 else (tokens[i - 1] * bg["mul_prev"] + t * bg["mul_cur"]) % bg["buckets"])
        x = x + w["bigram"][rows]
    return x


# ------------------------------------------------------------------------------------------- rotary positions
def rotate_half(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, d]: pair (i, i + dims/2) of the first `dims` dims turned by p * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------ softmax attention
def distance_bucket(n: int, B: int, D: float) -> int:
    h = B // 2
    if n < h:
        return n
    return min(B - 1, h + int(math.floor(math.log(n / h) / math.log(D / h) * (B - h))))


def sink_attention(q, k, v, scale: float, sink: torch.Tensor, window: Optional[int], bias=None) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv]; head h reads key/value head h // (H / G). Query i sees j <= i
    (and i - j < window). bias: [T, T, H] added after scaling, or None. The softmax denominator has one more
    term exp(sink[h])."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if bias is not None:
            s = s + bias[:, :, h]
        i = torch.arange(T)[:, None]
        j = torch.arange(T)[None, :]
        ok = j <= i
        if window:
            ok = ok & (i - j < window)
        s = s.masked_fill(~ok, -math.inf)
        m = torch.maximum(s.max(-1, keepdim=True).values, sink[h])
        p = torch.exp(s - m)
        den = p.sum(-1, keepdim=True) + torch.exp(sink[h] - m)
        out[:, h] = (p / den) @ v[:, g]
    return out


def left_attention(h: torch.Tensor, w, pre: str, m: dict, eps: float) -> torch.Tensor:
    """Rotary GQA attention with unit-RMS values, causal, with a sink."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, d)
    k = (h @ w[pre + "k"].T).view(T, G, d)
    v = (h @ w[pre + "v"].T).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, rot["dims"], rot["base"])
        k = rotate_half(k, rot["dims"], rot["base"])
    v = rms(v, eps)
    o = sink_attention(q, k, v, m["scale"], w[pre + "sink"], None)
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def biased_window_attention(h, w, pre: str, m: dict, eps: float, v_first: Optional[torch.Tensor]):
    """GQA attention without rotation: q/k normed over the whole projection, a learned bias per (distance bucket,
    head), a sliding window, a sink, and values blended with the first such layer's. Returns (output, this layer's
    own blended values)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(h @ w[pre + "q"].T, eps) * w[pre + "q.norm"]
    k = rms(h @ w[pre + "k"].T, eps) * w[pre + "k.norm"]
    v = h @ w[pre + "v"].T
    if m.get("v_mix") and v_first is not None:
        lam = w[pre + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    rel = w[pre + "rel"]
    B = rel.shape[0]
    bias = torch.zeros(T, T, H, dtype=F64)
    for i in range(T):
        for j in range(i + 1):
            bias[i, j] = rel[distance_bucket(i - j, B, m["bias_max"])]
    window = (m.get("mask") or {}).get("size")
    o = sink_attention(q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv), m["scale"], w[pre + "sink"], window, bias)
    return o.reshape(T, H * dv) @ w[pre + "o"].T, v


# ------------------------------------------------------------------------------------------- gated delta rule
def short_conv(x: torch.Tensor, cw: torch.Tensor) -> torch.Tensor:
    """x [T, C], cw [C, taps] (last column: the current token), zeros before the start."""
    T, C = x.shape
    taps = cw.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                out[t] += cw[:, j] * x[s]
    return out


def gated_delta_rule(h: torch.Tensor, w, pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).view(T, G, d)
    k = silu(short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).view(T, G, d)
    v = silu(short_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    g = torch.exp(-torch.exp(w[pre + "A_log"]) * torch.nn.functional.softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    gate = silu(h @ w[pre + "g"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        kh = hd // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hd] = S.T @ q[t, kh]
    o = rms(o, eps) * w[pre + "norm"] * gate
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def parallel_mixer(h, w, pre: str, m: dict, eps: float) -> torch.Tensor:
    return (m["left_scale"] * left_attention(h, w, pre + "left.", m["left"], eps)
            + m["right_scale"] * gated_delta_rule(h, w, pre + "right.", m["right"], eps))


# ------------------------------------------------------------------------------------------------ feed-forward
def polynorm_ff(h, w, pre: str, eps: float) -> torch.Tensor:
    z = h @ w[pre + "up"].T
    a, b, c, e = [w[pre + "act"][i] for i in range(4)]
    act = a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e
    return act @ w[pre + "down"].T


# ---------------------------------------------------------------------------------------------------- the model
def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * g


def forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict, layer_out: Optional[list] = None):
    """Logits [T, vocab] of one whole sequence. ``layer_out``: receives the sum of the streams after every layer."""
    w = {k: v.to(F64) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    x0 = embedding(tokens, w, cfg)
    S = cfg.get("streams")
    xs = [x0.clone() for _ in range(S)] if S else [x0]
    v_first = None
    for li, lc in enumerate(cfg["layers"]):
        pre = f"l{li}."
        for q in (1, 2):
            if q == 2 and lc.get("mlp") is None:
                continue
            hc = pre + f"hc{q}."
            u = sum(w[hc + "in"][s] * xs[s] for s in range(S)) if S else xs[0]
            hin = scalar_norm(u, w[pre + f"norm{q}"], eps)
            if q == 1:
                if lc["type"] == "parallel":
                    y = parallel_mixer(hin, w, pre + "mix.", lc["mixer"], eps)
                elif lc["type"] == "attention":
                    y, v_own = biased_window_attention(hin, w, pre + "mix.", lc["mixer"], eps, v_first)
                    if lc["mixer"].get("v_mix") and v_first is None:
                        v_first = v_own
                else:
                    raise ValueError(lc["type"])
            else:
                if lc["mlp"]["kind"] != "dense":
                    raise ValueError(lc["mlp"]["kind"])
                y = polynorm_ff(hin, w, pre + "mlp.", eps)
            if S:
                xs = [sum(w[hc + "mix"][s, t] * xs[s] for s in range(S)) + w[hc + "out"][t] * y for t in range(S)]
            else:
                xs = [xs[0] + y]
        if layer_out is not None:
            layer_out.append(sum(xs))
    x = scalar_norm(sum(xs), w["final.norm"], eps)
    return x @ w["head"].T


# --------------------------------------------------------------------------------- configurations and weights
def attn_cfg(heads=4, kv_heads=2, dim=16, vdim=8, window=6, bias_max=10, v_mix=True, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_max": bias_max, "v_mix": v_mix,
         "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    return m


def parallel_cfg(heads=4, kv_heads=2, dim=16, vdim=8, rot_dims=8, rot_base=100.0, r_heads=2, r_kv_heads=1, r_dim=8,
                 r_vdim=16, conv=3, left_scale=0.7, right_scale=1.1):
    return {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                     "rot": {"base": rot_base, "dims": rot_dims}},
            "right": {"heads": r_heads, "kv_heads": r_kv_heads, "dim": r_dim, "vdim": r_vdim, "conv": conv},
            "left_scale": left_scale, "right_scale": right_scale}


def make_config(layers, width=32, vocab=50, streams=2, buckets=37, eps=1e-5, embed_scale=0.7):
    """layers: list of (type, mixer config, ff or None)."""
    c = {"architecture": "Fekolorn", "embedding": {"scale": embed_scale}, "norm": {"eps": eps}, "vocab": vocab,
         "width": width,
         "layers": [{"type": t, "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
                    for t, m, ff in layers]}
    if buckets:
        c["embedding"]["bigram"] = {"buckets": buckets, "mul_prev": 5, "mul_cur": 3}
    if streams:
        c["streams"] = streams
    return c


def make_weights(cfg: dict, seed: int = 0, rel_rows: int = 12) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names, every value exactly representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams")
    w: Dict[str, torch.Tensor] = {}

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(shape or (1,), generator=g) * std + mean).bfloat16()

    lin = lambda o, i: r(o, i, std=i ** -0.5)  # noqa: E731
    w["embed"] = r(cfg["vocab"], W)
    bg = cfg["embedding"].get("bigram")
    if bg:
        w["bigram"] = r(bg["buckets"] + 1, W, std=0.7)
    for li, lc in enumerate(cfg["layers"]):
        p = f"l{li}."
        for q in (1, 2):
            if q == 2 and lc["mlp"] is None:
                continue
            w[p + f"norm{q}"] = r(std=0.1, mean=1.0).reshape(())
            if S:
                w[p + f"hc{q}.in"] = r(S, std=0.2, mean=1.0 / S)
                w[p + f"hc{q}.out"] = r(S, std=0.2, mean=0.8)
                w[p + f"hc{q}.mix"] = (torch.eye(S) * 0.9 + torch.randn(S, S, generator=g) * 0.1).bfloat16()
        m = lc["mixer"]

        def attn(pre, a, biased):
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            w[pre + "q"], w[pre + "k"], w[pre + "v"] = lin(H * d, W) * 2, lin(G * d, W) * 2, lin(G * dv, W)
            w[pre + "o"] = lin(W, H * dv)
            w[pre + "sink"] = r(H, std=1.0)
            if biased:
                w[pre + "q.norm"], w[pre + "k.norm"] = r(H * d, std=0.2, mean=1.5), r(G * d, std=0.2, mean=1.5)
                w[pre + "rel"] = r(rel_rows, H, std=1.0)
                w[pre + "vmix"] = r(std=0.1, mean=0.4).reshape(())

        if lc["type"] == "attention":
            attn(p + "mix.", m, True)
        else:
            attn(p + "mix.left.", m["left"], False)
            a = m["right"]
            H, G, d, dv, taps = a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["conv"]
            pre = p + "mix.right."
            w[pre + "q"], w[pre + "k"], w[pre + "v"] = lin(G * d, W) * 2, lin(G * d, W) * 2, lin(H * dv, W) * 2
            for nm, n in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w[pre + nm + ".conv"] = r(n, taps, std=0.6)
            w[pre + "b"], w[pre + "a"] = lin(H, W) * 2, lin(H, W) * 2
            w[pre + "A_log"], w[pre + "dt_bias"] = r(H, std=0.5, mean=-0.5), r(H, std=0.5)
            w[pre + "norm"] = r(dv, std=0.2, mean=1.0)
            w[pre + "g"], w[pre + "o"] = lin(H * dv, W) * 2, lin(W, H * dv)
        if lc["mlp"] is not None:
            ff = lc["mlp"]["ff"]
            w[p + "mlp.up"], w[p + "mlp.down"] = lin(ff, W) * 2, lin(W, ff)
            w[p + "mlp.act"] = r(4, std=0.5, mean=0.3)
    w["final.norm"] = r(std=0.1, mean=1.0).reshape(())
    w["head"] = lin(cfg["vocab"], W)
    return w
