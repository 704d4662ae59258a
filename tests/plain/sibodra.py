"""A plain, slow statement of the Sibodra decoder in float64 torch on the CPU: one function per
mechanism, whole sequences, no cache and no state.  It shares nothing with the product path; the
GPU tests hold the framework to it.

The model keeps ``S`` copies of the residual stream (all start as the embedded row).  A sublayer
reads a weighted sum of the copies through a layer norm without bias, and its result goes back
into every copy while the copies are mixed among themselves.  Two mixers: a grouped-query softmax
attention (per-head RMS norm of queries and keys, partial rotation with frequencies stretched for
long contexts, capped scores, a sink of score zero in the denominator, one sigmoid gate per head)
and a latent attention (queries through a normed low-rank latent, keys and values from another
latent plus one rotated key part shared by the heads, a sigmoid gate per output channel).  Two
feed-forwards: a SiLU-gated dense one, and a mixture of experts (squared-ReLU experts, a router
with a bias, weights from the softmax over the chosen logits, a shared expert for every token).
The logits pass a cap.

``rounding=torch.bfloat16`` rounds where a bfloat16 run rounds (inputs and outputs of matrix
products), which gives the yardstick for the error that rounding alone costs.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch

F64 = torch.float64


def _r(x: torch.Tensor, rounding) -> torch.Tensor:
    return x if rounding is None else x.to(rounding).to(F64)


def matmul(x, w, rounding=None):
    """``x [T, in] -> [T, out]`` with ``w [out, in]``."""
    return _r(_r(x, rounding) @ w.to(F64).T, rounding)


def layer_norm(x, w, eps: float):
    """Mean taken off, divided by the root of (variance + eps), times a weight; no bias."""
    mu = x.mean(dim=-1, keepdim=True)
    dev = x - mu
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w.to(F64)


def rms_norm(x, w, eps: float):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def cap(z, c: float):
    return c * torch.tanh(z / c)


def pair_frequencies(dims: int, base: float, scaling=None) -> torch.Tensor:
    """Frequency of pair i of ``dims`` rotated places: ``base^(-2i/dims)``; with ``scaling`` the
    slow pairs (wavelength beyond ``original / low``) are slowed by ``factor``, the fast ones
    (wavelength below ``original / high``) kept, and those between blended linearly in
    ``original / wavelength``."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f:
            wave = 2.0 * math.pi / fi
            if wave < orig / hi:
                out.append(fi)
            elif wave > orig / lo:
                out.append(fi / fac)
            else:
                s = (orig / wave - lo) / (hi - lo)
                out.append((1.0 - s) * fi / fac + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate_half(x, freq):
    """``x [T, ..., n]``: the first ``2 len(freq)`` places turn by position * freq, place i paired
    with place i + len(freq); the rest pass."""
    T, half = x.shape[0], freq.shape[0]
    ang = torch.arange(T, dtype=F64)[:, None] * freq[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], dim=-1)


def causal_scores_softmax(scores, sink_one: bool):
    """``scores [H, T, T]`` -> weights over keys j <= i; ``sink_one`` puts a one (a key of score
    zero that has no value) into the denominator."""
    T = scores.shape[-1]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, -math.inf)
    m = scores.max(dim=-1, keepdim=True).values
    if sink_one:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(scores - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink_one:
        den = den + torch.exp(-m)
    return e / den


def attention(h, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float, rounding=None):
    """Grouped-query attention on ``h [T, width]`` with the tensors ``p + name``."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = matmul(h, t[p + "q"], rounding).reshape(T, H, d)
    k = matmul(h, t[p + "k"], rounding).reshape(T, G, d)
    v = matmul(h, t[p + "v"], rounding).reshape(T, G, dv)
    q = rms_norm(q, t[p + "q.norm"], eps)
    k = rms_norm(k, t[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        freq = pair_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_half(q, freq), rotate_half(k, freq)
    q, k = _r(q, rounding), _r(k, rounding)
    per = H // G
    k = k.repeat_interleave(per, dim=1)
    v = v.repeat_interleave(per, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    if m.get("softcap"):
        scores = cap(scores, m["softcap"])
    w = causal_scores_softmax(scores, sink_one=True)
    ctx = torch.einsum("hij,jhd->ihd", w, v)
    gate = torch.sigmoid(matmul(h, t[p + "g"], rounding))          # [T, H]
    ctx = _r(ctx, rounding) * gate[:, :, None]
    return matmul(ctx.reshape(T, H * dv), t[p + "o"], rounding)


def latent_attention(h, t: Dict[str, torch.Tensor], p: str, m: dict, eps: float, rounding=None):
    T = h.shape[0]
    H, d, rd, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = _r(rms_norm(matmul(h, t[p + "dq"], rounding), t[p + "dq.norm"], eps), rounding)
    q = matmul(cq, t[p + "uq"], rounding).reshape(T, H, d + rd)
    kv = matmul(h, t[p + "dkv"], rounding)
    c = _r(rms_norm(kv[:, :r], t[p + "dkv.norm"], eps), rounding)
    k_rot = kv[:, r:r + rd]
    freq = pair_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q_un, q_rot = q[..., :d], rotate_half(q[..., d:], freq)
    k_rot = rotate_half(k_rot, freq)
    k_un = matmul(c, t[p + "uk"], rounding).reshape(T, H, d)
    v = matmul(c, t[p + "uv"], rounding).reshape(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_un, k_un)
              + torch.einsum("ihd,jd->hij", _r(q_rot, rounding), _r(k_rot, rounding))) * m["scale"]
    w = causal_scores_softmax(scores, sink_one=False)
    ctx = _r(torch.einsum("hij,jhd->ihd", w, v), rounding).reshape(T, H * dv)
    ctx = ctx * torch.sigmoid(matmul(h, t[p + "g"], rounding))
    return matmul(ctx, t[p + "o"], rounding)


def dense_ff(h, t, p: str, rounding=None):
    act = silu(matmul(h, t[p + "gate"], rounding)) * matmul(h, t[p + "up"], rounding)
    return matmul(act, t[p + "down"], rounding)


def expert(h, t, p: str, rounding=None):
    z = torch.relu(matmul(h, t[p + "up"], rounding))
    return matmul(z * z, t[p + "down"], rounding)


def moe_ff(h, t, p: str, mlp: dict, rounding=None, margins: list = None):
    """``margins``: gets, row by row, how far the last chosen logit stands above the first one
    that was not chosen (infinite when every expert is chosen)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = _r(h, rounding) @ t[p + "router"].to(F64).T + t[p + "router.b"].to(F64)
    if margins is not None:
        srt = logits.sort(dim=1, descending=True).values
        margins.append(srt[:, top - 1] - srt[:, top] if top < E
                       else torch.full((h.shape[0],), math.inf, dtype=F64))
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(logits[i, e]), e))[:top]
        chosen = logits[i, order]
        wts = torch.softmax(chosen, dim=0)
        for w, e in zip(wts, order):
            out[i] += w * expert(h[i:i + 1], t, f"{p}e{e}.", rounding)[0]
    if mlp.get("shared"):
        out = out + expert(h, t, p + "shared.", rounding)
    return out


def forward(cfg: dict, t: Dict[str, torch.Tensor], tokens: List[int], rounding=None,
            layers_out: list = None, margins: list = None):
    """Float64 logits [len(tokens), vocab].  ``layers_out``: gets the sum of the stream's copies
    after every layer; ``margins``: gets every router's margins (``moe_ff``)."""
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    x = t["embed"].to(F64)[torch.tensor(tokens, dtype=torch.long)]
    xs = [x.clone() for _ in range(S or 1)]

    def sublayer(q: int, p: str, fn):
        nonlocal xs
        if S is None:
            xs = [xs[0] + fn(layer_norm(xs[0], t[f"{p}norm{q}"], eps))]
            return
        w_in = t[f"{p}hc{q}.in"].to(F64)
        w_out = t[f"{p}hc{q}.out"].to(F64)
        w_mix = t[f"{p}hc{q}.mix"].to(F64)              # [from, to]
        u = sum(w_in[s] * xs[s] for s in range(S))
        y = fn(layer_norm(u, t[f"{p}norm{q}"], eps))
        xs = [sum(w_mix[s, to] * xs[s] for s in range(S)) + w_out[to] * y for to in range(S)]

    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        kind, m, mlp = layer["type"], layer["mixer"], layer.get("mlp")
        if kind == "attention":
            sublayer(1, p, lambda h: attention(h, t, p + "mix.", m, eps, rounding))
        elif kind == "latent_attention":
            sublayer(1, p, lambda h: latent_attention(h, t, p + "mix.", m, eps, rounding))
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        if mlp is not None:
            if mlp["kind"] == "dense":
                sublayer(2, p, lambda h: dense_ff(h, t, p + "mlp.", rounding))
            else:
                sublayer(2, p, lambda h: moe_ff(h, t, p + "mlp.", mlp, rounding, margins))
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = layer_norm(sum(xs), t["final.norm"], eps)
    logits = matmul(x, t["head"], rounding)
    c = cfg.get("logit_softcap")
    return cap(logits, c) if c else logits
