"""A plain, slow statement of the Zumuzen decoder in float64 torch on the CPU: one function per
mechanism, whole sequences, no cache and no state.  It shares nothing with the product path; the
tests hold the framework to it.

The model: ``x = E[token]``; a layer is ``x += mixer(n1(x))``, ``x += ff(n2(x))`` with plain RMS
norms; a run of layers may be passed several times with the same weights (before every pass but
the first the embedded rows are added again, and before every pass a learned row of that pass).
Three mixers:

* ``parallel``: a softmax attention over chunks of positions (grouped heads, biases, rotation of
  the first places of a head) beside a linear attention with one fixed decay a head; each side's
  output is normed over the model width, and the two are averaged;
* ``rglru``: a gated branch times a linear recurrence with a gate per channel made by
  block-diagonal maps, behind a short causal convolution;
* ``parallel_2``: a softmax attention over chunks whose values are its unrotated keys, with
  stretched rotation frequencies and a sink, beside a time mixing with a matrix of state per
  head, a decay per key channel made from the token and a bonus for the token itself; the two
  are added with weights.

``rounding=torch.bfloat16`` rounds where a bfloat16 run rounds (inputs and outputs of matrix
products and convolutions), the yardstick for the error that rounding alone costs.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def _r(x, rounding):
    return x if rounding is None else x.to(rounding).to(F64)


def matmul(x, w, rounding=None, bias=None):
    y = _r(x, rounding) @ w.to(F64).T
    if bias is not None:
        y = y + bias.to(F64)
    return _r(y, rounding)


def rms(x, eps: float):
    return torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm(x, w, eps: float):
    return x / rms(x, eps) * w.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ---------------------------------------------------------------------------------------
# rotation
# ---------------------------------------------------------------------------------------
def rotation_frequencies(rot: dict):
    """Frequencies of the pairs and the factor on cosine and sine.  With ``scaling`` the
    frequencies between two wavelengths are blended towards ``f / factor``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def place(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(place(float(sc["fast"]))), 0)
    hi = min(math.ceil(place(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((torch.arange(half, dtype=F64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot: dict):
    """``x`` [T, heads, dim]: the first ``dims`` places of every head turn by the position, place
    i paired with place i + dims/2."""
    dims = int(rot["dims"])
    half = dims // 2
    f, mag = rotation_frequencies(rot)
    ang = positions.to(F64)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------------------------------
# attention over chunks
# ---------------------------------------------------------------------------------------
def chunk_mask(T: int, size: int):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i // size) == (j // size))


def chunked_attention(h, W, p: str, m: dict, rounding=None):
    """The softmax side.  ``W[p + 'v']`` missing: the values are the keys before rotation."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = matmul(h, W[p + "q"], rounding, W[p + "q.b"]).reshape(T, H, d)
    k = matmul(h, W[p + "k"], rounding, W[p + "k.b"]).reshape(T, G, d)
    if p + "v" in W:
        dv = int(m["vdim"])
        v = matmul(h, W[p + "v"], rounding, W[p + "v.b"]).reshape(T, G, dv)
    else:
        dv, v = d, k
    pos = torch.arange(T)
    q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    q, k = _r(q, rounding), _r(k, rounding)
    seen = chunk_mask(T, int(m["mask"]["size"]))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~seen, -math.inf)
        top = s.max(dim=-1, keepdim=True).values
        extra = 0.0
        if p + "sink" in W:
            sink = W[p + "sink"].to(F64)[hd]
            top = torch.maximum(top, sink)
            extra = torch.exp(sink - top)
        e = torch.exp(s - top)
        out[:, hd] = (e / (e.sum(dim=-1, keepdim=True) + extra)) @ v[:, g]
    return matmul(out.reshape(T, H * dv), W[p + "o"], rounding)


# ---------------------------------------------------------------------------------------
# linear attention with a fixed decay a head
# ---------------------------------------------------------------------------------------
def fixed_decay_attention(h, W, p: str, m: dict, eps: float, rounding=None):
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(matmul(h, W[p + "q"], rounding)).reshape(T, H, d)
    k = silu(matmul(h, W[p + "k"], rounding)).reshape(T, H, d)
    v = silu(matmul(h, W[p + "v"], rounding)).reshape(T, H, dv)
    gate = torch.sigmoid(matmul(h, W[p + "g"], rounding))
    decay = [float(a) for a in m["decay"]]
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = decay[hd] * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    y = norm(out.reshape(T, H * dv), W[p + "norm"], eps) * gate
    return matmul(y, W[p + "o"], rounding)


# ---------------------------------------------------------------------------------------
# gated linear recurrence per channel
# ---------------------------------------------------------------------------------------
def causal_conv(x, taps, bias):
    """``x`` [T, C], ``taps`` [C, n]: the last column weighs the token itself; zeros before the
    start."""
    T, C = x.shape
    n = taps.shape[1]
    pad = torch.cat([torch.zeros(n - 1, C, dtype=F64), x], dim=0)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(n):
        y = y + pad[j:j + T] * taps.to(F64)[:, j]
    return y + bias.to(F64)


def gated_channel_recurrence(h, W, p: str, m: dict, rounding=None):
    T = h.shape[0]
    C, B = int(m["width"]), int(m["blocks"])
    y = _r(gelu_tanh(matmul(h, W[p + "y"], rounding, W[p + "y.b"])), rounding)
    u = _r(causal_conv(matmul(h, W[p + "x"], rounding, W[p + "x.b"]), W[p + "conv"],
                       W[p + "conv.b"]), rounding)
    ub = u.reshape(T, B, C // B)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, W[p + "ra"].to(F64))
                      + W[p + "ra.b"].to(F64)).reshape(T, C)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, W[p + "ri"].to(F64))
                      + W[p + "ri.b"].to(F64)).reshape(T, C)
    a = torch.exp(-8.0 * r * softplus(W[p + "lam"].to(F64)))
    b = torch.sqrt(1.0 - a * a) * i * u
    S = torch.zeros(C, dtype=F64)
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        S = a[t] * S + b[t]
        out[t] = S
    return matmul(out * y, W[p + "o"], rounding)


# ---------------------------------------------------------------------------------------
# time mixing with a decay per key channel and a bonus for the token itself
# ---------------------------------------------------------------------------------------
def bonus_time_mixing(h, W, p: str, m: dict, eps: float, rounding=None):
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    before = torch.cat([torch.zeros(1, h.shape[1], dtype=F64), h[:-1]], dim=0)

    def mixed(s):
        return h + (before - h) * W[p + "mu." + s].to(F64)

    r = matmul(mixed("r"), W[p + "r"], rounding).reshape(T, H, d)
    k = matmul(mixed("k"), W[p + "k"], rounding).reshape(T, H, d)
    v = matmul(mixed("v"), W[p + "v"], rounding).reshape(T, H, d)
    gate = silu(matmul(mixed("g"), W[p + "g"], rounding))
    z = matmul(torch.tanh(matmul(mixed("w"), W[p + "w1"], rounding)), W[p + "w2"], rounding)
    w = torch.exp(-torch.exp(z + W[p + "w0"].to(F64))).reshape(T, H, d)
    u = W[p + "u"].to(F64)
    out = torch.zeros(T, H, d, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(T):
            kv = torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = (S + u[hd][:, None] * kv).T @ r[t, hd]
            S = w[t, hd][:, None] * S + kv
    out = out / rms(out, eps)
    y = out.reshape(T, H * d) * W[p + "norm"].to(F64) * gate
    return matmul(y, W[p + "o"], rounding)


# ---------------------------------------------------------------------------------------
# the layers and the model
# ---------------------------------------------------------------------------------------
def mixer(kind: str, h, W, p: str, m: dict, eps: float, rounding=None):
    if kind == "rglru":
        return gated_channel_recurrence(h, W, p, m, rounding)
    left = chunked_attention(h, W, p + "left.", m["left"], rounding)
    if kind == "parallel":
        right = fixed_decay_attention(h, W, p + "right.", m["right"], eps, rounding)
        return 0.5 * (norm(left, W[p + "left.out"], eps) + norm(right, W[p + "right.out"], eps))
    if kind == "parallel_2":
        right = bonus_time_mixing(h, W, p + "right.", m["right"], eps, rounding)
        return float(m["left_scale"]) * left + float(m["right_scale"]) * right
    raise ValueError(kind)


def feed_forward(h, W, p: str, rounding=None):
    g = matmul(h, W[p + "gate"], rounding)
    u = matmul(h, W[p + "up"], rounding)
    return matmul(silu(g) * u, W[p + "down"], rounding)


def layer_order(config: dict) -> List[tuple]:
    """(layer, pass number or None) in the order they run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def forward(config: dict, W: Dict[str, torch.Tensor], tokens, rounding=None,
            streams: Optional[list] = None):
    """Logits [T, vocab] in float64.  ``streams``: a list that receives the stream after every
    run of a layer."""
    eps = float(config["norm"]["eps"])
    x0 = W["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    for i, enters in layer_order(config):
        if enters is not None:
            if enters > 0:
                x = x + x0
            x = x + W["loop.step"].to(F64)[enters]
        layer = config["layers"][i]
        p = f"l{i}."
        h = _r(norm(x, W[p + "norm1"], eps), rounding)
        x = x + mixer(layer["type"], h, W, p + "mix.", layer["mixer"], eps, rounding)
        if layer.get("mlp") is not None:
            h = _r(norm(x, W[p + "norm2"], eps), rounding)
            x = x + feed_forward(h, W, p + "mlp.", rounding)
        if streams is not None:
            streams.append(x.clone())
    h = _r(norm(x, W["final.norm"], eps), rounding)
    return matmul(h, W["head"], rounding)
