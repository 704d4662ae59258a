"""Tiny Sibodra configurations that differ in every size and option, and helpers that write them
as model folders with random weights and hold results to the plain implementation."""
from __future__ import annotations

import copy
import json

import numpy as np
import torch

from kappai_amd.config import config_from_dict
from kappai_amd.weights import write_random_model


def attention(heads, kv_heads, dim, vdim, scale, softcap, base, dims, scaling, mlp):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "rot": rot}
    if softcap is not None:
        mixer["softcap"] = softcap
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, mlp):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim}}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def config(vocab, width, eps, streams, logit_softcap, layers):
    out = {"architecture": "Sibodra", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": layers}
    if streams is not None:
        out["streams"] = streams
    if logit_softcap is not None:
        out["logit_softcap"] = logit_softcap
    return out


# three copies of the stream; three query heads a kv head, values wider than keys, a rotation
# over part of the head with scaled frequencies whose blended band holds some pairs; a latent
# attention with five heads; experts with a shared one of another size; a layer without
# feed-forward
TINY_A = config(211, 72, 1e-5, 3, 12.0, [
    attention(6, 2, 16, 24, 0.2, 8.0, 100.0, 12, (4.0, 1.0, 4.0, 64), dense(80)),
    latent(5, 16, 8, 24, 20, 28, 0.21, 9000.0, moe(24, 6, 2, shared=40)),
    attention(3, 3, 24, 16, 0.15, 30.0, 5000.0, 24, None, None),
    latent(2, 8, 16, 8, 40, 12, 0.3, 50.0, moe(16, 4, 1)),
])
INIT_A = dict(seed=41, std=0.15, norm_jitter=0.1)

# one copy of the stream with connection weights; the latent attention first; no cap on scores or
# logits; one head on one kv head; every expert used by every token (top = experts)
TINY_B = config(97, 48, 1e-6, 1, None, [
    latent(3, 16, 4, 16, 8, 8, 0.25, 10000.0, dense(56)),
    attention(1, 1, 40, 8, 0.3, None, 1000.0, 8, (8.0, 1.0, 2.0, 32), moe(8, 3, 3, shared=8)),
    attention(4, 1, 8, 8, 0.35, 0.5, 10000.0, 8, None, dense(40)),
])
INIT_B = dict(seed=42, std=0.2, norm_jitter=0.1)

# no "streams" key at all: the plain residual sum and no connection tensors; four copies in the
# next one, a width that is no multiple of 8, heads that are 48 and 80 wide once widened
TINY_C = config(150, 64, 1e-5, None, 30.0, [
    attention(8, 8, 8, 8, 0.35, 20.0, 300.0, 4, None, moe(32, 8, 3)),
    latent(4, 24, 8, 16, 24, 16, 0.18, 300.0, dense(48)),
])
INIT_C = dict(seed=43, std=0.12, norm_jitter=0.1)

TINY_D = config(500, 100, 1e-5, 4, 25.0, [
    attention(6, 3, 32, 48, 0.17, 15.0, 10000.0, 16, (8.0, 1.0, 4.0, 128), moe(40, 10, 4, 24)),
    latent(5, 32, 16, 40, 64, 48, 0.14, 5000.0, dense(200)),
    latent(2, 16, 32, 16, 48, 20, 0.2, 20000.0, None),
    attention(4, 1, 64, 64, 0.125, 50.0, 500000.0, 64, (16.0, 1.0, 4.0, 256), dense(128)),
])
INIT_D = dict(seed=44, std=0.08, norm_jitter=0.1)

# a width, a vocabulary and head sizes that are multiples of nothing: no kernel takes 16 bytes at
# a time here; two copies of the stream
TINY_E = config(131, 54, 1e-5, 2, 9.0, [
    latent(3, 10, 6, 14, 11, 9, 0.22, 777.0, moe(10, 5, 2, shared=6)),
    attention(3, 1, 10, 6, 0.3, 6.0, 1234.0, 4, (3.0, 1.0, 3.0, 16), dense(34)),
])
INIT_E = dict(seed=45, std=0.2, norm_jitter=0.1)

TINY = {"A": (TINY_A, INIT_A), "B": (TINY_B, INIT_B), "C": (TINY_C, INIT_C),
        "D": (TINY_D, INIT_D), "E": (TINY_E, INIT_E)}


def write_tiny(name: str, folder, **overrides):
    cfg, init = TINY[name]
    return write_random_model(folder, config_from_dict(copy.deepcopy(cfg)), **{**init, **overrides})


def read_model_dir(model_dir):
    """(config dictionary, {name: tensor}) of a model folder, for the plain implementation."""
    from kappai_amd.weights.safetensors_io import SafetensorsFile
    cfg = json.loads((model_dir / "config.json").read_text())
    f = SafetensorsFile(model_dir / "model.safetensors")
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    return cfg, tensors


_plain_cache = {}


def plain_logits(model_dir, requests, rounding=None):
    """{id: float64 numpy [len, vocab]} from the plain implementation (cached per folder)."""
    from plain import sibodra as plain
    key = (str(model_dir), json.dumps(requests, sort_keys=True), str(rounding))
    if key not in _plain_cache:
        cfg, t = read_model_dir(model_dir)
        _plain_cache[key] = {rid: plain.forward(cfg, t, toks, rounding=rounding).numpy()
                             for rid, toks in requests.items()}
    return _plain_cache[key]


def row_errors(got, ref):
    """{(id, pos): error of the row}: root mean square of the difference with its mean taken off,
    over the root mean square of all reference logits."""
    scale = float(np.sqrt(np.mean([np.mean(v * v) for v in ref.values()])))
    out = {}
    for (rid, pos), row in got.items():
        assert np.isfinite(row).all(), f"non-finite logits at {rid} position {pos}"
        d = row.astype(np.float64) - ref[rid][pos]
        d = d - d.mean()
        out[(rid, pos)] = float(np.sqrt((d * d).mean())) / scale
    return out


FP32_TOL = 2e-5
CLOSE_CALL = 0.05       # a router's margin below this may go the other way in bfloat16


def first_close_calls(model_dir, requests):
    """{id: the first position at which some router of the model makes a close call} (the
    request's length when none does).  From there on a bfloat16 run may have chosen another
    expert, which the keys and values of that position carry to every later one."""
    from plain import sibodra as plain
    cfg, t = read_model_dir(model_dir)
    out = {}
    for rid, toks in requests.items():
        margins = []
        plain.forward(cfg, t, toks, margins=margins)
        first = len(toks)
        for m in margins:
            close = (m < CLOSE_CALL).nonzero().flatten()
            if close.numel():
                first = min(first, int(close[0]))
        out[rid] = first
    return out


def assert_matches_plain(got, model_dir, requests, dtype, what="", min_strict=0.1):
    """float32: every row within FP32_TOL.  bfloat16: against what rounding the same values to
    bfloat16 costs the plain implementation itself: no row over six times its root mean square
    row error and at most one row in fifty over three times (but for rows where the plain
    implementation's own rounding error is that large too), for the rows before a request's first
    close call of a router (at least ``min_strict`` of all rows must be such); the rows behind it
    must stay finite and within twice the logits' own size (another expert may have been chosen,
    rightly, and where one expert is chosen its whole output changes)."""
    ref = plain_logits(model_dir, requests)
    errs = row_errors(got, ref)
    worst = max(errs, key=errs.get)
    if dtype == "float32":
        assert errs[worst] < FP32_TOL, (what, worst, errs[worst])
        return
    own = row_errors({k: plain_logits(model_dir, requests, torch.bfloat16)[k[0]][k[1]]
                      for k in got}, ref)
    yard = float(np.sqrt(np.mean(np.square(list(own.values())))))
    close = first_close_calls(model_dir, requests)
    strict = {k: e for k, e in errs.items() if k[1] < close[k[0]]}
    assert len(strict) >= len(errs) * min_strict, (what, "too few rows before a close call",
                                                   len(strict), len(errs))
    bad = [k for k, e in strict.items() if e > max(6 * yard, 1.5 * own[k])]
    over = [k for k, e in strict.items() if e > max(3 * yard, 1.5 * own[k])]
    assert not bad, (what, bad[:5], [errs[k] for k in bad[:5]], yard)
    assert len(over) <= max(1, len(strict) // 50), (what, len(over), len(strict), yard, over[:5])
    assert max(errs.values()) < 2.0, (what, max(errs, key=errs.get), max(errs.values()))
