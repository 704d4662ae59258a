"""Tiny Zumuzen configurations that differ in every size and option, and helpers that write them
as model folders with random weights and hold results to the plain implementation."""
from __future__ import annotations

import copy
import json

import numpy as np
import torch

from kappai_amd.config import config_from_dict
from kappai_amd.weights import write_random_model


def left(heads, kv_heads, dim, vdim, scale, base, dims, chunk, stretch=None):
    rot = {"base": base, "dims": dims}
    if stretch is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "scale": scale, "rot": rot,
           "mask": {"size": chunk}}
    if vdim is not None:
        out["vdim"] = vdim
    return out


def parallel(lt, r_heads, r_dim, r_vdim, decay, mlp):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": lt, "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim,
                                            "decay": decay}}}


def parallel_2(lt, r_heads, r_dim, rank, left_scale, right_scale, mlp):
    return {"type": "parallel_2", "mlp": mlp,
            "mixer": {"left": lt, "right": {"heads": r_heads, "dim": r_dim, "decay_rank": rank},
                      "left_scale": left_scale, "right_scale": right_scale}}


def rglru(width, blocks, conv, mlp):
    return {"type": "rglru", "mlp": mlp, "mixer": {"width": width, "blocks": blocks,
                                                   "conv": conv}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(vocab, width, eps, layers, loop=None):
    out = {"architecture": "Zumuzen", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# every mixer once, the last two passed twice; three query heads a kv head with values wider than
# keys, rotation over part of a head, chunks of 19 (no multiple of a page), scores so sharp that
# a key too many or too few decides; a real-gated unit of three blocks and three taps; stretched
# frequencies whose ramp lies inside the pairs; a layer without feed-forward
TINY_A = config(211, 72, 1e-5, [
    parallel(left(6, 2, 16, 24, 0.9, 9000.0, 8, 19), 3, 8, 16, [0.5, 0.97, 1.0], dense(80)),
    rglru(48, 3, 3, dense(64)),
    parallel_2(left(4, 2, 24, None, 0.7, 3000.0, 16, 33, (4.0, 64, 8.0, 1.0)), 3, 8, 5, 0.7, 1.3,
               None),
], loop=(1, 3, 2))
INIT_A = dict(seed=41, std=0.15, norm_jitter=0.1)

# the recurrent layer first and passed three times by itself; one tap; one block; chunks of one
# position (a token sees itself and, on the second side, the sink); no stretch; one kv head;
# rotation over the whole head; a decay of zero (the state is the token's own product)
TINY_B = config(97, 48, 1e-6, [
    rglru(40, 1, 1, dense(56)),
    parallel_2(left(4, 1, 8, 8, 0.5, 100.0, 8, 1), 1, 24, 3, 1.0, 0.25, dense(40)),
    parallel(left(1, 1, 24, 8, 0.4, 50.0, 24, 1000), 2, 40, 8, [0.0, 0.9], None),
], loop=(0, 1, 3))
INIT_B = dict(seed=42, std=0.2, norm_jitter=0.0)

# no loop; keys wider than one lane group of the recurrences (72 and 136 key channels); five
# taps; eight heads on eight kv heads; no rotation at all on one layer; a chunk that is a page
TINY_C = config(150, 64, 1e-5, [
    parallel_2(left(8, 8, 8, 8, 0.6, 10000.0, 0, 16), 2, 72, 4, 0.5, 0.5, dense(48)),
    parallel(left(2, 2, 16, 16, 0.35, 500.0, 2, 48), 1, 136, 8, [0.8], dense(32)),
    rglru(64, 8, 5, None),
    rglru(24, 2, 2, dense(32)),
])
INIT_C = dict(seed=43, std=0.12, norm_jitter=0.0)

# sizes in between: attention heads of 48, 80 and 96 once widened, four heads on one kv head, a
# width of 100 and a vocabulary of 301 (no multiples of eight), chunks of 50 and 70, every layer
# inside the passes, frequencies stretched over every pair
TINY_D = config(301, 100, 1e-5, [
    parallel(left(6, 3, 32, 48, 0.3, 15000.0, 32, 50), 4, 24, 40, [0.3, 0.6, 0.9, 0.99],
             dense(120)),
    parallel_2(left(4, 1, 80, 80, 0.2, 5000.0, 40, 70, (8.0, 32, 1000.0, 0.001)), 5, 20, 6, 0.9,
               0.6, dense(96)),
    rglru(60, 4, 4, dense(88)),
    parallel(left(2, 2, 96, 64, 0.15, 200.0, 96, 64), 2, 16, 16, [1.0, 0.5], None),
], loop=(0, 4, 2))
INIT_D = dict(seed=44, std=0.08, norm_jitter=0.05)

# wider: the time mixing first, heads of 32 and 64 that the matrix cores take as they are, values
# half as wide as keys, a real-gated unit of 256 channels in blocks of 64 (the matrix per block
# on the matrix cores) and one of a single block of 128, the two middle layers passed twice
TINY_E = config(500, 192, 1e-6, [
    parallel_2(left(6, 3, 32, 32, 0.25, 40000.0, 16, 40, (3.0, 128, 16.0, 2.0)), 3, 64, 16, 1.2,
               0.4, dense(256)),
    rglru(256, 4, 4, dense(224)),
    parallel(left(8, 2, 64, 32, 0.11, 200000.0, 64, 128), 4, 16, 48, [0.2, 0.7, 0.95, 0.999],
             dense(160)),
    rglru(128, 1, 3, None),
], loop=(1, 3, 2))
INIT_E = dict(seed=45, std=0.06, norm_jitter=0.05)

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
    from plain import zumuzen as plain
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


FP32_TOL = 3e-5


def assert_matches_plain(got, model_dir, requests, dtype, what=""):
    """float32: every row within FP32_TOL.  bfloat16: against what rounding the same values to
    bfloat16 costs the plain implementation itself.  Its root mean square row error is the yard:
    no row over six yards and at most one row in fifty over three.  Rows that rounding alone
    moves by more than two yards in the plain implementation are badly conditioned (a head's
    read-out that nearly cancels before it is divided by its root mean square, say): the error
    there is a draw from a wide spread, so such a row may err by eight times the plain one's own
    error."""
    ref = plain_logits(model_dir, requests)
    errs = row_errors(got, ref)
    worst = max(errs, key=errs.get)
    if dtype == "float32":
        assert errs[worst] < FP32_TOL, (what, worst, errs[worst])
        return
    own = row_errors({k: plain_logits(model_dir, requests, torch.bfloat16)[k[0]][k[1]]
                      for k in got}, ref)
    yard = float(np.sqrt(np.mean(np.square(list(own.values())))))
    touchy = {k for k in errs if own[k] > 2 * yard}

    def bound(k, yards):
        return max(yards * yard, 8.0 * own[k] if k in touchy else 1.5 * own[k])

    bad = [k for k, e in errs.items() if e > bound(k, 6)]
    over = [k for k, e in errs.items() if e > bound(k, 3)]
    assert not bad, (what, bad[:5], [errs[k] for k in bad[:5]], yard)
    assert len(over) <= max(1, len(errs) // 50), (what, len(over), len(errs), yard, over[:5])
