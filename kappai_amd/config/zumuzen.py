"""Configuration of the Zumuzen decoder: a list of pre-norm layers, each with one of three mixers
and an optional dense feed-forward, a run of which may be passed several times.

config.json names the design under ``architecture`` and nests its keys::

    {"architecture": "Zumuzen", "vocab": V, "width": D, "norm": {"eps": e},
     "loop": {"start": a, "stop": b, "times": n},
     "layers": [
       {"type": "parallel",
        "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale",
                           "rot": {"base", "dims"}, "mask": {"size"}},
                  "right": {"heads", "dim", "vdim", "decay": [one a head]}},
        "mlp": {"kind": "dense", "ff": F}},
       {"type": "rglru", "mixer": {"width", "blocks", "conv"}, "mlp": ...},
       {"type": "parallel_2",
        "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale",
                           "rot": {"base", "dims", "scaling": {"factor", "original", "fast",
                                                               "slow"}},
                           "mask": {"size"}},
                  "right": {"heads", "dim"}, "left_scale": a, "right_scale": b},
        "mlp": null}]}

``loop`` may be left out (every layer runs once).  The rank of the low-rank map behind the
decay of a ``parallel_2`` layer (``right.decay_rank``) may be left out of the file: the tensors'
shapes then give it (``adopt_tensor_shapes``); a file for the random-weights mode states it.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, KeyReader, ModelConfig

ARCHITECTURE = "Zumuzen"

MIXER_TYPES = ("parallel", "rglru", "parallel_2")


@dataclass
class ZumuzenLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]               # None: the layer has no feed-forward


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.raw.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: required key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _positive(where: str, **values) -> None:
    for name, v in values.items():
        if v < 1:
            raise ConfigError(f"{where}: mixer.{name} must be positive, got {v}")


def _chunked_attention(left: KeyReader, where: str, values_are_keys: bool) -> Dict[str, Any]:
    rot, mask = _sub(left, "rot"), _sub(left, "mask")
    out = {"heads": left.int("heads"), "kv_heads": left.int("kv_heads"), "dim": left.int("dim"),
           "scale": left.float("scale"), "rot_base": rot.float("base"),
           "rot_dims": rot.int("dims"), "stretch": None, "chunk": mask.int("size")}
    # (values that are the keys have the keys' size, whatever the file says of them)
    out["vdim"] = out["dim"] if values_are_keys else left.int("vdim")
    _positive(where + " left", heads=out["heads"], kv_heads=out["kv_heads"], dim=out["dim"],
              vdim=out["vdim"])
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{where}: {out['heads']} heads cannot be shared out over "
                          f"{out['kv_heads']} kv heads")
    if out["rot_dims"] < 0 or out["rot_dims"] % 2 or out["rot_dims"] > out["dim"]:
        raise ConfigError(f"{where}: mixer.left.rot.dims ({out['rot_dims']}) must be even and at "
                          f"most mixer.left.dim ({out['dim']})")
    if out["chunk"] < 1:
        raise ConfigError(f"{where}: mixer.left.mask.size must be at least 1")
    if rot.raw.get("scaling") is not None:
        sc = _sub(rot, "scaling")
        out["stretch"] = {k: sc.float(k) for k in ("factor", "original", "fast", "slow")}
        if min(out["stretch"].values()) <= 0.0:
            raise ConfigError(f"{where}: mixer.left.rot.scaling holds positive numbers")
    return out


def _parallel(m: KeyReader, where: str) -> Dict[str, Any]:
    right = _sub(m, "right")
    decay = right.raw.get("decay")
    rt = {"heads": right.int("heads"), "dim": right.int("dim"), "vdim": right.int("vdim")}
    _positive(where + " right", heads=rt["heads"], dim=rt["dim"], vdim=rt["vdim"])
    if (not isinstance(decay, list) or len(decay) != rt["heads"]
            or not all(isinstance(a, (int, float)) and not isinstance(a, bool)
                       and 0.0 <= a <= 1.0 for a in decay)):
        raise ConfigError(f"{where}: mixer.right.decay must list one number between 0 and 1 for "
                          f"each of the {rt['heads']} heads")
    rt["decay"] = [float(a) for a in decay]
    return {"left": _chunked_attention(_sub(m, "left"), where, False), "right": rt}


def _parallel_2(m: KeyReader, where: str) -> Dict[str, Any]:
    right = _sub(m, "right")
    rt = {"heads": right.int("heads"), "dim": right.int("dim"),
          "decay_rank": right.int("decay_rank", None)}
    _positive(where + " right", heads=rt["heads"], dim=rt["dim"])
    return {"left": _chunked_attention(_sub(m, "left"), where, True), "right": rt,
            "left_scale": m.float("left_scale"), "right_scale": m.float("right_scale")}


def _rglru(m: KeyReader, where: str) -> Dict[str, Any]:
    out = {"width": m.int("width"), "blocks": m.int("blocks"), "conv": m.int("conv")}
    _positive(where, width=out["width"], blocks=out["blocks"], conv=out["conv"])
    if out["width"] % out["blocks"]:
        raise ConfigError(f"{where}: mixer.width ({out['width']}) cannot be cut into "
                          f"{out['blocks']} equal blocks")
    return out


def _layer(raw: Any, i: int) -> ZumuzenLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(raw, where)
    kind = raw.get("type")
    if kind not in MIXER_TYPES:
        raise ConfigError(f"{where}: type = {kind!r}; known: {', '.join(MIXER_TYPES)}")
    mixer = {"parallel": _parallel, "rglru": _rglru, "parallel_2": _parallel_2}[kind](
        _sub(r, "mixer"), where)
    mlp = None
    if raw.get("mlp") is not None:
        f = _sub(r, "mlp")
        if f.raw.get("kind") != "dense":
            raise ConfigError(f"{where}: mlp.kind = {f.raw.get('kind')!r}; known: dense")
        mlp = {"kind": "dense", "ff": f.int("ff")}
        if mlp["ff"] < 1:
            raise ConfigError(f"{where}: the feed-forward width must be positive")
    return ZumuzenLayer(kind, mixer, mlp)


@dataclass
class ZumuzenConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 0.0
    layers: List[ZumuzenLayer] = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    max_position_embeddings: int = 0
    eos_token_id: Optional[Union[int, List[int]]] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ZumuzenConfig":
        r = KeyReader(raw)
        cfg = cls(
            architecture=ARCHITECTURE,
            vocab_size=r.int("vocab"),
            width=r.int("width"),
            norm_eps=_sub(r, "norm").float("eps"),
            layers=[_layer(x, i) for i, x in enumerate(r.list("layers"))],
            eos_token_id=r.int_or_ints("eos_token_id", None),
            raw=copy.deepcopy(raw),
        )
        if cfg.vocab_size < 1 or cfg.width < 1:
            raise ConfigError("config.json: vocab and width must be positive")
        if not cfg.layers:
            raise ConfigError("config.json: layers must name at least one layer")
        if cfg.norm_eps <= 0.0:
            raise ConfigError("config.json: norm.eps must be positive")
        if raw.get("loop") is not None:
            lp = _sub(r, "loop")
            cfg.loop_start, cfg.loop_stop = lp.int("start"), lp.int("stop")
            cfg.loop_times = lp.int("times")
            if not 0 <= cfg.loop_start < cfg.loop_stop <= len(cfg.layers) or cfg.loop_times < 1:
                raise ConfigError(
                    f"config.json: loop runs layers {cfg.loop_start} to {cfg.loop_stop} - 1 "
                    f"{cfg.loop_times} times; there are {len(cfg.layers)} layers")
        return cfg

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    def adopt_tensor_shapes(self, shapes: Dict[str, tuple]) -> None:
        """Fill in the sizes that the file leaves to the tensors: the rank of the low-rank map
        behind a decay.  A size that config.json states is kept."""
        for i, layer in enumerate(self.layers):
            if layer.type != "parallel_2" or layer.mixer["right"].get("decay_rank") is not None:
                continue
            name = f"l{i}.mix.right.w1"
            if name not in shapes or not shapes[name]:
                raise ConfigError(f"config.json: layers[{i}] mixer.right.decay_rank is neither "
                                  f"stated nor given by a tensor '{name}'")
            layer.mixer["right"]["decay_rank"] = int(shapes[name][0])

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
