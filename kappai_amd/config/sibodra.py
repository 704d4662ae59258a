"""Configuration of the Sibodra decoder: a list of pre-norm layers (layer norms without bias), each
with a grouped-query or a latent attention and a dense or routed feed-forward, around a residual
stream that may be kept in several copies ("hyper-connections").

config.json names the design under ``architecture`` and nests its keys::

    {"architecture": "Sibodra", "vocab": V, "width": D, "norm": {"eps": e}, "streams": S,
     "logit_softcap": c,
     "layers": [
       {"type": "attention",
        "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap",
                  "rot": {"base", "dims", "scaling": {"factor", "low", "high", "original"}}},
        "mlp": {"kind": "dense", "ff": F}},
       {"type": "latent_attention",
        "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale",
                  "rot": {"base", "dims"}},
        "mlp": {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": k},
                "shared": {"ff": Fs}}}]}

``streams`` absent: one stream with the plain residual sum (no connection weights in the file).
``softcap``, ``logit_softcap``, ``rot.scaling``, ``mlp.shared`` and ``mlp`` itself may be absent
or null.  ``q_rank`` may be left to the tensors' shapes (``adopt_tensor_shapes``).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, KeyReader, ModelConfig

ARCHITECTURE = "Sibodra"

MIXER_TYPES = ("attention", "latent_attention")


@dataclass
class SibodraLayer:
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
            raise ConfigError(f"{where}: {name} must be positive, got {v}")


def _rotation(m: KeyReader, where: str, most: int) -> Optional[Dict[str, Any]]:
    """``rot``: base, rotated places, and the optional stretch of the frequencies."""
    if m.raw.get("rot") is None:
        return None
    rot = _sub(m, "rot")
    out = {"base": rot.float("base"), "dims": rot.int("dims"), "scaling": None}
    if out["dims"] % 2 or not 0 <= out["dims"] <= most:
        raise ConfigError(f"{where}: mixer.rot.dims ({out['dims']}) must be even and at most "
                          f"{most}")
    if out["base"] <= 0.0:
        raise ConfigError(f"{where}: mixer.rot.base must be positive")
    if rot.raw.get("scaling") is not None:
        s = _sub(rot, "scaling")
        sc = {k: s.float(k) for k in ("factor", "low", "high", "original")}
        if sc["factor"] <= 0.0 or sc["original"] <= 0.0 or not sc["high"] > sc["low"] > 0.0:
            raise ConfigError(f"{where}: mixer.rot.scaling needs a positive factor and original "
                              f"length and high > low > 0, got {sc}")
        out["scaling"] = sc
    return out if out["dims"] else None


def _attention(m: KeyReader, where: str) -> Dict[str, Any]:
    out = {"heads": m.int("heads"), "kv_heads": m.int("kv_heads"), "dim": m.int("dim"),
           "vdim": m.int("vdim"), "scale": m.float("scale"),
           "softcap": m.float("softcap", 0.0) or 0.0}
    _positive(where, heads=out["heads"], kv_heads=out["kv_heads"], dim=out["dim"],
              vdim=out["vdim"])
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{where}: {out['heads']} heads cannot be shared out over "
                          f"{out['kv_heads']} kv heads")
    if out["softcap"] < 0.0:
        raise ConfigError(f"{where}: mixer.softcap must not be negative")
    out["rot"] = _rotation(m, where, out["dim"])
    return out


def _latent(m: KeyReader, where: str) -> Dict[str, Any]:
    out = {"heads": m.int("heads"), "dim": m.int("dim"), "rot_dim": m.int("rot_dim"),
           "vdim": m.int("vdim"), "kv_rank": m.int("kv_rank"), "q_rank": m.int("q_rank", None),
           "scale": m.float("scale")}
    _positive(where, heads=out["heads"], dim=out["dim"], vdim=out["vdim"],
              kv_rank=out["kv_rank"])
    if out["rot_dim"] < 0:
        raise ConfigError(f"{where}: mixer.rot_dim must not be negative")
    out["rot"] = _rotation(m, where, out["rot_dim"])
    return out


def _mlp(f: KeyReader, where: str) -> Dict[str, Any]:
    kind = f.raw.get("kind")
    if kind == "dense":
        out = {"kind": "dense", "ff": f.int("ff")}
        _positive(where, **{"mlp.ff": out["ff"]})
        return out
    if kind != "moe":
        raise ConfigError(f"{where}: mlp.kind = {kind!r}; known: dense, moe")
    router = _sub(f, "router")
    out = {"kind": "moe", "ff": _sub(f, "expert").int("ff"), "experts": router.int("experts"),
           "top": router.int("top"), "shared_ff": None}
    if f.raw.get("shared") is not None:
        out["shared_ff"] = _sub(f, "shared").int("ff")
        _positive(where, **{"mlp.shared.ff": out["shared_ff"]})
    _positive(where, **{"mlp.expert.ff": out["ff"], "mlp.router.experts": out["experts"],
                        "mlp.router.top": out["top"]})
    if out["top"] > out["experts"]:
        raise ConfigError(f"{where}: mlp.router.top ({out['top']}) exceeds mlp.router.experts "
                          f"({out['experts']})")
    return out


def _layer(raw: Any, i: int) -> SibodraLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(raw, where)
    kind = raw.get("type")
    if kind not in MIXER_TYPES:
        raise ConfigError(f"{where}: type = {kind!r}; known: {', '.join(MIXER_TYPES)}")
    mixer = {"attention": _attention, "latent_attention": _latent}[kind](_sub(r, "mixer"), where)
    mlp = _mlp(_sub(r, "mlp"), where) if raw.get("mlp") is not None else None
    return SibodraLayer(kind, mixer, mlp)


@dataclass
class SibodraConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 0.0
    streams: Optional[int] = None               # None: one stream, plain residual sums
    logit_softcap: float = 0.0                  # 0: the logits pass as they are
    layers: List[SibodraLayer] = field(default_factory=list)
    max_position_embeddings: int = 0
    eos_token_id: Optional[Union[int, List[int]]] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "SibodraConfig":
        r = KeyReader(raw)
        cfg = cls(
            architecture=ARCHITECTURE,
            vocab_size=r.int("vocab"),
            width=r.int("width"),
            norm_eps=_sub(r, "norm").float("eps"),
            streams=r.int("streams", None),
            logit_softcap=r.float("logit_softcap", 0.0) or 0.0,
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
        if cfg.streams is not None and cfg.streams < 1:
            raise ConfigError("config.json: streams must be at least 1")
        if cfg.logit_softcap < 0.0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        return cfg

    def adopt_tensor_shapes(self, shapes: Dict[str, tuple]) -> None:
        """The rank of the queries' latent is the row count of its map where the file leaves it
        out.  A size that config.json states is kept."""
        for i, layer in enumerate(self.layers):
            if layer.type == "latent_attention" and layer.mixer.get("q_rank") is None:
                name = f"l{i}.mix.dq"
                if name not in shapes or not shapes[name]:
                    raise ConfigError(f"config.json: layers[{i}] mixer.q_rank is neither stated "
                                      f"nor given by a tensor '{name}'")
                layer.mixer["q_rank"] = int(shapes[name][0])

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
