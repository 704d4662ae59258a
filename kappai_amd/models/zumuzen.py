"""The Zumuzen decoder put together from parts.

Every layer is ``block.pre_norm`` (plain RMS norms) around one of three mixers: a softmax
attention over chunks of positions beside a linear attention with a fixed decay a head, each
side normed over the model width and the two averaged (``mixer.parallel`` with side norms); a
recurrent block around a real-gated linear unit; or a softmax attention over chunks whose values
are its keys, with stretched rotation frequencies and a sink, beside a time mixing with a bonus
for the token itself, added with two weights.  The feed-forward is a SiLU-gated dense layer.  A
run of layers may be passed several times: the schedule names those blocks once a pass (so every
pass has caches of its own) and the first call of a pass enters through a ``PassEntry``.  Tensor
names: ``embed``, ``loop.step``, ``final.norm``, ``head`` and per layer ``l<i>.norm1|norm2``,
``l<i>.mix.*``, ``l<i>.mlp.*``; no name ends in ``.weight``, biases end in ``.b``.
"""
from __future__ import annotations

import torch

from ..config.base import register_architecture
from ..config.zumuzen import ARCHITECTURE, ZumuzenConfig
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.passes import PassEntry
from .base import LayerCall, Model

HALF = 0.5      # the two sides of a "parallel" mixer are averaged


def _chunked_attention(lt: dict, p: str, width: int, eps: float, dtype, values_from_keys: bool):
    position = None
    if lt["rot_dims"]:
        position = make_part("position_encoding", "rotary", head_dim=lt["dim"],
                             theta=lt["rot_base"], rot_dim=lt["rot_dims"], pairing="half",
                             stretch=lt["stretch"])
    return make_part(
        "mixer", "scored_attention", prefix=p, width=width, num_heads=lt["heads"],
        num_kv_heads=lt["kv_heads"], dim=lt["dim"], vdim=lt["vdim"], scale=lt["scale"],
        dtype=dtype, norm_eps=eps, sink=values_from_keys, chunk=lt["chunk"], position=position,
        bias=True, bias_suffix=".b", weight_suffix="", values_from_keys=values_from_keys)


def _mixer(kind: str, m: dict, p: str, width: int, eps: float, dtype):
    if kind == "parallel":
        rt = m["right"]
        left = _chunked_attention(m["left"], p + "left.", width, eps, dtype, False)
        right = make_part("mixer", "fixed_decay_attention", prefix=p + "right.", width=width,
                          num_heads=rt["heads"], dim=rt["dim"], vdim=rt["vdim"],
                          decay=rt["decay"], norm_eps=eps, dtype=dtype, weight_suffix="")
        return make_part("mixer", "parallel", left=left, right=right, left_scale=HALF,
                         right_scale=HALF, side_norms=(p + "left.out", p + "right.out"),
                         width=width, norm_eps=eps)
    if kind == "parallel_2":
        rt = m["right"]
        if rt.get("decay_rank") is None:
            raise ValueError("config.json does not state mixer.right.decay_rank, and no tensor "
                             "shapes were read that could give it")
        left = _chunked_attention(m["left"], p + "left.", width, eps, dtype, True)
        right = make_part("mixer", "bonus_time_mixing", prefix=p + "right.", width=width,
                          num_heads=rt["heads"], dim=rt["dim"], decay_rank=rt["decay_rank"],
                          norm_eps=eps, dtype=dtype, weight_suffix="")
        return make_part("mixer", "parallel", left=left, right=right,
                         left_scale=m["left_scale"], right_scale=m["right_scale"], summed=True)
    return make_part("mixer", "real_gated_unit", prefix=p, width=width, inner=m["width"],
                     blocks=m["blocks"], taps=m["conv"], dtype=dtype, rate=8.0,
                     weight_suffix="", bias_suffix=".b")


def build_zumuzen(config: ZumuzenConfig, dtype: torch.dtype) -> Model:
    width, eps = config.width, config.norm_eps

    def norm(name):
        return make_part("norm", "rmsnorm", name=name, width=width, eps=eps, dtype=dtype,
                         suffix="")

    layers, unused = [], []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        mixer = _mixer(layer.type, layer.mixer, p + "mix.", width, eps, dtype)
        feed_forward = ffn_norm = None
        if layer.mlp is not None:
            feed_forward = make_part("feed_forward", "swiglu", prefix=p + "mlp.", width=width,
                                     hidden=layer.mlp["ff"], dtype=dtype, activation="silu",
                                     names={"gate": "gate", "up": "up", "down": "down"},
                                     weight_suffix="")
            ffn_norm = norm(p + "norm2")
        else:
            unused.append(p + "norm2")
        layers.append(make_part("block", "pre_norm", mixer_norm=norm(p + "norm1"), mixer=mixer,
                                ffn_norm=ffn_norm, feed_forward=feed_forward))
    # the order of the calls: the layers before the run once, the run `times` times (its first
    # call of every pass enters through that pass's entry), the rest once
    entries, schedule = [], []
    n, a, b = len(layers), config.loop_start, config.loop_stop
    if config.has_loop:
        schedule += [LayerCall(i) for i in range(a)]
        for t in range(config.loop_times):
            entries.append(PassEntry("loop.step", config.loop_times, t, width,
                                     add_embedded=t > 0))
            schedule += [LayerCall(i, enters=t if i == a else None) for i in range(a, b)]
        schedule += [LayerCall(i) for i in range(b, n)]
    else:
        schedule = [LayerCall(i) for i in range(n)]
    embedding = TokenEmbedding("embed", config.vocab_size, width, suffix="")
    head = OutputHead("head", config.vocab_size, width, tied_to=None, suffix="")
    model = Model(config, dtype, embedding, layers, norm("final.norm"), head, schedule=schedule,
                  entries=entries)
    model.unused_tensor_names = unused
    return model


register_architecture(ARCHITECTURE, ZumuzenConfig, build_zumuzen)
