"""The Sibodra decoder put together from parts.

Every layer is ``block.hyper_connection`` (a pre-norm layer around a residual stream kept in
``streams`` copies; without ``streams`` in the configuration: one copy and the plain residual
sum) with layer norms without bias around one of two mixers: ``mixer.scored_attention`` in its
grouped-query form (every q and k head normed by itself, a rotation over the first places whose
frequencies may be scaled by wavelength, capped scores, a sink of score zero, one sigmoid gate a
head) or ``mixer.latent_attention`` (queries through a normed latent of their own, rotate-half
pairs, a sigmoid gate a channel); a SiLU-gated dense feed-forward, a mixture of squared-ReLU
experts with a router bias and a shared expert, or none.  The last norm reads the copies' sum;
the logits pass a cap.  Tensor names: ``embed``, ``final.norm``, ``head`` and per layer
``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.hc1|hc2.in|out|mix``; no name ends
in ``.weight``, biases end in ``.b``.
"""
from __future__ import annotations

import torch

from ..config.base import register_architecture
from ..config.sibodra import ARCHITECTURE, SibodraConfig
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from .base import Model


def _rotary(rot, head_dim: int):
    if not rot:
        return None
    return make_part("position_encoding", "rotary", head_dim=head_dim, theta=rot["base"],
                     rot_dim=rot["dims"], pairing="half", wavelength_scaling=rot["scaling"])


def _mixer(kind: str, m: dict, p: str, width: int, eps: float, dtype):
    if kind == "attention":
        return make_part(
            "mixer", "scored_attention", prefix=p, width=width, num_heads=m["heads"],
            num_kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], scale=m["scale"],
            dtype=dtype, norm_eps=eps, softcap=m["softcap"], head_qk_norm=True, sink_value=0.0,
            head_gate=True, position=_rotary(m["rot"], m["dim"]), weight_suffix="")
    if m.get("q_rank") is None:
        raise ValueError("config.json does not state mixer.q_rank, and no tensor shapes were "
                         "read that could give it")
    return make_part(
        "mixer", "latent_attention", prefix=p, width=width, num_heads=m["heads"], dim=m["dim"],
        rot_dim=m["rot_dim"], vdim=m["vdim"], rank=m["kv_rank"], scale=m["scale"], norm_eps=eps,
        dtype=dtype, position=_rotary(m["rot"], m["rot_dim"]), q_rank=m["q_rank"], gate=True,
        weight_suffix="")


def _feed_forward(mlp: dict, p: str, width: int, dtype):
    if mlp["kind"] == "dense":
        return make_part("feed_forward", "swiglu", prefix=p, width=width, hidden=mlp["ff"],
                         dtype=dtype, activation="silu",
                         names={"gate": "gate", "up": "up", "down": "down"}, weight_suffix="")
    return make_part("feed_forward", "moe", prefix=p, width=width, hidden=mlp["ff"],
                     experts=mlp["experts"], top=mlp["top"], dtype=dtype, weight_suffix="",
                     activation="relu_squared", router_bias=True, bias_suffix=".b",
                     shared_hidden=mlp["shared_ff"])


def build_sibodra(config: SibodraConfig, dtype: torch.dtype) -> Model:
    width, eps = config.width, config.norm_eps
    learned = config.streams is not None
    streams = config.streams if learned else 1

    def norm(name):
        return make_part("norm", "layernorm", name=name, width=width, eps=eps, dtype=dtype)

    layers, unused = [], []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        mixer = _mixer(layer.type, layer.mixer, p + "mix.", width, eps, dtype)
        feed_forward = ffn_norm = None
        if layer.mlp is not None:
            feed_forward = _feed_forward(layer.mlp, p + "mlp.", width, dtype)
            ffn_norm = norm(p + "norm2")
        else:
            unused.append(p + "norm2")
        block = make_part("block", "hyper_connection", prefix=p, streams=streams, width=width,
                          mixer_norm=norm(p + "norm1"), mixer=mixer, ffn_norm=ffn_norm,
                          feed_forward=feed_forward, learned=learned)
        unused += block.unused_tensor_names()
        layers.append(block)
    embedding = TokenEmbedding("embed", config.vocab_size, width, suffix="")
    head = OutputHead("head", config.vocab_size, width, tied_to=None, suffix="",
                      softcap=config.logit_softcap)
    model = Model(config, dtype, embedding, layers, norm("final.norm"), head)
    model.unused_tensor_names = unused
    return model


register_architecture(ARCHITECTURE, SibodraConfig, build_sibodra)
