"""Named configurations for the random-weights mode: config.json contents by name.

These are data, not defaults: no part of the engine reads a size from here.  ``--random-weights
NAME`` writes a model folder of that shape; the benchmark uses the same dictionaries.  The sizes
are those of the architecture's published models (the three LFM2 shapes) and of two tiny
configurations that differ in every size and option.
"""
from __future__ import annotations

import copy
from typing import Dict


def _lfm2(hidden, layers, attention_at, heads, kv_heads, intermediate, **more) -> dict:
    raw = {
        "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": hidden,
        "num_hidden_layers": layers,
        "layer_types": ["full_attention" if i in attention_at else "conv" for i in range(layers)],
        "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": 64,
        "intermediate_size": intermediate, "block_auto_adjust_ff_dim": True,
        "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0, "vocab_size": 65536,
        "norm_eps": 1e-5, "rope_theta": 1000000.0, "conv_L_cache": 3, "conv_bias": False,
        "tie_embedding": True, "max_position_embeddings": 128000,
    }
    raw.update(more)
    return raw


SHAPES: Dict[str, dict] = {
    # 16 layers, attention at 2, 5, 8, 10, 12, 14; feed-forward 12288 -> 8192
    "lfm2-1.2b": _lfm2(2048, 16, (2, 5, 8, 10, 12, 14), 32, 8, 12288),
    # the same pattern at half the width; feed-forward 6656 -> 4608
    "lfm2-350m": _lfm2(1024, 16, (2, 5, 8, 10, 12, 14), 16, 8, 6656),
    # 30 layers, attention at 2, 6, 10, 14, 18, 21, 24, 27; feed-forward 10752 -> 7168
    "lfm2-2.6b": _lfm2(2048, 30, (2, 6, 10, 14, 18, 21, 24, 27), 32, 8, 10752),
    # 4 layers conv/attention alternating, two kv heads for four heads, tied head
    "tiny-a": {
        "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 64,
        "num_hidden_layers": 4,
        "layer_types": ["conv", "full_attention", "conv", "full_attention"],
        "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
        "intermediate_size": 192, "block_auto_adjust_ff_dim": False, "vocab_size": 256,
        "norm_eps": 1e-5, "rope_theta": 10000.0, "conv_L_cache": 3, "conv_bias": False,
        "tie_embedding": True, "max_position_embeddings": 4096,
    },
    # 6 layers, attention at 0, 3, 4, one kv head for three heads, a width that is no power of two,
    # adjusted feed-forward width (480 -> 320), 4 taps with biases, untied head
    "tiny-b": {
        "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 96,
        "num_hidden_layers": 6,
        "layer_types": ["full_attention", "conv", "conv", "full_attention", "full_attention",
                        "conv"],
        "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
        "intermediate_size": 480, "block_auto_adjust_ff_dim": True, "block_multiple_of": 64,
        "block_ffn_dim_multiplier": 1.0, "vocab_size": 512, "norm_eps": 1e-6,
        "rope_theta": 1000000.0, "conv_L_cache": 4, "conv_bias": True, "tie_embedding": False,
        "max_position_embeddings": 8192,
    },
}


def _dapipel(width, mixers, heads, kv_heads, dim, vdim, window, ff, experts, top, vocab=65536,
             positions=8192, inner=None) -> dict:
    """Layers by letter: "a" windowed differential attention, "g" minGRU; dense feed-forwards of
    ``ff`` and mixtures of ``experts`` experts of ``ff * 2 // (top * 2)`` (as many active weights
    as the dense layer) in turns."""
    layers = []
    for i, kind in enumerate(mixers):
        if kind == "a":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                     "scale": dim ** -0.5, "diff": 0.8, "mask": {"size": window}}
        else:
            mixer = {"width": inner or width}
        mlp = ({"kind": "dense", "ff": ff} if i % 2 == 0 else
               {"kind": "moe", "expert": {"ff": ff // top}, "router": {"experts": experts,
                                                                       "top": top}})
        layers.append({"type": "attention" if kind == "a" else "mingru", "mixer": mixer,
                       "mlp": mlp})
    return {"architecture": "Dapipel", "vocab": vocab, "width": width, "max_positions": positions,
            "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5, "groups": 8},
            "canon": {"taps": 4}, "layers": layers}


SHAPES.update({
    # eight layers at a width of 1024: attention where the LFM2 pattern has it (2, 5, 7; 16 heads
    # on 4 kv heads, so each map's 16 heads share 4 kv heads as LFM2's 32 share 8), a recurrent
    # layer elsewhere; feed-forward 4608 dense or 16 experts of 2304, two a token
    "dapipel-w1024": _dapipel(1024, "ggaggaga", 16, 4, 32, 64, 1024, 4608, 16, 2),
    # the same at a width of 2048: heads of 128 values on maps of 64, feed-forward 8192
    "dapipel-w2048": _dapipel(2048, "ggaggaga", 16, 4, 64, 128, 2048, 8192, 16, 2),
    # a tiny one for smoke runs
    "dapipel-tiny": _dapipel(64, "gaga", 4, 2, 8, 16, 24, 96, 4, 2, vocab=256, positions=512,
                             inner=48),
})
# the LFM2 shapes of the same widths, depths, attention layers and feed-forward widths
SHAPES.update({
    "lfm2-like-w1024": _lfm2(1024, 8, (2, 5, 7), 16, 8, 4608, block_auto_adjust_ff_dim=False,
                             max_position_embeddings=8192),
    "lfm2-like-w2048": _lfm2(2048, 8, (2, 5, 7), 32, 8, 8192, block_auto_adjust_ff_dim=False,
                             max_position_embeddings=8192),
})


def _dukolorn(width, mixers, heads, kv_heads, dim, r_heads, r_dim, r_vdim, l_heads, l_dim, l_rot,
              l_vdim, l_rank, window, d_heads, d_qk_heads, d_dim, d_vdim, ff, vocab=65536,
              rank=32, buckets=64, bias_max=512.0) -> dict:
    """Layers by letter: "p" a scored softmax attention beside a gated linear attention, "l" a
    latent attention under a sliding window, "d" the gated delta rule (without feed-forward, as
    the design's own models have it); dense feed-forwards of ``ff`` elsewhere."""
    layers = []
    for kind in mixers:
        if kind == "p":
            left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                    "scale": dim ** -0.5, "softcap": 50.0, "bias_max": bias_max,
                    "buckets": buckets, "q_temp": {"coef": 0.1, "every": 256}}
            right = {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": 8.0,
                     "decay_rank": rank}
            layers.append({"type": "parallel", "mlp": {"kind": "dense", "ff": ff},
                           "mixer": {"left": left, "right": right, "left_scale": 1.0,
                                     "right_scale": 1.0}})
        elif kind == "l":
            layers.append({"type": "latent_attention", "mlp": {"kind": "dense", "ff": ff},
                           "mixer": {"heads": l_heads, "dim": l_dim, "rot_dim": l_rot,
                                     "vdim": l_vdim, "kv_rank": l_rank,
                                     "scale": (l_dim + l_rot) ** -0.5,
                                     "rot": {"base": 10000.0, "dims": l_rot},
                                     "mask": {"size": window}}})
        else:
            layers.append({"type": "channel_delta", "mlp": None,
                           "mixer": {"heads": d_heads, "kv_heads": d_qk_heads, "dim": d_dim,
                                     "vdim": d_vdim, "conv": 4, "decay_rank": rank,
                                     "gate_rank": rank}})
    return {"architecture": "Dukolorn", "vocab": vocab, "width": width, "norm": {"eps": 1e-5},
            "logit_scale": 1.0, "layers": layers}


SHAPES.update({
    # eight layers at a width of 1024 in the order pair, latent, latent, delta rule, twice: 16
    # heads of 64 on 4 kv heads beside 8 recurrent heads of 64 x 64; latent attention with 16
    # heads of 64 + 32 rotated places on a latent of 224 under a window of 1024; the delta rule
    # with 16 heads of 64 x 64 on 4 q/k heads; feed-forward 4608
    "dukolorn-w1024": _dukolorn(1024, "plldplld", 16, 4, 64, 8, 64, 64, 16, 64, 32, 64, 224, 1024,
                                16, 4, 64, 64, 4608),
    # the same at a width of 2048: 32 heads on 8 kv heads, recurrent heads of 64 x 128, 16 latent
    # heads of 128 + 64 on a latent of 192 under a window of 2048, feed-forward 8192
    "dukolorn-w2048": _dukolorn(2048, "plldplld", 32, 8, 64, 16, 64, 128, 16, 128, 64, 128, 192,
                                2048, 16, 4, 128, 128, 8192),
    # a tiny one for smoke runs
    "dukolorn-tiny": _dukolorn(64, "pld", 4, 2, 8, 2, 8, 16, 2, 8, 8, 16, 24, 24, 2, 1, 16, 8, 96,
                               vocab=256, rank=4, buckets=8, bias_max=40.0),
})


def _zumuzen(width, mixers, heads, kv_heads, dim, chunk, l_heads, l_dim, l_vdim, t_heads, t_dim,
             inner, blocks, ff, vocab=65536, rank=64, taps=4, loop=None) -> dict:
    """Layers by letter: "p" a softmax attention over chunks beside a linear attention with a
    fixed decay a head, "t" a softmax attention over chunks whose values are its keys (stretched
    frequencies, a sink) beside a time mixing with a bonus, "r" a real-gated unit; dense
    feed-forwards of ``ff`` everywhere."""
    layers = []
    for kind in mixers:
        left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                "scale": dim ** -0.5, "rot": {"base": 10000.0, "dims": dim},
                "mask": {"size": chunk}}
        if kind == "p":
            decay = [1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, l_heads - 1)) for h in range(l_heads)]
            mixer = {"left": left, "right": {"heads": l_heads, "dim": l_dim, "vdim": l_vdim,
                                             "decay": decay}}
            layers.append({"type": "parallel", "mixer": mixer})
        elif kind == "t":
            left["rot"]["scaling"] = {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}
            mixer = {"left": left, "right": {"heads": t_heads, "dim": t_dim, "decay_rank": rank},
                     "left_scale": 1.0, "right_scale": 1.0}
            layers.append({"type": "parallel_2", "mixer": mixer})
        else:
            layers.append({"type": "rglru", "mixer": {"width": inner, "blocks": blocks,
                                                      "conv": taps}})
        layers[-1]["mlp"] = {"kind": "dense", "ff": ff}
    out = {"architecture": "Zumuzen", "vocab": vocab, "width": width, "norm": {"eps": 1e-5},
           "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


SHAPES.update({
    # eight layers at a width of 1024: a pair of mixers where the LFM2 pattern has attention (2,
    # 5, 7; 16 heads of 64 on 4 kv heads in chunks of 1024), a real-gated unit of 1024 channels
    # in 8 blocks elsewhere; 8 linear-attention heads of 64 x 64, 16 time-mixing heads of 64
    "zumuzen-w1024": _zumuzen(1024, "rrprrtrp", 16, 4, 64, 1024, 8, 64, 64, 16, 64, 1024, 8,
                              4608),
    # the same at a width of 2048: 32 heads on 8 kv heads in chunks of 2048, linear-attention
    # heads of 64 x 128, 32 time-mixing heads of 64, 2048 channels in 16 blocks
    "zumuzen-w2048": _zumuzen(2048, "rrprrtrp", 32, 8, 64, 2048, 16, 64, 128, 32, 64, 2048, 16,
                              8192),
    # a tiny one for smoke runs: the last two layers are passed twice
    "zumuzen-tiny": _zumuzen(64, "prt", 4, 2, 8, 24, 2, 8, 16, 2, 16, 48, 3, 96, vocab=256,
                             rank=4, taps=3, loop=(1, 3, 2)),
})


def _sibodra(width, mixers, heads, kv_heads, dim, rot, l_heads, l_dim, l_rot, l_vdim, l_rank,
             q_rank, ff, experts, top, streams, vocab=65536, original=8192) -> dict:
    """Layers by letter: "a" grouped-query attention (per-head norms, partial rotation with scaled
    frequencies, capped scores), "l" latent attention; dense feed-forwards of ``ff`` and mixtures
    of ``experts`` squared-ReLU experts of ``ff // top`` with a shared expert of the same size in
    turns; the stream in ``streams`` copies."""
    layers = []
    for i, kind in enumerate(mixers):
        if kind == "a":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                     "scale": dim ** -0.5, "softcap": 50.0,
                     "rot": {"base": 10000.0, "dims": rot,
                             "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                                         "original": original}}}
        else:
            mixer = {"heads": l_heads, "dim": l_dim, "rot_dim": l_rot, "vdim": l_vdim,
                     "kv_rank": l_rank, "q_rank": q_rank, "scale": (l_dim + l_rot) ** -0.5,
                     "rot": {"base": 10000.0, "dims": l_rot}}
        mlp = ({"kind": "dense", "ff": ff} if i % 2 == 0 else
               {"kind": "moe", "expert": {"ff": ff // top}, "shared": {"ff": ff // top},
                "router": {"experts": experts, "top": top}})
        layers.append({"type": "attention" if kind == "a" else "latent_attention",
                       "mixer": mixer, "mlp": mlp})
    return {"architecture": "Sibodra", "vocab": vocab, "width": width, "norm": {"eps": 1e-5},
            "streams": streams, "logit_softcap": 30.0, "layers": layers}


SHAPES.update({
    # eight layers at a width of 1024, grouped-query and latent attention in turns: 16 heads of
    # 64 on 4 kv heads, half of every head rotated; 16 latent heads of 64 + 32 rotated places on
    # a latent of 224, queries through a latent of 384; feed-forward 4608 dense or 16 experts of
    # 2304 beside a shared one, two a token; the stream in four copies
    "sibodra-w1024": _sibodra(1024, "alalalal", 16, 4, 64, 32, 16, 64, 32, 64, 224, 384, 4608,
                              16, 2, 4),
    # the same at a width of 2048: 32 heads on 8 kv heads, 16 latent heads of 128 + 64 on a
    # latent of 192, queries through a latent of 768, feed-forward 8192
    "sibodra-w2048": _sibodra(2048, "alalalal", 32, 8, 64, 32, 16, 128, 64, 128, 192, 768, 8192,
                              16, 2, 4),
    # a tiny one for smoke runs
    "sibodra-tiny": _sibodra(64, "ala", 4, 2, 8, 4, 2, 8, 8, 16, 24, 16, 96, 4, 2, 2, vocab=256,
                             original=64),
})


def named_shape(name: str) -> dict:
    """A copy of the configuration called ``name`` (any case), or a ``KeyError`` naming them all."""
    key = name.strip().lower()
    if key not in SHAPES:
        raise KeyError(f"no shape named {name!r}; known: {', '.join(sorted(SHAPES))}")
    return copy.deepcopy(SHAPES[key])
