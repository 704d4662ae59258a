"""Arrangements of parts in a layer."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..kernels import ops
from ..weights.spec import TensorSpec
from ctypes import Structure

from .base import (Block, FeedForward, Hidden, Mixer, Norm, StreamUpdate, register_part,
                   summed_delta)
from ..weights.spec import INIT_CONNECT, VECTOR
from .cdesc import NormPartDesc, PartDesc, defined_together


class PreNormBlockDesc(Structure):
    """``kappai_pre_norm_block`` of csrc/engine_parts.h."""
    _fields_ = [("mixer_norm", NormPartDesc), ("mixer", PartDesc), ("ffn_norm", NormPartDesc),
                ("feed_forward", PartDesc)]


def _takes_defer(norm) -> bool:
    return getattr(norm, "can_defer", False)


class PreNormBlock(Block):
    """``x += mixer(norm(x)); x += feed_forward(norm(x))`` (kappai: src/models/lfm.c:7-53 with
    the tail src/recipe/builders.c:378-388).  Each residual sum is made inside the norm
    that follows it.  ``feed_forward`` (with its norm) may be None: the layer is then its mixer
    alone."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm = None,
                 feed_forward: FeedForward = None):
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.ffn_norm, self.feed_forward = ffn_norm, feed_forward

    def _parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward)
                     if p is not None)

    @property
    def capturable(self) -> bool:
        return all(p.capturable for p in self._parts())

    @property
    def step_tables(self):
        out = []
        for p in self._parts():
            asked = p.step_tables
            if asked is not None:
                out += list(asked) if isinstance(asked, (list, tuple)) else [asked]
        return out

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self._parts() for s in p.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)

    takes_next_block = True

    def first_norm(self):
        """The norm a block before this one may fold into its last product, and the part that
        takes its rows."""
        return self.mixer_norm, self.mixer

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False,
                next_block=None) -> Hidden:
        # decode steps with few rows: a product may add its result into the residual stream
        # itself and hand the next product its rows without a norm kernel in between
        resid = h.resid
        x = self._normed(self.mixer_norm, resid, h.delta, self.mixer)
        if self.feed_forward is None:
            # (no product of this layer folds anything in: the mixer's result is the update)
            mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache)
            return Hidden(self._resid_after(x, resid), mixed)
        into = self._into(self.mixer, resid, self.ffn_norm, self.feed_forward)
        if into is not None:
            mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache, into=into)
        else:
            mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache)
        resid = self._resid_after(x, resid)
        x = self._normed(self.ffn_norm, resid, mixed, self.feed_forward)
        nxt = getattr(next_block, "first_norm", None)
        norm, consumer = nxt() if nxt is not None else (None, None)
        into = self._into(self.feed_forward, resid, norm, consumer)
        out = (self.feed_forward.forward(x, batch, into=into) if into is not None
               else self.feed_forward.forward(x, batch))
        return Hidden(self._resid_after(x, resid), out)

    @staticmethod
    def _into(producer, resid, norm, consumer):
        """What ``producer`` may add its result into, or None when it does not do such things."""
        if not getattr(producer, "adds_residual", False):
            return None
        fold = getattr(norm, "fold", None)
        if fold is not None and getattr(consumer, "takes_deferred_rows", False):
            return ops.AddInto(resid, *fold())
        return ops.AddInto(resid)

    @staticmethod
    def _normed(norm, resid, delta, consumer):
        delta = summed_delta(norm, delta)
        if getattr(consumer, "takes_deferred_rows", False) and _takes_defer(norm):
            return norm.add_norm(resid, delta, defer=True)
        return norm.add_norm(resid, delta)

    @staticmethod
    def _resid_after(x, resid):
        after = getattr(x, "resid_after", resid) if not isinstance(x, torch.Tensor) else resid
        if after is None:
            raise RuntimeError("a part that takes deferred rows did not use them")
        return after

    def c_call(self, plan, view, shared_cache: bool = False):
        """The block as the C side of a step runs it (runner "block.pre_norm"): the four parts'
        own descriptions side by side, or None when one of them has none.  A part whose class
        changed ``forward`` (or a norm's ``add_norm``) without giving a description of its own
        counts as having none."""
        if self.feed_forward is None:
            return None            # the runner on the C side knows the four-part layer only
        for part, method, c_method in ((self.mixer_norm, "add_norm", "c_norm"),
                                       (self.mixer, "forward", "c_part"),
                                       (self.ffn_norm, "add_norm", "c_norm"),
                                       (self.feed_forward, "forward", "c_part")):
            if not defined_together(part, method, c_method):
                return None
        n1, n2 = self.mixer_norm.c_norm(plan), self.ffn_norm.c_norm(plan)
        mixer = self.mixer.c_part(plan, view, shared_cache)
        feed_forward = self.feed_forward.c_part(plan, None, False)
        if n1 is None or n2 is None or mixer is None or feed_forward is None:
            return None
        return plan.call("block.pre_norm", PreNormBlockDesc(n1, mixer, n2, feed_forward),
                         first_norm=n1, first_consumer=mixer)

    def weight_bytes(self) -> int:
        return sum(p.weight_bytes() for p in self._parts())


register_part("block", "pre_norm", PreNormBlock)


class ConvInputBlock(Block):
    """``x += mixer(conv(norm(x))); x += feed_forward(conv(norm(x)))``: the pre-norm arrangement
    with a short causal convolution (``parts.input_conv.ShortInputConv``) between each norm and
    the sublayer that reads it.  The norm hands the convolution float32 rows; the convolution
    rounds to the compute dtype once.  ``feed_forward`` (with its norm and convolution) may be
    None: the layer is then its mixer alone.  The block's cache is a bundle: the mixer's own need
    under "mixer" and the convolutions' histories under "mixer_conv" and "ffn_conv"."""

    def __init__(self, mixer_norm: Norm, mixer_conv, mixer: Mixer, ffn_norm=None, ffn_conv=None,
                 feed_forward=None):
        self.mixer_norm, self.mixer_conv, self.mixer = mixer_norm, mixer_conv, mixer
        self.ffn_norm, self.ffn_conv, self.feed_forward = ffn_norm, ffn_conv, feed_forward
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")

    def _parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer_conv, self.mixer, self.ffn_norm,
                                 self.ffn_conv, self.feed_forward) if p is not None)

    @property
    def capturable(self) -> bool:
        return all(p.capturable for p in self._parts())

    @property
    def step_tables(self):
        return [t for t in (p.step_tables for p in self._parts()) if t is not None]

    def cache_spec(self):
        from ..cache.specs import CacheBundle
        members = [("mixer", self.mixer.cache_spec())]
        if self.mixer_conv is not None:
            members.append(("mixer_conv", self.mixer_conv.cache_spec()))
        if self.ffn_conv is not None:
            members.append(("ffn_conv", self.ffn_conv.cache_spec()))
        return CacheBundle(tuple(members))

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self._parts() for s in p.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)

    @staticmethod
    def _read(norm, conv, resid, delta, batch, state):
        delta = summed_delta(norm, delta)
        if conv is None:
            return norm.add_norm(resid, delta)
        if batch.max_segment_rows == 1 and hasattr(norm, "add_norm_conv_step"):
            return norm.add_norm_conv_step(resid, delta, conv, batch, state)    # decode: one kernel
        if getattr(norm, "takes_out_dtype", False):
            h = norm.add_norm(resid, delta, out_dtype=torch.float32)
        else:
            h = ops.cast(norm.add_norm(resid, delta), torch.float32)
        return conv.forward(h, batch, state)

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False) -> Hidden:
        if shared_cache:
            raise ValueError("the input convolutions' histories cannot be read by another layer")
        resid = h.resid
        x = self._read(self.mixer_norm, self.mixer_conv, resid, h.delta, batch,
                       cache.parts.get("mixer_conv"))
        mixed = self.mixer.forward(x, batch, cache.part("mixer"))
        if self.feed_forward is None:
            return Hidden(resid, mixed)
        x = self._read(self.ffn_norm, self.ffn_conv, resid, mixed, batch,
                       cache.parts.get("ffn_conv"))
        return Hidden(resid, self.feed_forward.forward(x, batch))

    def weight_bytes(self) -> int:
        return sum(p.weight_bytes() for p in self._parts())


register_part("block", "conv_input", ConvInputBlock)


class OutputNormBlock(Block):
    """``x += norm1(mixer(x)); x += norm2(feed_forward(x))``: the sublayers read the stream itself
    and the norm sits on what they return.  ``feed_forward`` (with its norm) may be None.  The
    stream is float32; the kernel that adds a normalised result also writes the stream rounded to
    the compute dtype, which is what the next sublayer reads (``Hidden.rows``).  The norms are
    RMS norms that know ``norm_output`` (``parts.norm.RMSNorm``)."""

    def __init__(self, mixer: Mixer, mixer_norm: Norm, feed_forward=None, ffn_norm=None):
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        for n in (mixer_norm, ffn_norm):
            if n is not None and not hasattr(n, "norm_output"):
                raise ValueError(f"{type(n).__name__} cannot norm a sublayer's output into the "
                                 "stream (no norm_output)")
        self.mixer, self.mixer_norm = mixer, mixer_norm
        self.feed_forward, self.ffn_norm = feed_forward, ffn_norm

    def _parts(self):
        return tuple(p for p in (self.mixer, self.mixer_norm, self.feed_forward, self.ffn_norm)
                     if p is not None)

    @property
    def capturable(self) -> bool:
        return all(p.capturable for p in self._parts())

    @property
    def step_tables(self):
        out = []
        for p in self._parts():
            asked = p.step_tables
            if asked is not None:
                out += list(asked) if isinstance(asked, (list, tuple)) else [asked]
        return out

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self._parts() for s in p.tensor_specs()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False) -> Hidden:
        resid = h.resid
        if h.delta is not None:
            raise ValueError("the block before left an update that was not added to the stream")
        narrow = self.mixer_norm.dtype != torch.float32
        rows_dtype = self.mixer_norm.dtype if narrow else None
        x = h.rows if narrow else resid
        if x is None:
            x = ops.cast(resid, self.mixer_norm.dtype)
        mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache)
        rows = self.mixer_norm.norm_output(resid, mixed, rows_dtype=rows_dtype)
        if self.feed_forward is not None:
            out = self.feed_forward.forward(rows if narrow else resid, batch)
            rows = self.ffn_norm.norm_output(resid, out, rows_dtype=rows_dtype)
        return Hidden(resid, None, rows)

    def weight_bytes(self) -> int:
        return sum(p.weight_bytes() for p in self._parts())


register_part("block", "output_norm", OutputNormBlock)


class HyperConnectionBlock(Block):
    """A pre-norm layer around a residual stream kept in ``streams`` copies x_1 .. x_S
    ("hyper-connections"; all copies start as the embedded row).  Sublayer q (1: the mixer, 2: the
    feed-forward) reads ``u = sum_s in_q[s] x_s`` through its norm, and its result y goes back as

        x_t <- sum_s mix_q[s, t] x_s + out_q[t] * y        (all t at once, from the old copies)

    with ``in_q`` [S], ``out_q`` [S] and ``mix_q`` [S, S] (indexed [from, to]) from the file
    (``<prefix>hc<q>.in|out|mix``).  ``learned`` False: one copy with in = out = mix = 1, the
    plain residual sum, and no such tensors.  After the last layer the stream is the copies' sum,
    which is what the model's last norm (``parts.norm.LayerNorm.add_norm``) reads.

    A sublayer's result is not applied when it is made: it travels as a ``StreamUpdate`` to the
    pass that reads the stream next, so each sublayer costs ONE pass over the copies (apply the
    update before, sum for this sublayer, normalise).  The norms must know ``read_streams``."""

    def __init__(self, prefix: str, streams: int, width: int, mixer_norm: Norm, mixer: Mixer,
                 ffn_norm: Norm = None, feed_forward: FeedForward = None, learned: bool = True,
                 names=None):
        n = {"mixer": "hc1.", "feed_forward": "hc2.", "in": "in", "out": "out", "mix": "mix"}
        n.update(names or {})
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        if not 1 <= streams <= ops.HYPER_MAX_STREAMS:
            raise ValueError(f"{prefix}: {streams} copies of the stream; the kernel takes 1 to "
                             f"{ops.HYPER_MAX_STREAMS}")
        if not learned and streams != 1:
            raise ValueError(f"{prefix}: {streams} copies of the stream need connection weights")
        for norm in (mixer_norm, ffn_norm):
            if norm is not None and not hasattr(norm, "read_streams"):
                raise ValueError(f"{type(norm).__name__} cannot read a stream kept in copies (no "
                                 "read_streams)")
        self.S, self.width, self.learned = int(streams), int(width), bool(learned)
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.ffn_norm, self.feed_forward = ffn_norm, feed_forward
        self._names = {q: {k: prefix + n[q] + n[k] for k in ("in", "out", "mix")}
                       for q in ("mixer", "feed_forward")}
        self.weights = {}        # sublayer -> (in [S], out [S], mix [S, S]) float32

    def _parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward)
                     if p is not None)

    def _sublayers(self):
        return ("mixer",) if self.feed_forward is None else ("mixer", "feed_forward")

    @property
    def capturable(self) -> bool:
        return all(p.capturable for p in self._parts())

    @property
    def step_tables(self):
        out = []
        for p in self._parts():
            asked = p.step_tables
            if asked is not None:
                out += list(asked) if isinstance(asked, (list, tuple)) else [asked]
        return out

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for p in self._parts() for s in p.tensor_specs()]
        if self.learned:
            for q in self._sublayers():
                nm = self._names[q]
                specs += [TensorSpec(nm["in"], (self.S,), VECTOR, INIT_CONNECT),
                          TensorSpec(nm["out"], (self.S,), VECTOR, INIT_CONNECT),
                          TensorSpec(nm["mix"], (self.S, self.S), VECTOR, INIT_CONNECT)]
        return specs

    def unused_tensor_names(self) -> List[str]:
        """What a file may hold for the feed-forward this layer does not have."""
        if self.feed_forward is not None or not self.learned:
            return []
        return list(self._names["feed_forward"].values())

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self._parts():
            p.bind(tensors)
        for q in self._sublayers():
            if self.learned:
                nm = self._names[q]
                self.weights[q] = tuple(tensors[nm[k]].to(torch.float32).contiguous()
                                        for k in ("in", "out", "mix"))
            else:
                one = self.mixer_norm.ones
                self.weights[q] = (one(1), one(1), one(1, 1))

    def forward(self, h: Hidden, batch, cache, shared_cache: bool = False) -> Hidden:
        streams, pending = h.resid, h.delta
        w_in, w_out, w_mix = self.weights["mixer"]
        if streams.dim() == 2:
            # what the embedding left: every copy starts as that row
            if pending is not None:
                raise ValueError("an update is pending on a stream that has no copies yet")
            source = streams
            streams = torch.empty((source.shape[0], self.S, self.width), dtype=torch.float32,
                                  device=source.device)
            x = self.mixer_norm.read_streams(streams, w_in, source=source)
        else:
            if pending is not None and not isinstance(pending, StreamUpdate):
                raise ValueError("a stream kept in copies takes its updates as StreamUpdate")
            x = self.mixer_norm.read_streams(streams, w_in, pending=pending)
        mixed = self.mixer.forward(x, batch, cache, shared_cache=shared_cache)
        update = StreamUpdate(mixed, w_mix, w_out)
        if self.feed_forward is None:
            return Hidden(streams, update)
        w_in, w_out, w_mix = self.weights["feed_forward"]
        x = self.ffn_norm.read_streams(streams, w_in, pending=update)
        return Hidden(streams, StreamUpdate(self.feed_forward.forward(x, batch), w_mix, w_out))

    def weight_bytes(self) -> int:
        return sum(p.weight_bytes() for p in self._parts())


register_part("block", "hyper_connection", HyperConnectionBlock)
