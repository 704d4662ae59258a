"""The Zumuzen decoder on the GPU against the plain implementation (tests/plain/zumuzen.py): the
new kernels alone, every mixer as a part over portions and single tokens, keys made to stand out
(at position 0, at page borders, far back in a long chunk, just inside and just outside a chunk's
edge), the sink shown by a weight that makes it decide, whole models of four tiny configurations
under the four schedule families in float32 and bfloat16 with pools so small that pages and slots
are used again, long decoding, a batch against its requests alone, the stream layer by layer, and
greedy generation through the engine and its scheduler."""
import math

import numpy as np
import pytest
import torch

import schedules
from plain import zumuzen as P
from replay_common import collect, make_requests
from tiny_zumuzen import TINY, assert_matches_plain, read_model_dir, write_tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16, F64 = torch.float32, torch.bfloat16, torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rel(got, want):
    got = got.detach().to("cpu", F64)
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def tables(segments, slots=None):
    """int32 row tables on the GPU for segments [(first position, rows), ...]."""
    row_pos, row_seg, seg_start = [], [], [0]
    for s, (p0, n) in enumerate(segments):
        row_pos += list(range(p0, p0 + n))
        row_seg += [s] * n
        seg_start.append(seg_start[-1] + n)
    slots = list(range(len(segments))) if slots is None else slots
    host = dict(row_pos=row_pos, row_seg=row_seg, seg_start=seg_start,
                seg_pos0=[p for p, _ in segments], seg_slot=slots)
    return {k: torch.tensor(v, dtype=torch.int32, device=DEV) for k, v in host.items()}


def bind_random(part, seed, dtype, std=0.2, change=None):
    from kappai_amd.weights import random_tensors, stored_to_runtime
    t = random_tensors(part.tensor_specs(), seed, std=std)
    if change:
        change(t)
    part.bind({k: stored_to_runtime(v, dtype).to(DEV) for k, v in t.items()})
    return t


def one_segment_batch(cm, n, rc=None):
    """A RowBatch for ``n`` more tokens of one request, with the tables the parts ask for (tiles
    of query rows, chunks of rows for the scans)."""
    from kappai_amd.engine import StepEntry, StepRunner
    from kappai_amd.kernels import ops, tuning
    from kappai_amd.parts.attention import AttentionTiles
    from kappai_amd.parts.mingru import ScanChunks
    rc = rc or cm.open("r")
    cm.extend(rc, n)
    runner = StepRunner.__new__(StepRunner)
    runner.model = type("M", (), {"vocab_size": 10 ** 9})()
    runner.step_tables = [AttentionTiles(ops.ATTENTION_TILE_ROWS),
                          ScanChunks(tuning.SCAN_CHUNK_ROWS)]
    runner.cache, runner.device, runner._staging, runner._staged = cm, torch.device(DEV), None, None
    return rc, runner.make_batch([StepEntry(rc, [0] * n, [])])


def step_through(part, cm, x, portions, view):
    """One request through a mixer in ``portions``; returns the outputs in order."""
    from kappai_amd.kernels import ops
    from kappai_amd.parts.base import WeightedTerms
    rc, outs, done = None, [], 0
    for n in portions:
        rc, b = one_segment_batch(cm, n, rc=rc)
        if n > 64:
            assert b.extra.get("scan_chunks") is not None
        y = part.forward(x[done:done + n].to(DEV), b, view)
        if isinstance(y, WeightedTerms):
            y = ops.pair_norm_sum(y.a.sum(0) if y.a.dim() == 3 else y.a,
                                  y.b.sum(0) if y.b.dim() == 3 else y.b, y.scale_a, y.scale_b)
        outs.append(y if y.dim() == 2 else y.sum(0))
        cm.commit(rc, n)
        cm.check()
        done += n
    assert done == x.shape[0]
    return torch.cat(outs).float(), rc


PORTIONS_150 = [37, 3] + [1] * 50 + [2, 33] + [1] * 25


# ---------------------------------------------------------------------------------------------
# kernels alone
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("D", [72, 64, 100, 2048])
def test_what_a_pass_starts_with(D):
    """Pending update, the embedded rows once more and the pass's row, each present or not."""
    from kappai_amd.kernels import ops
    T = 11
    x = torch.randn(T, D, generator=gen(1)) * 3
    e = torch.randn(T, D, generator=gen(2))
    row = torch.randn(D, generator=gen(3))
    for dd in (None, F32, BF16):
        for again in (False, True):
            for with_row in (False, True):
                d = None if dd is None else torch.randn(T, D, generator=gen(4)).to(dd)
                want = x.double()
                if d is not None:
                    want = want + d.double()
                if again:
                    want = want + e.double()
                if with_row:
                    want = want + row.double()
                resid = x.clone().to(DEV)
                ops.stream_enter(resid, None if d is None else d.to(DEV),
                                 e.to(DEV) if again else None, row.to(DEV) if with_row else None)
                assert rel(resid, want) < 1e-6, (dd, again, with_row)


@pytest.mark.parametrize("D", [72, 100, 256, 2048])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_two_sides_normed_and_added(D, dtype):
    from kappai_amd.kernels import ops
    T = 13
    a = (torch.randn(T, D, generator=gen(5)) * 2).to(dtype)
    b = (torch.randn(T, D, generator=gen(6)) * 0.3).to(dtype)
    wa = 1 + 0.3 * torch.randn(D, generator=gen(7))
    wb = 1 + 0.3 * torch.randn(D, generator=gen(8))
    got = ops.pair_norm_sum(a.to(DEV), b.to(DEV), 0.5, 0.5, wa.to(DEV), wb.to(DEV), 1e-3)
    want = 0.5 * (P.norm(a.double(), wa, 1e-3) + P.norm(b.double(), wb, 1e-3))
    assert rel(got, want) < 2e-6
    got = ops.pair_norm_sum(a.to(DEV), b.to(DEV), 0.7, 1.3)
    assert rel(got, 0.7 * a.double() + 1.3 * b.double()) < 1e-6


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_mixes_with_the_token_before_over_portions_and_slots(dtype):
    """Two requests side by side in slots 3 and 1 of states that hold NaN, in portions down to one
    row: the first row of a portion reads the request's last row from its slot, position 0 reads
    zeros."""
    from kappai_amd.kernels import ops
    W, T, n_mix = 72, 31, 5
    mu = torch.rand(n_mix, W, generator=gen(9))
    xs = [torch.randn(T, W, generator=gen(10 + i)).to(BF16) for i in range(2)]
    state = torch.full((5, W), float("nan"), device=DEV)
    outs, done = [[], []], 0
    for n in [5, 1, 1, 2, 9, 1, 12]:
        tb = tables([(done, n), (done, n)], slots=[3, 1])
        x = torch.cat([xs[0][done:done + n], xs[1][done:done + n]]).to(dtype).to(DEV)
        y = ops.token_shift_mix(x, mu.to(DEV), state, tb["row_pos"], tb["row_seg"],
                                tb["seg_start"], tb["seg_slot"])
        outs[0].append(y[:, :n])
        outs[1].append(y[:, n:])
        done += n
    for i in range(2):
        h = xs[i].double()
        before = torch.cat([torch.zeros(1, W, dtype=F64), h[:-1]])
        want = h[None] + (before - h)[None] * mu.double()[:, None, :]
        assert rel(torch.cat(outs[i], dim=1).float(), want) < (1e-6 if dtype == F32 else 1e-2)


def plain_state_scan(q, k, v, a, bonus):
    """o [T, H, dv] of ``S <- diag(a_t) S + k v^T`` read after the write (no bonus) or before it
    with the token itself weighed by ``bonus``; q, k, a [T, H, d], v [T, H, dv], float64."""
    T, H, d = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        S = torch.zeros(d, v.shape[2], dtype=F64)
        for t in range(T):
            kv = torch.outer(k[t, h], v[t, h])
            if bonus is None:
                S = a[t, h][:, None] * S + kv
                out[t, h] = S.T @ q[t, h]
            else:
                out[t, h] = (S + bonus[h][:, None] * kv).T @ q[t, h]
                S = a[t, h][:, None] * S + kv
    return out


@pytest.mark.parametrize("H,d,dv", [(3, 8, 16), (1, 72, 24), (2, 136, 8), (2, 24, 70),
                                    (2, 64, 128), (1, 300, 4), (5, 20, 20)])
@pytest.mark.parametrize("form", ["wave", "block", "auto"])
@pytest.mark.parametrize("kind", ["fixed", "bonus"])
def test_recurrences_with_a_fixed_decay_and_with_a_bonus(H, d, dv, form, kind):
    """Three requests in portions (slots in another order, NaN in the states before) by both
    kernels, against a loop in float64: a fixed decay a head with SiLU on the inputs (a head of
    decay 1 and one of 0 among them), and the doubly exponential decay with the bonus."""
    from kappai_amd.kernels import ops
    if form == "block" and d % 4:
        pytest.skip("the kernel that works through LDS takes key sizes that are multiples of four")
    if kind == "bonus":
        dv = d
    T, g = 45, gen(11)
    seqs = [dict(q=torch.randn(T, H * d, generator=g), k=torch.randn(T, H * d, generator=g),
                 v=torch.randn(T, H * dv, generator=g), z=torch.randn(T, H * d, generator=g))
            for _ in range(3)]
    rate = torch.tensor(([1.0, 0.0, 0.9, 0.5, 0.97] * 2)[:H])
    w0 = torch.randn(H * d, generator=g) - 1.0
    bonus = torch.randn(H, d, generator=g)
    want = []
    for s in seqs:
        q, k, v = (s[n].double().reshape(T, H, -1) for n in "qkv")
        if kind == "fixed":
            a = rate.double()[None, :, None].expand(T, H, d)
            want.append(plain_state_scan(P.silu(q), P.silu(k), P.silu(v), a, None))
        else:
            a = torch.exp(-torch.exp(s["z"].double() + w0.double())).reshape(T, H, d)
            want.append(plain_state_scan(q, k, v, a, bonus.double()))
    state = torch.full((6, H, dv, d), float("nan"), device=DEV)
    got, done = [[], [], []], 0
    for n in [7, 1, 2, 1, 20, 1, 13]:
        tb = tables([(done, n)] * 3, slots=[4, 0, 2])
        cat = {c: torch.cat([s[c][done:done + n] for s in seqs]).to(DEV) for c in "qkvz"}
        if kind == "fixed":
            o = ops.matrix_state_recurrence(
                cat["q"], cat["k"], cat["v"], None, H, H, d, dv, rate.to(DEV), None, 1.0, 1.0,
                state, tb["seg_start"], tb["seg_pos0"], tb["seg_slot"], decay="fixed",
                silu_inputs=True, form=form)
        else:
            o = ops.matrix_state_recurrence(
                cat["q"], cat["k"], cat["v"], cat["z"], H, H, d, dv, None, w0.to(DEV), 1.0, 1.0,
                state, tb["seg_start"], tb["seg_pos0"], tb["seg_slot"], decay="double_exp",
                bonus=bonus.to(DEV), form=form)
        for i in range(3):
            got[i].append(o[i * n:(i + 1) * n])
        done += n
    for i in range(3):
        assert rel(torch.cat(got[i]), want[i].reshape(T, H * dv)) < 2e-5, i


def chunk_tables(segments, rows):
    """``scan_chunks`` and ``scan_seg_chunk0`` for segments [(first position, rows), ...]."""
    chunks, first, row = [], [0], 0
    for s, (_, n) in enumerate(segments):
        for at in range(0, n, rows):
            chunks.append([s, row + at, min(rows, n - at)])
        row += n
        first.append(len(chunks))
    return (torch.tensor(chunks, dtype=torch.int32, device=DEV),
            torch.tensor(first, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("H,d,dv", [(3, 8, 16), (1, 72, 24), (2, 136, 8), (2, 24, 70),
                                    (2, 64, 128), (1, 300, 4), (5, 20, 20), (2, 64, 200)])
@pytest.mark.parametrize("rows", [32, 7])
@pytest.mark.parametrize("kind", ["fixed", "bonus"])
def test_recurrences_chunk_by_chunk(H, d, dv, rows, kind):
    """Three unequal requests side by side, in portions that end inside a chunk and single rows
    (slots in another order, NaN in the states before), by the forms that work chunks of rows in
    passes: against a loop in float64, and against the kernel that walks the tokens.  The decays
    of the form with a bonus reach from next to one down to nothing at all (a decay that
    underflows to zero: what came before is gone)."""
    from kappai_amd.kernels import ops
    if kind == "bonus":
        dv = d
    g = gen(12)
    lens = [150, 77, 120]
    seqs = [dict(q=torch.randn(n, H * d, generator=g) * 0.5, k=torch.randn(n, H * d, generator=g),
                 v=torch.randn(n, H * dv, generator=g),
                 z=torch.randn(n, H * d, generator=g) * 2.5 - 2.0) for n in lens]
    seqs[0]["z"][40, :d // 2 + 1] = 6.0           # exp(-exp(6)) is zero in float32
    rate = torch.tensor(([1.0, 0.0, 0.9, 0.5, 0.97] * 2)[:H])
    w0 = torch.randn(H * d, generator=g) * 0.5
    bonus = torch.randn(H, d, generator=g)
    want = []
    for s, n in zip(seqs, lens):
        if kind == "fixed":
            q, k, v = (P.silu(s[c].double()).reshape(n, H, -1) for c in "qkv")
            want.append(plain_state_scan(q, k, v, rate.double()[None, :, None].expand(n, H, d),
                                         None))
        else:
            q, k, v = (s[c].double().reshape(n, H, -1) for c in "qkv")
            a = torch.exp(-torch.exp(s["z"].double() + w0.double())).reshape(n, H, d)
            want.append(plain_state_scan(q, k, v, a, bonus.double()))
    states = [torch.full((6, H, dv, d), float("nan"), device=DEV) for _ in range(2)]
    got, walked, done = [[], [], []], [[], [], []], [0, 0, 0]
    for step in ([70, 33, 1], [1, 1, 64], [40, 43, 2], [39, 0, 53]):
        live = [i for i in range(3) if step[i]]
        segs = [(done[i], step[i]) for i in live]
        tb = tables(segs, slots=[[4, 0, 2][i] for i in live])
        ch, first = chunk_tables(segs, rows)
        cat = {c: torch.cat([seqs[i][c][done[i]:done[i] + step[i]] for i in live]).to(DEV)
               for c in "qkvz"}
        outs = []
        for st, kw in ((states[0], dict(chunks=ch, seg_chunk0=first, chunk_rows=rows)),
                       (states[1], {})):
            if kind == "fixed":
                outs.append(ops.matrix_state_recurrence(
                    cat["q"], cat["k"], cat["v"], None, H, H, d, dv, rate.to(DEV), None, 1.0, 1.0,
                    st, tb["seg_start"], tb["seg_pos0"], tb["seg_slot"], decay="fixed",
                    silu_inputs=True, **kw))
            else:
                outs.append(ops.matrix_state_recurrence(
                    cat["q"], cat["k"], cat["v"], cat["z"], H, H, d, dv, None, w0.to(DEV), 1.0,
                    1.0, st, tb["seg_start"], tb["seg_pos0"], tb["seg_slot"], decay="double_exp",
                    bonus=bonus.to(DEV), **kw))
        at = 0
        for i in live:
            got[i].append(outs[0][at:at + step[i]])
            walked[i].append(outs[1][at:at + step[i]])
            at += step[i]
            done[i] += step[i]
    assert done == lens
    for i in range(3):
        assert rel(torch.cat(got[i]), want[i].reshape(lens[i], H * dv)) < 2e-5, i
        assert rel(torch.cat(got[i]), torch.cat(walked[i]).cpu().double()) < 2e-5, i
    for slot in (4, 0, 2):
        assert rel(states[0][slot], states[1][slot].cpu().double()) < 2e-5


# ---------------------------------------------------------------------------------------------
# the mixers as parts, over portions and single tokens
# ---------------------------------------------------------------------------------------------
def chunked_part(dtype, W, H, G, d, dv, chunk, scale, base, dims, stretch=None, keys_as_values=False):
    from kappai_amd.parts import RotaryEncoding, ScoredAttention
    position = None
    if dims:
        st = dict(zip(("factor", "original", "fast", "slow"), stretch)) if stretch else None
        position = RotaryEncoding(d, base, rot_dim=dims, pairing="half", stretch=st)
    return ScoredAttention("a.", W, H, G, d, dv, scale, dtype, sink=keys_as_values, chunk=chunk,
                           position=position, bias=True, bias_suffix=".b", weight_suffix="",
                           values_from_keys=keys_as_values)


def chunked_dict(H, G, d, dv, chunk, scale, base, dims, stretch=None):
    rot = {"base": base, "dims": dims}
    if stretch:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    return {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale, "rot": rot,
            "mask": {"size": chunk}}


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 3e-2)])
@pytest.mark.parametrize("H,G,d,dv,chunk,dims,stretch,kav", [
    (6, 2, 16, 24, 19, 8, None, False), (3, 3, 24, 24, 33, 24, (4.0, 64, 8.0, 1.0), True),
    (1, 1, 40, 8, 1, 0, None, False), (8, 1, 16, 16, 16, 16, (8.0, 32, 1000.0, 0.001), True),
    (18, 1, 16, 32, 1000, 2, None, False), (40, 2, 8, 8, 64, 8, None, True),
    (4, 2, 80, 80, 50, 40, (2.0, 128, 4.0, 2.0), True), (2, 2, 96, 64, 70, 96, None, False)])
def test_chunked_attention_part(dtype, tol, H, G, d, dv, chunk, dims, stretch, kav):
    from kappai_amd.cache import CacheManager
    part = chunked_part(dtype, 72, H, G, d, dv, chunk, 0.3, 700.0, dims, stretch, kav)
    t = bind_random(part, 3, dtype)
    cm = CacheManager([part.cache_spec()], 16, 12, 1)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(14)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    want = P.chunked_attention(x.double(), t, "a.", chunked_dict(H, G, d, dv, chunk, 0.3, 700.0,
                                                                 dims, stretch))
    assert rel(got, want) < tol


def needle_rows(T, needle, H, d, free_from, seed):
    """[T, 2 H d] rows whose first half is what queries read and whose second half is what keys
    read, head by head.  In the places of a head from ``free_from`` on (those no rotation turns)
    every query after the needle points along ``u`` and so does the needle's key; every other key
    lies along ``r`` at right angles to it: all of a later query's weight falls on the needle
    wherever it is, if the query may see it."""
    n = d - free_from
    u = torch.zeros(d)
    u[free_from:] = 1.0 / math.sqrt(n)
    r = torch.zeros(d)
    r[free_from:] = (torch.tensor([1.0, -1.0]).repeat(n // 2)) / math.sqrt(n)
    half = H * d
    x = torch.randn(T, 2 * half, generator=gen(seed)) * 0.02
    x[:, half:] += r.repeat(H)
    x[needle, half:] = 5.0 * u.repeat(H)
    x[needle + 1:, :half] += 4.0 * u.repeat(H)
    return x.to(BF16)


@pytest.mark.parametrize("dtype,tol", [(F32, 1e-4), (BF16, 5e-2)])
@pytest.mark.parametrize("chunk", [64, 70, 200, 500])
def test_a_chunk_holds_a_key_up_to_its_edge_and_not_beyond(dtype, tol, chunk):
    """Queries and keys read the input through identity maps (no biases); half of every head
    turns with the position, the needle lies in the other half.  One key gets all the weight of
    every later query of its chunk and none from the next chunk on: at a chunk's first and last
    position, at page borders, and 400 keys back in a long chunk; in a portion that crosses the
    edge and token by token.  Then a sink so large that nothing else counts."""
    from kappai_amd.cache import CacheManager
    H = G = 2
    d = 16
    half, W = H * d, 2 * H * d
    for keys_as_values in (False, True):
        def build(sink=-20.0):
            part = chunked_part(dtype, W, H, G, d, d, chunk, 1.5, 300.0, 8, None, keys_as_values)

            def change(t):
                eye, zero = torch.eye(half), torch.zeros(half, half)
                t["a.q"] = torch.cat([eye, zero], 1).to(BF16)
                t["a.k"] = torch.cat([zero, eye], 1).to(BF16)
                t["a.q.b"] = torch.zeros(half).to(BF16)
                t["a.k.b"] = torch.zeros(half).to(BF16)
                if keys_as_values:
                    t["a.sink"] = torch.full((H,), sink).to(BF16)
            return part, bind_random(part, 4, dtype, std=0.3, change=change)

        m = chunked_dict(H, G, d, d, chunk, 1.5, 300.0, 8)
        needles = [0, 15, 16, chunk - 1, chunk, chunk + 17] + ([chunk + 63] if chunk >= 450 else [])
        for needle in needles:
            edge = (needle // chunk + 1) * chunk           # the first position that sees it no more
            T = edge + 5
            x = needle_rows(T, needle, H, d, 8, needle)
            part, t = build()
            want = P.chunked_attention(x.double(), t, "a.", m)
            if edge - 1 > needle:
                inside, outside = want[edge - 1], want[edge]
                assert float((inside - outside).abs().max() / want.abs().max()) > 0.2
            for portions in ([needle + 1, T - needle - 8] + [1] * 7,
                             [needle + 2, T - needle - 2] if T - needle - 2 > 0 else [T]):
                portions = [n for n in portions if n > 0]
                if sum(portions) != T:
                    portions = [T - 7] + [1] * 7
                cm = CacheManager([part.cache_spec()], 16, T // 16 + 2, 1)
                cm.allocate_storage(dtype, DEV, poison=True)
                got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
                err = (got.cpu().double() - want).abs().max(dim=1).values / want.abs().max()
                assert float(err.max()) < tol, (needle, keys_as_values, int(err.argmax()))
        if keys_as_values:
            x = needle_rows(chunk + 5, 3, H, d, 8, 1)
            found = P.chunked_attention(x.double(), build()[1], "a.", m)[chunk - 1]
            part, t = build(60.0)
            drowned = P.chunked_attention(x.double(), t, "a.", m)
            assert float(drowned.abs().max()) < 1e-3 * float(found.abs().max())
            cm = CacheManager([part.cache_spec()], 16, (chunk + 5) // 16 + 2, 1)
            cm.allocate_storage(dtype, DEV, poison=True)
            got, _ = step_through(part, cm, x.to(dtype), [chunk - 2] + [1] * 7, cm.view(0))
            assert float(got.abs().max()) < 1e-3 * float(found.abs().max())


@pytest.mark.parametrize("dtype,tol", [(F32, 3e-5), (BF16, 4e-2)])
@pytest.mark.parametrize("H,d,dv,decay", [(3, 8, 16, [0.5, 0.97, 1.0]), (1, 72, 24, [0.9]),
                                          (2, 40, 8, [0.0, 0.999]), (2, 136, 8, [0.8, 0.3]),
                                          (4, 24, 40, [0.3, 0.6, 0.9, 0.99])])
def test_fixed_decay_attention_part(dtype, tol, H, d, dv, decay):
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import FixedDecayAttention
    part = FixedDecayAttention("a.", 72, H, d, dv, decay, 1e-5, dtype, weight_suffix="")
    t = bind_random(part, 7, dtype)
    cm = CacheManager([part.cache_spec()], 16, 1, 2)
    cm.allocate_storage(dtype, DEV, poison=True)
    m = {"heads": H, "dim": d, "vdim": dv, "decay": decay}
    # short portions and single tokens; then portions long enough to be worked chunk by chunk
    for T, portions, seed in ((150, PORTIONS_150, 16), (330, [200, 1, 97, 2, 30], 26)):
        cm = CacheManager([part.cache_spec()], 16, 1, 2)
        cm.allocate_storage(dtype, DEV, poison=True)
        x = torch.randn(T, 72, generator=gen(seed)).to(BF16)
        got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
        assert rel(got, P.fixed_decay_attention(x.double(), t, "a.", m, 1e-5)) < tol, T


@pytest.mark.parametrize("dtype,tol", [(F32, 1e-4), (BF16, 5e-2)])
def test_a_decay_of_one_keeps_a_far_token_and_a_smaller_one_loses_it(dtype, tol):
    """One token's key and value are large, 400 tokens back; every later query points along that
    key.  The head with decay 1 still returns that value, the head with decay 0.9 has lost it:
    token by token and in portions, against the plain statement."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import FixedDecayAttention
    H, d, W = 2, 16, 96
    part = FixedDecayAttention("a.", W, H, d, d, [1.0, 0.9], 1e-5, dtype, weight_suffix="")

    def change(t):
        sel = torch.zeros(H * d, W)
        sel[:, :H * d] = torch.eye(H * d)
        t["a.q"] = sel.to(BF16)
        sel2 = torch.zeros(H * d, W)
        sel2[:, H * d:2 * H * d] = torch.eye(H * d)
        t["a.k"] = sel2.to(BF16)
        sel3 = torch.zeros(H * d, W)
        sel3[:, 2 * H * d:] = torch.eye(H * d)
        t["a.v"] = sel3.to(BF16)
    t = bind_random(part, 8, dtype, std=0.3, change=change)
    T, needle = 420, 9
    x = torch.randn(T, W, generator=gen(17)) * 0.05
    x[:, H * d:2 * H * d] -= 3.0            # silu(-3) is small: ordinary keys write little
    x[needle, H * d:] = 6.0
    x[needle + 1:, :H * d] += 3.0
    x = x.to(BF16)
    m = {"heads": H, "dim": d, "vdim": d, "decay": [1.0, 0.9]}
    want = P.fixed_decay_attention(x.double(), t, "a.", m, 1e-5)
    for portions in ([needle + 1, 380] + [1] * (T - needle - 381), [needle + 2, T - needle - 2]):
        cm = CacheManager([part.cache_spec()], 16, 1, 1)
        cm.allocate_storage(dtype, DEV, poison=True)
        got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
        assert rel(got, want) < tol
    # the plain statement itself: with the far token taken away the last rows change
    y = x.clone()
    y[needle, H * d:] = x[needle + 1, H * d:]
    other = P.fixed_decay_attention(y.double(), t, "a.", m, 1e-5)
    assert float((other[-1] - want[-1]).abs().max()) > 0.2 * float(want[-1].abs().max())


@pytest.mark.parametrize("dtype,tol", [(F32, 3e-5), (BF16, 4e-2)])
@pytest.mark.parametrize("H,d,rank", [(3, 8, 5), (1, 72, 8), (2, 40, 4), (5, 20, 6), (1, 136, 3)])
def test_bonus_time_mixing_part(dtype, tol, H, d, rank):
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import BonusTimeMixing
    part = BonusTimeMixing("a.", 72, H, d, rank, 1e-5, dtype, weight_suffix="")
    t = bind_random(part, 9, dtype)
    cm = CacheManager([part.cache_spec()], 16, 1, 2)
    cm.allocate_storage(dtype, DEV, poison=True)
    m = {"heads": H, "dim": d}
    # short portions and single tokens; then portions long enough to be worked chunk by chunk
    for T, portions, seed in ((150, PORTIONS_150, 18), (330, [200, 1, 97, 2, 30], 27)):
        cm = CacheManager([part.cache_spec()], 16, 1, 2)
        cm.allocate_storage(dtype, DEV, poison=True)
        x = torch.randn(T, 72, generator=gen(seed)).to(BF16)
        got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
        assert rel(got, P.bonus_time_mixing(x.double(), t, "a.", m, 1e-5)) < tol, T


def test_the_bonus_weighs_the_token_itself_and_the_shift_reads_the_token_before():
    """With every mix weight at one the projections read the token BEFORE (so the first token
    reads zeros and returns nothing); with them at zero and a bonus of zero the first token
    returns nothing either (the state is empty and its own product is weighed by zero), while a
    bonus of one returns it."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import BonusTimeMixing
    H, d, W = 2, 8, 40
    x = torch.randn(6, W, generator=gen(19)).to(BF16)
    for mu, bonus in ((1.0, 1.0), (0.0, 0.0), (0.0, 1.0)):
        part = BonusTimeMixing("a.", W, H, d, 3, 1e-5, F32, weight_suffix="")

        def change(t):
            for s in part.MIXES:
                t["a.mu." + s] = torch.full((W,), mu).to(BF16)
            t["a.u"] = torch.full((H, d), bonus).to(BF16)
        t = bind_random(part, 10, F32, std=0.4, change=change)
        cm = CacheManager([part.cache_spec()], 16, 1, 1)
        cm.allocate_storage(F32, DEV, poison=True)
        got, _ = step_through(part, cm, x.float(), [1, 2, 1, 2], cm.view(0))
        want = P.bonus_time_mixing(x.double(), t, "a.", {"heads": H, "dim": d}, 1e-5)
        assert rel(got, want) < 3e-5
        first = float(got[0].abs().max())
        assert (first > 1e-3) == (mu == 0.0 and bonus == 1.0), (mu, bonus, first)


@pytest.mark.parametrize("dtype,tol", [(F32, 3e-5), (BF16, 4e-2)])
@pytest.mark.parametrize("inner,blocks,taps", [(48, 3, 3), (40, 1, 1), (64, 8, 5), (24, 2, 2),
                                               (60, 4, 4), (136, 1, 4), (96, 2, 17)])
def test_real_gated_unit_part(dtype, tol, inner, blocks, taps):
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import RealGatedUnit
    part = RealGatedUnit("a.", 72, inner, blocks, taps, dtype, weight_suffix="", bias_suffix=".b")
    t = bind_random(part, 11, dtype)
    m = {"width": inner, "blocks": blocks}
    # short portions and single tokens; then portions long enough to be scanned chunk by chunk
    for T, portions, seed in ((150, PORTIONS_150, 20), (330, [200, 1, 97, 2, 30], 21)):
        cm = CacheManager([part.cache_spec()], 16, 1, 2)
        cm.allocate_storage(dtype, DEV, poison=True)
        x = torch.randn(T, 72, generator=gen(seed)).to(BF16)
        got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
        assert rel(got, P.gated_channel_recurrence(x.double(), t, "a.", m)) < tol, T


def test_the_gated_unit_keeps_a_far_token_while_its_decay_stays_near_one():
    """``lam`` far below zero makes every decay nearly one: a large input 300 tokens back is still
    in the state at the end; with ``lam`` above zero it is gone at once.  Both against the plain
    statement, in portions that are scanned chunk by chunk and token by token."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import RealGatedUnit
    inner, W, m = 32, 48, {"width": 32, "blocks": 2}
    x = torch.randn(320, W, generator=gen(22)).to(BF16) * 0.02
    x[5] = 4.0
    y = x.clone()
    y[5] = x[6]
    moved = {}
    for lam in (-9.0, 3.0):
        part = RealGatedUnit("a.", W, inner, 2, 2, F32, weight_suffix="", bias_suffix=".b")

        def change(t):
            t["a.lam"] = torch.full((inner,), lam).to(BF16)
            for name in ("a.x.b", "a.conv.b"):       # (no input but the tokens' own)
                t[name] = torch.zeros_like(t[name])
        t = bind_random(part, 12, F32, std=0.3, change=change)
        cm = CacheManager([part.cache_spec()], 16, 1, 1)
        cm.allocate_storage(F32, DEV, poison=True)
        got, _ = step_through(part, cm, x.float(), [6, 280] + [1] * 34, cm.view(0))
        want = P.gated_channel_recurrence(x.double(), t, "a.", m)
        assert rel(got, want) < 1e-4     # (300 decays next to one, each rounded, multiply up)
        without = P.gated_channel_recurrence(y.double(), t, "a.", m)
        moved[lam] = float((without[-1] - want[-1]).abs().max() / want[-1].abs().max())
    assert moved[-9.0] > 0.5 and moved[3.0] < 1e-6, moved


@pytest.mark.parametrize("dtype,tol", [(F32, 3e-5), (BF16, 4e-2)])
@pytest.mark.parametrize("kind", ["parallel", "parallel_2"])
def test_a_pair_of_mixers(dtype, tol, kind):
    """Both mixers of a pair on the same rows, through the builder's own choice of parts: each
    side normed over the width and the two averaged, or added with two weights."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.models.zumuzen import _mixer
    W = 72
    lt = dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.4, rot_base=900.0, rot_dims=8,
              stretch=None, chunk=21)
    if kind == "parallel":
        m = {"left": lt, "right": {"heads": 3, "dim": 8, "vdim": 16, "decay": [0.5, 0.9, 1.0]}}
        plain_m = {"left": chunked_dict(4, 2, 16, 24, 21, 0.4, 900.0, 8),
                   "right": m["right"]}
    else:
        lt.update(vdim=16, stretch={"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0})
        m = {"left": lt, "right": {"heads": 3, "dim": 8, "decay_rank": 5}, "left_scale": 0.7,
             "right_scale": 1.3}
        plain_m = {"left": chunked_dict(4, 2, 16, 16, 21, 0.4, 900.0, 8, (4.0, 64.0, 8.0, 1.0)),
                   "right": m["right"], "left_scale": 0.7, "right_scale": 1.3}
    part = _mixer(kind, m, "a.", W, 1e-5, dtype)
    t = bind_random(part, 13, dtype)
    cm = CacheManager([part.cache_spec()], 16, 12, 2)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, W, generator=gen(23)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    want = P.mixer(kind, x.double(), t, "a.", plain_m, 1e-5)
    assert rel(got, want) < tol


# ---------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------
LENGTHS = {"A": [70, 45, 100, 37], "B": [66, 35, 90], "C": [50, 81, 36], "D": [150, 52, 75],
           "E": [300, 90]}
MIXED_LENGTHS = {"A": [70, 45, 100, 37, 83, 64, 29, 58], "B": [66, 35, 90, 41, 23, 77, 50, 62, 88],
                 "C": [50, 81, 36, 67, 44, 72, 90, 33, 58], "D": [75, 52, 160, 41, 66, 38, 90],
                 "E": [140, 52, 260, 41, 66, 90]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("zumuzen")
    return {name: write_tiny(name, base / name) for name in TINY}


_models = {}


def gpu_model(model_dir, dtype):
    from kappai_amd.models import load_model
    key = (str(model_dir), dtype)
    if key not in _models:
        _models[key] = load_model(model_dir, dtype, DEV)
    return _models[key]


def replay(model_dir, dtype, steps, index, max_tokens, out_dir, slots=4, graphs=True):
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    model = gpu_model(model_dir, dtype)
    cache = make_replay_cache(model, max_tokens, 16, num_slots=slots)
    cache.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cache, DEV, decode_graphs=graphs)
    rep = TraceReplayer(runner, out_dir)
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
    cache.check()
    assert not cache.live_requests()
    assert all(g.allocator.num_used == 0 for g in cache.paged_groups)
    return collect(index, outputs, model.vocab_size), runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("family", ["whole", "prefill_then_decode", "changing_portions", "mixed"])
def test_schedules(tmp_path, model_dirs, name, family, dtype):
    """Every logit of every request.  The mixed family runs in a pool smaller than its requests
    together with four state slots, so pages and slots are taken again."""
    requests = make_requests(TINY[name][0]["vocab"],
                             MIXED_LENGTHS[name] if family == "mixed" else LENGTHS[name], seed=21)
    steps, index, peak = getattr(schedules, family)(requests)
    if family == "mixed":
        assert sum(len(t) for t in requests.values()) > peak
    got, runner = replay(model_dirs[name], dtype, steps, index, peak, tmp_path / "out")
    assert len(got) == sum(len(t) for t in requests.values())
    assert_matches_plain(got, model_dirs[name], requests, dtype, (name, family, dtype))
    if family == "prefill_then_decode":
        assert runner.graph_replays > 0        # single tokens ran from captured graphs


def test_portions_of_two_tokens(tmp_path, model_dirs):
    """A prompt taken two tokens at a time from its start, beside one taken whole."""
    requests = make_requests(TINY["A"][0]["vocab"], [61, 40], seed=24)
    plans = {"r0": (0, [2] * 30 + [1]), "r1": (3, [40])}
    steps, index, peak = schedules.build(requests, plans)
    got, _ = replay(model_dirs["A"], "float32", steps, index, peak, tmp_path / "out")
    assert_matches_plain(got, model_dirs["A"], requests, "float32", "twos")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_chunk(tmp_path, model_dirs, dtype):
    """A short prompt and 330 tokens one by one (chunks of 19, 33 and 16 begun many times, the
    block tables of a graph grown), two requests side by side."""
    for name in ("A", "C"):
        requests = make_requests(TINY[name][0]["vocab"], [350, 290], seed=22)
        plans = {"r0": (0, [20] + [1] * 330), "r1": (5, [3] + [1] * 287)}
        steps, index, peak = schedules.build(requests, plans)
        got, runner = replay(model_dirs[name], dtype, steps, index, peak, tmp_path / name)
        assert_matches_plain(got, model_dirs[name], requests, dtype, (name, dtype))
        assert runner.graph_replays > 250


def test_a_batch_gives_what_its_requests_give_alone(tmp_path, model_dirs):
    """Unequal requests in one step (a long portion, a short one, single tokens) against each
    request stepped alone: the same logits up to rounding, with and without graphs."""
    requests = make_requests(TINY["A"][0]["vocab"], [120, 9, 40], seed=23)
    alone, _ = replay(model_dirs["A"], "float32", *schedules.changing_portions(requests),
                      tmp_path / "alone", graphs=False)
    plans = {"r0": (0, [100] + [1] * 20), "r1": (1, [2, 2] + [1] * 5), "r2": (0, [1, 30, 2, 7])}
    together, _ = replay(model_dirs["A"], "float32", *schedules.build(requests, plans),
                         tmp_path / "together")
    assert alone.keys() == together.keys()
    scale = max(float(np.abs(v).max()) for v in alone.values())
    worst = max(float(np.abs(alone[k] - together[k]).max()) / scale for k in alone)
    assert worst < 1e-5


@pytest.mark.parametrize("name", ["A", "D"])
def test_the_residual_stream_after_every_run_of_a_layer(model_dirs, name):
    """The stream after every run of a layer (a layer inside the passes counts each time) of a
    whole prompt, in float32, against the plain implementation's."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.engine import StepEntry, StepRunner
    model = gpu_model(model_dirs[name], "float32")
    cfg, t = read_model_dir(model_dirs[name])
    tokens = [int(x) for x in np.random.default_rng(3).integers(0, cfg["vocab"], size=41)]
    streams = []
    P.forward(cfg, t, tokens, streams=streams)
    cm = CacheManager(model.cache_specs(), 16, 8, 1)
    cm.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cm, DEV, decode_graphs=False)
    seen = []
    for layer in model.layers:
        inner = layer.forward

        def spy(h, batch, cache, inner=inner, **kw):
            from kappai_amd.kernels import ops
            from kappai_amd.parts.base import WeightedTerms
            kw.pop("next_block", None)       # (the block then leaves its update pending)
            out = inner(h, batch, cache, **kw)
            x = out.resid.detach().clone()
            d = out.delta
            if isinstance(d, WeightedTerms):
                d = ops.pair_norm_sum(d.a, d.b, d.scale_a, d.scale_b)
            if isinstance(d, torch.Tensor):
                x = x + (d.sum(0) if d.dim() == 3 else d).float()
            seen.append(x)
            return out
        layer.forward = spy
    try:
        runner.step([StepEntry(cm.open("a"), tokens, [len(tokens) - 1])])
    finally:
        for layer in model.layers:
            del layer.forward
    assert len(seen) == len(streams) == len(P.layer_order(cfg))
    for i, (got, want) in enumerate(zip(seen, streams)):
        assert rel(got, want) < 2e-5, i


def test_greedy_generation_through_the_engine(model_dirs):
    """Prompts of unequal length through ``Engine.generate`` (its scheduler cuts the prompts into
    portions of 16 beside decoding) against the plain implementation's greedy choice."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    for name in ("A", "B"):
        rng = np.random.default_rng(5)
        prompts = [[int(t) for t in rng.integers(0, TINY[name][0]["vocab"], size=n)]
                   for n in (45, 7, 23)]
        cfg, t = read_model_dir(model_dirs[name])
        want = []
        for p in prompts:
            toks = list(p)
            for _ in range(10):
                toks.append(int(P.forward(cfg, t, toks)[-1].argmax()))
            want.append(toks[len(p):])
        eng = Engine(str(model_dirs[name]), dtype="float32", num_pages=24, max_batch=3, chunk=16,
                     token_budget=24)
        got = eng.generate(prompts, SamplingParams.greedy(n_predict=10))
        assert got == want
        assert eng.cache.num_free_slots == 3
        assert all(g.allocator.num_used == 0 for g in eng.cache.paged_groups)
        eng.shutdown()


def test_command_line(model_dirs, tmp_path):
    """The command line on a model folder and in random-weights mode (a named shape), with the
    sampling options of any other model; ``--time`` prints the stages of the parts."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    prompt = [5, 17, 3, 88, 41, 7, 120]
    cfg, t = read_model_dir(model_dirs["A"])
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(P.forward(cfg, t, toks)[-1].argmax()))
    out = subprocess.run(
        [sys.executable, "-m", "kappai_amd", "-m", str(model_dirs["A"]), "--dtype", "float32",
         "-p", ",".join(map(str, prompt)), "-n", "6", "-t", "0", "--num-pages", "16", "--time"],
        cwd=str(root), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [int(x) for x in out.stdout.split()] == toks[len(prompt):]
    assert "scan" in out.stderr and "short_conv" in out.stderr and "attn" in out.stderr
    made = tmp_path / "made"
    out = subprocess.run(
        [sys.executable, str(root / "bin" / "kappai-cli"), "--random-weights", "zumuzen-tiny",
         "--model", str(made), "--weight-seed", "2", "--weight-std", "0.1", "-n", "5", "-t", "0.8",
         "-k", "20", "-s", "3", "--num-pages", "16", "7 8 9 10"],
        cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert len(out.stdout.split()) == 5 and (made / "config.json").is_file()


def test_trace_runner_program(model_dirs, tmp_path):
    """``bin/trace_run`` on a model folder: steps on standard input, a file of logits for every
    step that asks for some, a line ``done <step>`` after each, state given back at the end."""
    import json
    import subprocess
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    requests = make_requests(TINY["B"][0]["vocab"], [40, 21], seed=25)
    plans = {"r0": (0, [30] + [1] * 10), "r1": (1, [2, 19])}
    steps, index, peak = schedules.build(requests, plans)
    out_dir = tmp_path / "out"
    res = subprocess.run(
        [str(root / "bin" / "trace_run"), "--model", str(model_dirs["B"]), "--dtype", "float32",
         "--out", str(out_dir), "--max-tokens", str(peak)],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
        timeout=600, cwd=str(tmp_path))
    assert res.returncode == 0, res.stderr
    done = [ln for ln in res.stdout.splitlines() if ln.startswith("done ")]
    assert [int(ln.split()[1]) for ln in done] == [s["step"] for s in steps]
    from replay_common import read_outputs
    vocab = TINY["B"][0]["vocab"]
    got = collect(index, read_outputs(out_dir, index, vocab), vocab)
    assert_matches_plain(got, model_dirs["B"], requests, "float32", "trace_run")
