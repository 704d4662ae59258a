"""The Sibodra decoder on the GPU against the plain implementation (tests/plain/sibodra.py):
every new kernel alone, the two attention parts and the mixture of experts over portions and
single tokens, keys made to stand out (at position 0, at page borders, hundreds of keys back), a
sink that decides, whole models of four tiny configurations under the four schedule families in
float32 and bfloat16 with pools so small that pages and slots are used again, long decoding, a
batch against its requests alone, the stream's copies after every layer, and greedy generation
through the engine and its scheduler."""
import math

import numpy as np
import pytest
import torch

import schedules
from plain import sibodra as P
from replay_common import collect, make_requests
from tiny_sibodra import TINY, assert_matches_plain, read_model_dir, write_tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16, F64 = torch.float32, torch.bfloat16, torch.float64

LENGTHS = {"A": [70, 45, 100, 37], "B": [66, 35, 90], "C": [50, 81, 36], "D": [40, 75, 130], "E": [61, 30, 45]}
MIXED_LENGTHS = {"A": [70, 45, 100, 37, 83, 64, 29, 58], "B": [66, 35, 90, 41, 23, 77, 50, 62, 88],
                 "C": [50, 81, 36, 67, 44, 72, 90, 33, 58], "D": [40, 75, 52, 33, 61, 28, 97],
                 "E": [61, 30, 45, 38, 52, 27, 66]}


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rel(got, want):
    got = got.detach().to("cpu", F64)
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def bind_random(part, seed, dtype, std=0.2, change=None):
    from kappai_amd.weights import random_tensors, stored_to_runtime
    t = random_tensors(part.tensor_specs(), seed, std=std, norm_jitter=0.1)
    if change:
        change(t)
    part.bind({k: stored_to_runtime(v, dtype).to(DEV) for k, v in t.items()})
    return t


def step_through(part, cm, x, portions, view):
    """One request through a mixer in ``portions``; returns the outputs in order."""
    from test_parts_gpu import one_segment_batch
    rc, outs, done = None, [], 0
    for n in portions:
        rc, b = one_segment_batch(cm, n, rc=rc)
        y = part.forward(x[done:done + n].to(DEV), b, view)
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
@pytest.mark.parametrize("S", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("W", [72, 64, 328, 2048, 100, 67, 30])
def test_one_pass_over_the_copies_of_the_stream(S, W):
    """Update, weighted sum and layer norm in one kernel, against their formulas in float64: the
    update as float32 rows, bfloat16 rows and float32 partial sums; the read half alone; the write
    half alone; copies made from one row; only some rows read."""
    from kappai_amd.kernels import ops
    T, eps = 19, 1e-5
    g = gen(S * 1000 + W)
    x = torch.randn(T, S, W, generator=g) * 3 + 0.5
    mix = torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)
    out_w, in_w = torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw = 1 + 0.2 * torch.randn(W, generator=g)

    def want_of(xs, y):
        new = xs.double()
        if y is not None:
            upd = y.double().sum(0) if y.dim() == 3 else y.double()
            new = torch.einsum("st,nsw->ntw", mix.double(), xs.double()) \
                + out_w.double()[None, :, None] * upd[:, None, :]
        u = torch.einsum("s,nsw->nw", in_w.double(), new)
        return new, P.layer_norm(u, nw, eps)

    for kind in ("f32", "bf16", "parts", "read"):
        y = torch.randn(T, W, generator=g)
        if kind == "bf16":
            y = y.to(BF16)
        elif kind == "parts":
            y = torch.randn(5, T, W, generator=g)
        elif kind == "read":
            y = None
        new, normed = want_of(x, y)
        streams = x.clone().to(DEV)
        rows = ops.hyper_step(streams, S, W, y=None if y is None else y.to(DEV),
                              mix=mix.to(DEV), out_w=out_w.to(DEV), in_w=in_w.to(DEV),
                              norm_w=nw.to(DEV), eps=eps, rows_dtype=F32)
        assert rel(streams, new) < 2e-6, kind
        assert rel(rows, normed) < 2e-5, kind
    # the write half alone, then rounded rows of a read
    y = torch.randn(T, W, generator=g).to(BF16)
    new, normed = want_of(x, y)
    streams = x.clone().to(DEV)
    assert ops.hyper_step(streams, S, W, y=y.to(DEV), mix=mix.to(DEV), out_w=out_w.to(DEV)) is None
    assert rel(streams, new) < 2e-6
    rows = ops.hyper_step(streams, S, W, in_w=in_w.to(DEV), norm_w=nw.to(DEV), eps=eps,
                          rows_dtype=BF16)
    assert rows.dtype == BF16 and rel(rows.float(), normed) < 1e-2
    # copies made from one row
    src = torch.randn(T, W, generator=g)
    made = torch.full((T, S, W), float("nan"), device=DEV)
    rows = ops.hyper_step(made, S, W, source=src.to(DEV), in_w=in_w.to(DEV), norm_w=nw.to(DEV),
                          eps=eps, rows_dtype=F32)
    assert torch.equal(made.cpu(), src[:, None, :].expand(T, S, W))
    assert rel(rows, P.layer_norm(src.double() * in_w.double().sum(), nw, eps)) < 2e-5
    # some rows only: the update is applied for them on the way and nothing is stored
    pick = torch.tensor([17, 0, 5], dtype=torch.int32)
    streams = x.clone().to(DEV)
    rows = ops.hyper_step(streams, S, W, y=y.to(DEV), mix=mix.to(DEV), out_w=out_w.to(DEV),
                          in_w=in_w.to(DEV), norm_w=nw.to(DEV), eps=eps, rows=pick.to(DEV),
                          rows_dtype=F32)
    assert torch.equal(streams.cpu(), x)
    assert rel(rows, normed[pick.long()]) < 2e-5


def test_layer_norm_part_keeps_the_norm_interface():
    """On one stream [T, width]: the pending update is added in float32 and the rows normalised;
    with ``rows`` the stream stays as it is."""
    from kappai_amd.parts import LayerNorm
    T, W = 9, 88
    norm = LayerNorm("n", W, 1e-6, BF16)
    t = bind_random(norm, 3, BF16)
    x, d = torch.randn(T, W, generator=gen(1)) * 4, torch.randn(3, T, W, generator=gen(2))
    resid = x.clone().to(DEV)
    got = norm.add_norm(resid, d.to(DEV))
    assert rel(resid, x.double() + d.double().sum(0)) < 1e-6
    assert rel(got.float(), P.layer_norm(x.double() + d.double().sum(0), t["n"], 1e-6)) < 1e-2
    pick = torch.tensor([4, 8], dtype=torch.int32, device=DEV)
    before = resid.clone()
    got = norm.add_norm(resid, d[0].to(DEV), rows=pick)
    assert torch.equal(resid, before) and got.shape == (2, W)
    want = P.layer_norm(before.cpu().double() + d[0].double(), t["n"], 1e-6)[[4, 8]]
    assert rel(got.float(), want) < 1e-2


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_small_kernels_around_the_attention_layers(dtype):
    from kappai_amd.kernels import ops
    tol = 1e-6 if dtype == F32 else 1e-2
    T = 23
    x = (torch.randn(T, 50, generator=gen(1)) * 2).to(dtype)
    w = 1 + 0.3 * torch.randn(28, generator=gen(2))
    got = ops.rows_rmsnorm(x.to(DEV)[:, 3:45], 28, w.to(DEV), 1e-5)
    assert got.dtype == dtype and got.shape == (T, 28)
    assert rel(got.float(), P.rms_norm(x[:, 3:31].double(), w, 1e-5)) < tol
    for n, group in ((5 * 24, 24), (120, 1), (7, 7)):
        a = torch.randn(T, n, generator=gen(3)).to(dtype)
        gate = torch.randn(T, n // group + 9, generator=gen(4)).to(dtype)
        got = ops.sigmoid_gate(a.clone().to(DEV), gate.to(DEV)[:, 2:2 + n // group], group)
        want = a.double() * torch.sigmoid(gate[:, 2:2 + n // group].double()).repeat_interleave(
            group, dim=1)
        assert rel(got.float(), want) < tol
    z = (torch.randn(T, 77, generator=gen(5)) * 3).to(dtype)
    assert rel(ops.activate(z.to(DEV)).float(), torch.relu(z.double()) ** 2) < tol
    logits = torch.randn(T, 211, generator=gen(6)) * 40
    got = ops.softcap_rows(logits.clone().to(DEV), 30.0)
    assert rel(got, P.cap(logits.double(), 30.0)) < 1e-6


# ---------------------------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------------------------
def attention_dict(H, G, d, dv, scale, softcap, base, dims, scaling):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale, "softcap": softcap,
            "rot": rot}


def make_attention(W, m, dtype):
    from kappai_amd.parts import RotaryEncoding, ScoredAttention
    rot = m["rot"]
    pos = None
    if rot["dims"]:
        pos = RotaryEncoding(m["dim"], rot["base"], rot_dim=rot["dims"], pairing="half",
                             wavelength_scaling=rot.get("scaling"))
    return ScoredAttention("a.", W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
                           dtype, norm_eps=1e-5, softcap=m["softcap"] or 0.0, head_qk_norm=True,
                           sink_value=0.0, head_gate=True, position=pos, weight_suffix="")


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 3e-2)])
@pytest.mark.parametrize("H,G,d,dv,dims,scaling,softcap", [
    (6, 2, 16, 24, 12, (4.0, 1.0, 4.0, 64), 8.0), (3, 3, 24, 16, 24, None, 30.0),
    (1, 1, 40, 8, 8, (8.0, 1.0, 2.0, 32), None), (8, 1, 16, 16, 16, None, 0.5),
    (4, 2, 64, 64, 32, (8.0, 1.0, 4.0, 128), 50.0), (2, 2, 100, 20, 0, None, 5.0)])
def test_attention_part(dtype, tol, H, G, d, dv, dims, scaling, softcap):
    """Per-head norms, partial rotation with scaled frequencies, capped scores, the sink of score
    zero and a gate a head, over portions down to one token."""
    from kappai_amd.cache import CacheManager
    m = attention_dict(H, G, d, dv, 0.2, softcap, 700.0, dims, scaling)
    part = make_attention(72, m, dtype)
    t = bind_random(part, 4, dtype)
    cm = CacheManager([part.cache_spec()], 16, 12, 1)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(14)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    assert rel(got, P.attention(x.double(), t, "a.", m, 1e-5)) < tol


def needle_rows(T, needle, half, seed, others=1.0):
    """[T, 2 half] rows whose first half is what queries read and whose second half is what keys
    read.  Every query after the needle points along ``u``; the needle's key does too, every other
    key lies along ``others * r`` (``r`` at right angles to ``u``) but for a little noise."""
    u = torch.ones(half) / math.sqrt(half)
    r = u * torch.tensor([1.0, -1.0]).repeat(half // 2)
    x = torch.randn(T, 2 * half, generator=gen(seed)) * 0.02
    x[:, half:] += others * r
    x[needle, half:] = 3.0 * u
    x[needle + 1:, :half] += 1.5 * u
    return x.to(BF16)


@pytest.mark.parametrize("dtype,tol", [(F32, 1e-4), (BF16, 5e-2)])
def test_attention_finds_a_far_key_and_weighs_the_sink(dtype, tol):
    """Queries read the first half of the input and keys the second (identity maps; the norm of
    every head gives all keys the same length, so only the direction counts): one needle row
    takes nearly all the weight of every later query, at position 0, at page borders and 400 keys
    back, in a portion and token by token.  Then every key points away from the queries: the sink
    of score zero takes the weight and the result is near nothing, where a softmax without the
    sink would still return a mean of the values."""
    from kappai_amd.cache import CacheManager
    H = G = 2
    d = dv = 16
    half = H * d
    W = 2 * half
    m = attention_dict(H, G, d, dv, 1.0, 40.0, 10000.0, 4, None)

    def change(t):
        eye, zero = torch.eye(half), torch.zeros(half, half)
        t["a.q"] = torch.cat([eye, zero], 1).to(BF16)
        t["a.k"] = torch.cat([zero, eye], 1).to(BF16)
        t["a.q.norm"] = torch.full((d,), 1.0).to(BF16)
        t["a.k.norm"] = torch.full((d,), 1.0).to(BF16)
        t["a.g"] = torch.zeros(H, W).to(BF16)

    part = make_attention(W, m, dtype)
    t = bind_random(part, 4, dtype, std=0.3, change=change)
    for needle in (0, 15, 16, 63):
        T = needle + 403
        x = needle_rows(T, needle, half, needle)
        want = P.attention(x.double(), t, "a.", m, 1e-5)
        # the needle decides: without it the last row's result is another one
        gone = x.clone()
        gone[needle, half:] = gone[needle + 1, half:]
        other = P.attention(gone.double(), t, "a.", m, 1e-5)
        assert float((want[-1] - other[-1]).abs().max()) > 0.2 * float(want[-1].abs().max())
        for portions in ([needle + 1, T - needle - 7] + [1] * 6, [needle + 2, T - needle - 2]):
            cm = CacheManager([part.cache_spec()], 16, T // 16 + 2, 1)
            cm.allocate_storage(dtype, DEV, poison=True)
            got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
            err = (got.cpu().double() - want).abs().max(dim=1).values / want.abs().max()
            assert float(err.max()) < tol, (needle, int(err.argmax()), float(err.max()))
    # every key against the queries: all scores far below zero, the sink takes the weight
    T = 90
    u = torch.ones(half) / math.sqrt(half)
    x = torch.randn(T, W, generator=gen(7)) * 0.02
    x[:, :half] += 1.5 * u
    x[:, half:] -= u
    x = x.to(BF16)
    want = P.attention(x.double(), t, "a.", m, 1e-5)
    full = float((x.double() @ t["a.v"].double().T @ t["a.o"].double().T).abs().max())
    assert float(want.abs().max()) < 1e-3 * full
    cm = CacheManager([part.cache_spec()], 16, T // 16 + 2, 1)
    cm.allocate_storage(dtype, DEV, poison=True)
    got, _ = step_through(part, cm, x.to(dtype), [40, 2] + [1] * 48, cm.view(0))
    assert float(got.abs().max()) < 1e-3 * full


def latent_dict(H, d, rot, dv, r, qr, scale, base):
    return {"heads": H, "dim": d, "rot_dim": rot, "vdim": dv, "kv_rank": r, "q_rank": qr,
            "scale": scale, "rot": {"base": base, "dims": rot}}


def make_latent(W, m, dtype):
    from kappai_amd.parts import LatentAttention, RotaryEncoding
    pos = None
    if m["rot_dim"]:
        pos = RotaryEncoding(m["rot_dim"], m["rot"]["base"], rot_dim=m["rot_dim"], pairing="half")
    return LatentAttention("a.", W, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                           m["scale"], 1e-5, dtype, position=pos, q_rank=m["q_rank"], gate=True,
                           weight_suffix="")


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 3e-2)])
@pytest.mark.parametrize("H,d,rot,dv,r,qr", [(3, 16, 8, 24, 20, 28), (2, 8, 16, 8, 40, 12),
                                             (4, 24, 8, 16, 24, 16), (5, 32, 16, 40, 64, 48),
                                             (1, 10, 2, 6, 7, 5), (8, 24, 16, 72, 56, 96)])
def test_latent_attention_part(dtype, tol, H, d, rot, dv, r, qr):
    """Queries through their own normed latent, rotate-half pairs on the shared key part, a gate a
    channel, over portions down to one token."""
    from kappai_amd.cache import CacheManager
    m = latent_dict(H, d, rot, dv, r, qr, 0.2, 700.0)
    part = make_latent(72, m, dtype)
    t = bind_random(part, 5, dtype)
    cm = CacheManager([part.cache_spec()], 16, 12, 1)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(15)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    assert rel(got, P.latent_attention(x.double(), t, "a.", m, 1e-5)) < tol


@pytest.mark.parametrize("dtype,tol", [(F32, 1e-4), (BF16, 5e-2)])
def test_latent_attention_finds_a_far_key(dtype, tol):
    """Both latents are the input itself (identity maps, norm weights of one), keys and queries
    read them through identity up-projections, nothing rotates: one needle row gets nearly all the
    weight of every later query, wherever it lies."""
    from kappai_amd.cache import CacheManager
    H, d, r = 2, 16, 32
    W = 2 * r
    m = latent_dict(H, d, 0, d, r, r, 1.0, 10.0)
    part = make_latent(W, m, dtype)

    def change(t):
        eye, zero = torch.eye(r), torch.zeros(r, r)
        t["a.dq"] = torch.cat([eye, zero], 1).to(BF16)
        t["a.dq.norm"] = torch.full((r,), 1.0).to(BF16)
        t["a.uq"] = torch.eye(r).to(BF16)
        t["a.dkv"] = torch.cat([zero, eye], 1).to(BF16)
        t["a.dkv.norm"] = torch.full((r,), 1.0).to(BF16)
        t["a.uk"] = (torch.eye(r) * 0.5).to(BF16)
        t["a.g"] = torch.zeros(H * d, W).to(BF16)
    t = bind_random(part, 6, dtype, std=0.3, change=change)
    for needle in (0, 15, 16, 63, 100):
        T = needle + 303
        x = needle_rows(T, needle, r, needle)
        want = P.latent_attention(x.double(), t, "a.", m, 1e-5)
        gone = x.clone()
        gone[needle, r:] = gone[needle + 1, r:]
        other = P.latent_attention(gone.double(), t, "a.", m, 1e-5)
        assert float((want[-1] - other[-1]).abs().max()) > 0.2 * float(want[-1].abs().max())
        for portions in ([needle + 1, T - needle - 7] + [1] * 6, [needle + 2, T - needle - 2]):
            cm = CacheManager([part.cache_spec()], 16, T // 16 + 2, 1)
            cm.allocate_storage(dtype, DEV, poison=True)
            got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
            err = (got.cpu().double() - want).abs().max(dim=1).values / want.abs().max()
            assert float(err.max()) < tol, (needle, int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 3e-2)])
@pytest.mark.parametrize("W,F,E,top,shared,T", [(72, 24, 6, 2, 40, 37), (64, 32, 8, 3, None, 150),
                                                (48, 8, 3, 3, 8, 5), (96, 48, 12, 1, 16, 300),
                                                (100, 40, 10, 4, 24, 1), (64, 16, 4, 2, 64, 2)])
def test_experts_without_gate_with_router_bias_and_shared_expert(dtype, tol, W, F, E, top, shared,
                                                                 T):
    """Rows are made so that no choice of the router is close: the chosen logits stand clear of
    the others by the bias and a large router matrix."""
    from kappai_amd.parts import MixtureOfExperts
    part = MixtureOfExperts("f.", W, F, E, top, dtype, weight_suffix="",
                            activation="relu_squared", router_bias=True, bias_suffix=".b",
                            shared_hidden=shared)

    def change(t):
        t["f.router"] = (t["f.router"].float() * 8).to(BF16)
        t["f.router.b"] = (torch.randn(E, generator=gen(9)) * 2).to(BF16)
    t = bind_random(part, 8, dtype, change=change)
    x = torch.randn(T, W, generator=gen(18)).to(BF16)
    mlp = {"router": {"experts": E, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    rounding = None if dtype == F32 else BF16
    want = P.moe_ff(x.double(), t, "f.", mlp)
    # leave out rows whose choice is a close call for bfloat16 sums
    logits = x.double() @ t["f.router"].double().T + t["f.router.b"].double()
    srt = logits.sort(dim=1, descending=True).values
    clear = torch.ones(T, dtype=torch.bool) if top == E else (srt[:, top - 1] - srt[:, top]) > 0.05
    got = part.forward(x.to(dtype).to(DEV), None).float().cpu().double()
    assert clear.sum() >= max(1, T // 2)
    assert float((got[clear] - want[clear]).abs().max() / want.abs().max()) < tol


# ---------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("sibodra")
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path, model_dirs, dtype):
    """A short prompt and 330 tokens one by one (pages taken one after the other, the block tables
    of a graph grown, the rotation tables grown past their first size), two requests side by
    side.  In bfloat16 the configuration whose routers choose every expert is held to the plain
    implementation row by row to the end; the others meet a router's close call early, from where
    on their rows must stay finite and of the logits' size (their float32 runs are held to every
    row)."""
    for name in ("A", "B", "D"):
        requests = make_requests(TINY[name][0]["vocab"], [350, 290], seed=22)
        plans = {"r0": (0, [20] + [1] * 330), "r1": (5, [3] + [1] * 287)}
        steps, index, peak = schedules.build(requests, plans)
        got, runner = replay(model_dirs[name], dtype, steps, index, peak, tmp_path / name)
        assert_matches_plain(got, model_dirs[name], requests, dtype, (name, dtype),
                             min_strict=1.0 if name == "B" else 0.0)
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


@pytest.mark.parametrize("name", ["A", "C"])
def test_the_residual_stream_layer_by_layer(model_dirs, name):
    """The sum of the stream's copies after every layer of a whole prompt, in float32, against the
    plain implementation's (a layer leaves its last update pending; it is applied here)."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.engine import StepEntry, StepRunner
    model = gpu_model(model_dirs[name], "float32")
    cfg, t = read_model_dir(model_dirs[name])
    tokens = [int(x) for x in np.random.default_rng(3).integers(0, cfg["vocab"], size=41)]
    sums = []
    P.forward(cfg, t, tokens, layers_out=sums)
    cm = CacheManager(model.cache_specs(), 16, 8, 1)
    cm.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cm, DEV, decode_graphs=False)
    seen = []
    for layer in model.layers:
        inner = layer.forward

        def spy(h, batch, cache, shared_cache=False, inner=inner):
            out = inner(h, batch, cache, shared_cache=shared_cache)
            x, up = out.resid.detach().cpu().double(), out.delta
            y = up.y.detach().cpu().double()
            y = y.sum(0) if y.dim() == 3 else y
            new = torch.einsum("st,nsw->ntw", up.mix.cpu().double(), x) \
                + up.out.cpu().double()[None, :, None] * y[:, None, :]
            seen.append(new.sum(1))
            return out
        layer.forward = spy
    try:
        runner.step([StepEntry(cm.open("a"), tokens, [len(tokens) - 1])])
    finally:
        for layer in model.layers:
            del layer.forward
    assert len(seen) == len(sums)
    for i, (got, want) in enumerate(zip(seen, sums)):
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
    sampling options of any other model."""
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
    assert "router" in out.stderr and "attn" in out.stderr
    made = tmp_path / "made"
    out = subprocess.run(
        [sys.executable, str(root / "bin" / "kappai-cli"), "--random-weights", "sibodra-tiny",
         "--model", str(made), "--weight-seed", "2", "--weight-std", "0.1", "-n", "5", "-t", "0.8",
         "-k", "20", "-s", "3", "--num-pages", "16", "7 8 9 10"],
        cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert len(out.stdout.split()) == 5 and (made / "config.json").is_file()
