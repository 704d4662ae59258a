"""The Zumuzen decoder without a GPU: its configuration (also the size that only a tensor's shape
gives), the tensors its parts declare, the order of its calls and the caches they ask for, the
stretched rotation frequencies, and the engine's own logic (row tables, cache manager with
bundles, state slots, passes, step function, replay) against the plain implementation with the
kernels replaced by torch stand-ins."""
import copy
import json
import math

import numpy as np
import pytest
import torch

import emulated_ops
import schedules
from plain import zumuzen as P
from replay_common import collect, make_requests
from tiny_zumuzen import TINY, assert_matches_plain, write_tiny

from kappai_amd.cache import CacheBundle, CacheManager, FixedState, PagedKV
from kappai_amd.config import ConfigError, config_from_dict
from kappai_amd.config.zumuzen import ZumuzenConfig
from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
from kappai_amd.models import build_model, load_model

LENGTHS = {"A": [70, 45, 100, 37], "B": [66, 35, 90], "C": [50, 81, 36], "D": [75, 52]}
MIXED_LENGTHS = {"A": [70, 45, 100, 37, 83, 64, 29, 58], "B": [66, 35, 90, 41, 23, 77, 50, 62, 88],
                 "C": [50, 81, 36, 67, 44, 72, 90, 33, 58], "D": [75, 52, 60, 41, 66, 38]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("zumuzen")
    return {name: write_tiny(name, base / name) for name in TINY}


def test_config_reads_every_size_from_the_file():
    raw = copy.deepcopy(TINY["A"][0])
    cfg = config_from_dict(raw)
    assert isinstance(cfg, ZumuzenConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps) == (211, 72, 1e-5)
    assert (cfg.loop_start, cfg.loop_stop, cfg.loop_times, cfg.has_loop) == (1, 3, 2, True)
    assert [l.type for l in cfg.layers] == ["parallel", "rglru", "parallel_2"]
    lt = cfg.layers[0].mixer["left"]
    assert (lt["heads"], lt["kv_heads"], lt["dim"], lt["vdim"], lt["scale"]) == (6, 2, 16, 24, 0.9)
    assert (lt["rot_base"], lt["rot_dims"], lt["chunk"], lt["stretch"]) == (9000.0, 8, 19, None)
    assert cfg.layers[0].mixer["right"] == {"heads": 3, "dim": 8, "vdim": 16,
                                            "decay": [0.5, 0.97, 1.0]}
    assert cfg.layers[1].mixer == {"width": 48, "blocks": 3, "conv": 3}
    m = cfg.layers[2].mixer
    assert m["left"]["vdim"] == m["left"]["dim"] == 24           # the values are the keys
    assert m["left"]["stretch"] == {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0}
    assert (m["left_scale"], m["right_scale"], m["right"]["decay_rank"]) == (0.7, 1.3, 5)
    assert cfg.layers[2].mlp is None and cfg.layers[0].mlp == {"kind": "dense", "ff": 80}
    assert not config_from_dict(copy.deepcopy(TINY["C"][0])).has_loop
    assert cfg.to_dict() == raw


@pytest.mark.parametrize("change,match", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][1].update(type="attention"), "type"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5, 0.9]), "decay"),
    (lambda c: c["layers"][1]["mixer"].update(blocks=5), "blocks"),
    (lambda c: c["layers"][2]["mixer"].pop("right_scale"), "right_scale"),
    (lambda c: c["layers"][2]["mixer"]["left"]["rot"]["scaling"].pop("slow"), "slow"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c["loop"].update(stop=4), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
])
def test_config_errors_name_the_key(change, match):
    raw = copy.deepcopy(TINY["A"][0])
    change(raw)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_the_rank_that_the_file_leaves_out_comes_from_the_tensor(tmp_path, model_dirs):
    import shutil
    raw = copy.deepcopy(TINY["A"][0])
    raw["layers"][2]["mixer"]["right"].pop("decay_rank")
    with pytest.raises(ValueError, match="decay_rank"):
        build_model(config_from_dict(copy.deepcopy(raw)), "float32")
    folder = tmp_path / "bare"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(raw))
    shutil.copy(model_dirs["A"] / "model.safetensors", folder / "model.safetensors")
    model = load_model(folder, "float32", device="cpu")
    assert model.config.layers[2].mixer["right"]["decay_rank"] == 5


def test_tensor_names_and_shapes():
    model = build_model(config_from_dict(copy.deepcopy(TINY["A"][0])), "float32")
    shapes = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert shapes["embed"] == (211, 72) and shapes["head"] == (211, 72)
    assert shapes["loop.step"] == (2, 72) and shapes["final.norm"] == (72,)
    assert shapes["l0.mix.left.q"] == (96, 72) and shapes["l0.mix.left.q.b"] == (96,)
    assert shapes["l0.mix.left.k"] == (32, 72) and shapes["l0.mix.left.v"] == (48, 72)
    assert shapes["l0.mix.left.v.b"] == (48,) and shapes["l0.mix.left.o"] == (72, 144)
    assert shapes["l0.mix.left.out"] == (72,) and shapes["l0.mix.right.out"] == (72,)
    assert shapes["l0.mix.right.q"] == (24, 72) and shapes["l0.mix.right.v"] == (48, 72)
    assert shapes["l0.mix.right.g"] == (48, 72) and shapes["l0.mix.right.norm"] == (48,)
    assert shapes["l0.mix.right.o"] == (72, 48) and "l0.mix.left.sink" not in shapes
    assert shapes["l1.mix.y"] == (48, 72) and shapes["l1.mix.x.b"] == (48,)
    assert shapes["l1.mix.conv"] == (48, 3) and shapes["l1.mix.conv.b"] == (48,)
    assert shapes["l1.mix.ra"] == (3, 16, 16) and shapes["l1.mix.ri.b"] == (3, 16)
    assert shapes["l1.mix.lam"] == (48,) and shapes["l1.mix.o"] == (72, 48)
    assert shapes["l2.mix.left.q"] == (96, 72) and shapes["l2.mix.left.k.b"] == (48,)
    assert "l2.mix.left.v" not in shapes and shapes["l2.mix.left.sink"] == (4,)
    assert shapes["l2.mix.left.o"] == (72, 96)
    assert shapes["l2.mix.right.mu.w"] == (72,) and shapes["l2.mix.right.r"] == (24, 72)
    assert shapes["l2.mix.right.w1"] == (5, 72) and shapes["l2.mix.right.w2"] == (24, 5)
    assert shapes["l2.mix.right.w0"] == (24,) and shapes["l2.mix.right.u"] == (3, 8)
    assert shapes["l2.mix.right.norm"] == (24,) and shapes["l2.mix.right.o"] == (72, 24)
    assert "l2.norm2" not in shapes and "l2.norm1" in shapes and "l2.mlp.gate" not in shapes
    assert not any(n.endswith(".weight") or n.endswith(".bias") for n in shapes)


def test_the_order_of_the_calls_and_what_they_ask_of_the_cache_manager():
    model = build_model(config_from_dict(copy.deepcopy(TINY["A"][0])), "float32")
    assert [(c.layer, c.enters) for c in model.schedule] == [
        (0, None), (1, 0), (2, None), (1, 1), (2, None)]
    assert [e.add_embedded for e in model.entries] == [False, True]
    specs = model.cache_specs()
    assert len(specs) == 5 and specs[1] == specs[3] and specs[2] == specs[4]   # a cache a pass
    assert specs[0].member("left") == PagedKV(2, 32, None)         # heads of 16 / 24 in one size
    assert specs[0].member("right") == FixedState((3, 16, 8), "float32")
    assert specs[1].member("state") == FixedState((48,), "float32")
    assert specs[1].member("conv") == FixedState((2, 48), "float32")
    assert specs[2].member("left") == PagedKV(2, 32, None)
    assert specs[2].member("right.state") == FixedState((3, 8, 8), "float32")
    assert specs[2].member("right.shift") == FixedState((72,), "float32")
    # one tap: the convolution keeps no history; a run that starts at layer 0, three times
    b = build_model(config_from_dict(copy.deepcopy(TINY["B"][0])), "float32")
    assert b.cache_specs()[0] == FixedState((40,), "float32")
    assert [(c.layer, c.enters) for c in b.schedule] == [(0, 0), (0, 1), (0, 2), (1, None),
                                                          (2, None)]
    c = build_model(config_from_dict(copy.deepcopy(TINY["C"][0])), "float32")
    assert [(x.layer, x.enters) for x in c.schedule] == [(i, None) for i in range(4)]
    assert not c.entries and "loop.step" not in {s.name for s in c.tensor_specs()}
    cm = CacheManager(specs, 16, 8, 2)
    cm.allocate_storage(torch.float32, "cpu")
    rc = cm.open("a")
    cm.extend(rc, 40)
    cm.commit(rc, 40)
    assert all(b >= 0 for b in rc.blocks[0][:3])          # chunks give no pages back
    cm.close(rc)
    cm.check()


@pytest.mark.parametrize("base,dims,stretch", [
    (3000.0, 16, (4.0, 64, 8.0, 1.0)), (5000.0, 40, (8.0, 32, 1000.0, 0.001)),
    (300000.0, 24, (3.0, 256, 16.0, 2.0)), (10000.0, 64, (1.0, 4096, 32.0, 1.0)),
    (100.0, 8, (16.0, 16, 2.0, 2.0)), (9000.0, 8, None)])
def test_stretched_frequencies(base, dims, stretch):
    """The encoding's tables against the plain statement: unstretched pairs, slowed pairs and
    those between; the factor on cosine and sine."""
    from kappai_amd.parts.rotary import RotaryEncoding
    st = dict(zip(("factor", "original", "fast", "slow"), stretch)) if stretch else None
    enc = RotaryEncoding(dims + 8, base, rot_dim=dims, stretch=st)
    rot = {"base": base, "dims": dims, "scaling": st}
    f, mag = P.rotation_frequencies(rot)
    got_f, got_mag = enc.frequencies()
    assert np.allclose(got_f, f.numpy(), rtol=1e-12) and math.isclose(got_mag, mag)
    cos, sin = enc.tables(300)
    ang = torch.arange(300, dtype=torch.float64)[:, None] * f[None, :]
    assert np.allclose(cos, (torch.cos(ang) * mag).numpy(), atol=1e-6)
    assert np.allclose(sin, (torch.sin(ang) * mag).numpy(), atol=1e-6)
    if stretch and stretch[0] > 1.0:
        plain_f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
        assert (got_f <= plain_f + 1e-15).all() and (got_f >= plain_f / stretch[0] - 1e-15).all()


def run_emulated(monkeypatch, model_dir, steps, index, max_tokens, tmp_path):
    emulated_ops.install(monkeypatch)
    model = load_model(model_dir, "float32", device="cpu")
    cache = make_replay_cache(model, max_tokens, 16, num_slots=4)
    cache.allocate_storage(model.dtype, "cpu", poison=True)
    rep = TraceReplayer(emulated_ops.make_cpu_runner(model, cache), tmp_path / "out")
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
        cache.check()
    assert not cache.live_requests()
    assert all(g.allocator.num_used == 0 for g in cache.paged_groups)
    return collect(index, outputs, model.vocab_size)


@pytest.mark.parametrize("name,family", [("A", f) for f in
                                         ("whole", "prefill_then_decode", "changing_portions",
                                          "mixed")] + [("B", "mixed"), ("C", "mixed"),
                                                       ("D", "changing_portions")])
def test_schedules_float32(monkeypatch, tmp_path, model_dirs, name, family):
    cfg = TINY[name][0]
    lengths = MIXED_LENGTHS[name] if family == "mixed" else LENGTHS[name]
    requests = make_requests(cfg["vocab"], lengths, seed=21)
    steps, index, peak = getattr(schedules, family)(requests)
    if family == "mixed":
        assert sum(len(t) for t in requests.values()) > peak, "the pool must be reused"
    got = run_emulated(monkeypatch, model_dirs[name], steps, index, peak, tmp_path)
    assert len(got) == sum(len(t) for t in requests.values())
    assert_matches_plain(got, model_dirs[name], requests, "float32", (name, family))


def test_the_plain_mechanisms_one_by_one():
    """What the plain statement itself promises: a chunk's first position sees only itself, a
    sink takes weight away, the bonus weighs the token's own product, a decay of one keeps
    everything, and the real-gated unit starts from zero."""
    seen = P.chunk_mask(10, 4)
    assert seen[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert seen[7].tolist() == [False] * 4 + [True] * 4 + [False] * 2
    g = torch.Generator().manual_seed(1)
    W = {"q": torch.eye(4), "q.b": torch.zeros(4), "k": torch.eye(4), "k.b": torch.zeros(4),
         "o": torch.eye(4)}
    m = {"heads": 1, "kv_heads": 1, "dim": 4, "scale": 1.0, "rot": {"base": 10.0, "dims": 0},
         "mask": {"size": 3}}
    h = torch.randn(7, 4, generator=g, dtype=torch.float64)
    plain = P.chunked_attention(h, W, "", m)
    assert torch.allclose(plain[3], h[3]) and torch.allclose(plain[0], h[0])   # chunk starts
    sunk = P.chunked_attention(h, {**W, "sink": torch.tensor([30.0])}, "", m)
    assert float(sunk.abs().max()) < 1e-6 * float(plain.abs().max())           # the sink wins
    # the real-gated unit's first token: S_0 = sqrt(1 - a^2) i u
    Wg = {"y": torch.eye(2), "y.b": torch.zeros(2), "x": torch.eye(2), "x.b": torch.zeros(2),
          "conv": torch.ones(2, 1), "conv.b": torch.zeros(2), "ra": torch.zeros(1, 2, 2),
          "ra.b": torch.zeros(1, 2), "ri": torch.zeros(1, 2, 2), "ri.b": torch.zeros(1, 2),
          "lam": torch.zeros(2), "o": torch.eye(2)}
    x = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    a = math.exp(-8.0 * 0.5 * math.log(2.0))
    want = math.sqrt(1 - a * a) * 0.5 * x * P.gelu_tanh(x)
    assert torch.allclose(P.gated_channel_recurrence(x, Wg, "", {"width": 2, "blocks": 1}), want)


def test_a_file_may_hold_the_second_norm_of_a_layer_without_feed_forward(tmp_path, model_dirs):
    import shutil

    from kappai_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
    f = SafetensorsFile(model_dirs["A"] / "model.safetensors")
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    tensors["l2.norm2"] = torch.zeros(72, dtype=torch.bfloat16)
    folder = tmp_path / "more"
    folder.mkdir()
    shutil.copy(model_dirs["A"] / "config.json", folder / "config.json")
    write_safetensors(folder / "model.safetensors", tensors)
    assert load_model(folder, "float32", device="cpu").bound
