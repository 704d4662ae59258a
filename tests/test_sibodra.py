"""The Sibodra decoder without a GPU: its configuration, the tensors its parts declare, the
caches its layers ask for, the scaled rotation frequencies, and the engine's own logic (row
tables, cache manager, step function, replay) against the plain implementation with the kernels
replaced by torch stand-ins."""
import copy
import json

import numpy as np
import pytest
import torch

import emulated_ops
import schedules
from plain import sibodra as P
from replay_common import collect, make_requests
from tiny_sibodra import TINY, assert_matches_plain, read_model_dir, write_tiny

from kappai_amd.cache import PagedKV
from kappai_amd.config import ConfigError, config_from_dict
from kappai_amd.config.sibodra import SibodraConfig
from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
from kappai_amd.models import build_model, load_model

LENGTHS = {"A": [70, 45, 100, 37], "B": [66, 35, 90], "C": [50, 81, 36], "D": [40, 75], "E": [61, 30, 45]}
MIXED_LENGTHS = {"A": [70, 45, 100, 37, 83, 64, 29, 58], "B": [66, 35, 90, 41, 23, 77, 50, 62, 88],
                 "C": [50, 81, 36, 67, 44, 72, 90, 33, 58], "D": [40, 75, 52, 33, 61, 28],
                 "E": [61, 30, 45, 38, 52, 27, 66]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("sibodra")
    return {name: write_tiny(name, base / name) for name in TINY}


def test_config_reads_every_size_from_the_file():
    raw = copy.deepcopy(TINY["A"][0])
    cfg = config_from_dict(raw)
    assert isinstance(cfg, SibodraConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps, cfg.streams, cfg.logit_softcap) == (
        211, 72, 1e-5, 3, 12.0)
    assert [l.type for l in cfg.layers] == ["attention", "latent_attention", "attention",
                                            "latent_attention"]
    m = cfg.layers[0].mixer
    assert (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], m["softcap"]) == (
        6, 2, 16, 24, 0.2, 8.0)
    assert m["rot"] == {"base": 100.0, "dims": 12,
                        "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64.0}}
    assert cfg.layers[2].mixer["rot"]["scaling"] is None and cfg.layers[2].mlp is None
    m = cfg.layers[1].mixer
    assert (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]) == (
        5, 16, 8, 24, 20, 28)
    assert cfg.layers[1].mlp == {"kind": "moe", "ff": 24, "experts": 6, "top": 2, "shared_ff": 40}
    assert cfg.layers[3].mlp["shared_ff"] is None
    assert cfg.layers[0].mlp == {"kind": "dense", "ff": 80}
    c = config_from_dict(copy.deepcopy(TINY["C"][0]))
    assert c.streams is None and c.logit_softcap == 30.0
    b = config_from_dict(copy.deepcopy(TINY["B"][0]))
    assert b.streams == 1 and b.logit_softcap == 0.0 and b.layers[1].mixer["softcap"] == 0.0
    assert cfg.to_dict() == raw


@pytest.mark.parametrize("change,match", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c["layers"][1].update(type="mingru"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].update(high=0.5), "scaling"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("original"), "original"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][1]["mlp"].pop("expert"), "expert"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "kind"),
])
def test_config_errors_name_the_key(change, match):
    raw = copy.deepcopy(TINY["A"][0])
    change(raw)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_tensor_names_and_shapes():
    model = build_model(config_from_dict(copy.deepcopy(TINY["A"][0])), "float32")
    shapes = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert shapes["embed"] == (211, 72) and shapes["head"] == (211, 72)
    assert shapes["final.norm"] == (72,) and shapes["l0.norm1"] == (72,)
    assert shapes["l0.mix.q"] == (96, 72) and shapes["l0.mix.k"] == (32, 72)
    assert shapes["l0.mix.v"] == (48, 72) and shapes["l0.mix.o"] == (72, 144)
    assert shapes["l0.mix.q.norm"] == (16,) and shapes["l0.mix.k.norm"] == (16,)
    assert shapes["l0.mix.g"] == (6, 72)
    assert shapes["l0.mlp.gate"] == (80, 72) and shapes["l0.mlp.down"] == (72, 80)
    assert shapes["l0.hc1.in"] == (3,) and shapes["l0.hc2.out"] == (3,)
    assert shapes["l0.hc1.mix"] == (3, 3)
    assert shapes["l1.mix.dq"] == (28, 72) and shapes["l1.mix.dq.norm"] == (28,)
    assert shapes["l1.mix.uq"] == (5 * 24, 28) and shapes["l1.mix.dkv"] == (28, 72)
    assert shapes["l1.mix.dkv.norm"] == (20,) and shapes["l1.mix.uk"] == (80, 20)
    assert shapes["l1.mix.uv"] == (120, 20) and shapes["l1.mix.g"] == (120, 72)
    assert shapes["l1.mix.o"] == (72, 120)
    assert shapes["l1.mlp.router"] == (6, 72) and shapes["l1.mlp.router.b"] == (6,)
    assert shapes["l1.mlp.e5.up"] == (24, 72) and shapes["l1.mlp.e0.down"] == (72, 24)
    assert shapes["l1.mlp.shared.up"] == (40, 72) and shapes["l1.mlp.shared.down"] == (72, 40)
    assert "l1.mlp.e0.gate" not in shapes and "l3.mlp.shared.up" not in shapes
    assert "l2.norm2" not in shapes and "l2.hc2.in" not in shapes and "l2.hc1.in" in shapes
    assert not any(n.endswith(".weight") or n.endswith(".bias") for n in shapes)
    plain = build_model(config_from_dict(copy.deepcopy(TINY["C"][0])), "float32")
    assert not any(".hc" in s.name for s in plain.tensor_specs())


def test_what_the_layers_ask_of_the_cache_manager():
    model = build_model(config_from_dict(copy.deepcopy(TINY["A"][0])), "float32")
    assert model.cache_specs() == [PagedKV(2, 32, None), PagedKV(1, 32, None),
                                   PagedKV(3, 32, None), PagedKV(1, 64, None)]


@pytest.mark.parametrize("dims,base,scaling", [(12, 100.0, (4.0, 1.0, 4.0, 64)),
                                               (8, 1000.0, (8.0, 1.0, 2.0, 32)),
                                               (64, 500000.0, (16.0, 1.0, 4.0, 256)),
                                               (24, 10000.0, None)])
def test_rotation_frequencies_scaled_by_wavelength(dims, base, scaling):
    from kappai_amd.parts import RotaryEncoding
    sc = None if scaling is None else dict(zip(("factor", "low", "high", "original"), scaling))
    enc = RotaryEncoding(dims + 8, base, rot_dim=dims, pairing="half", wavelength_scaling=sc)
    freq, factor = enc.frequencies()
    want = P.pair_frequencies(dims, base, sc).numpy()
    assert factor == 1.0 and np.allclose(freq, want, rtol=1e-13, atol=0)
    if scaling is not None:
        plain = P.pair_frequencies(dims, base, None).numpy()
        kinds = {"kept": int((want == plain).sum()),
                 "slowed": int(np.isclose(want, plain / scaling[0], rtol=1e-13).sum())}
        assert kinds["kept"] and kinds["slowed"], kinds     # the case shows both ends of the rule
    cos, sin = enc.tables(50)
    assert np.allclose(cos[37], np.cos(37 * want), atol=1e-6)
    assert np.allclose(sin[37], np.sin(37 * want), atol=1e-6)


def test_a_file_without_the_query_rank_takes_it_from_the_tensor(tmp_path, model_dirs):
    import shutil
    raw = copy.deepcopy(TINY["A"][0])
    raw["layers"][1]["mixer"].pop("q_rank")
    with pytest.raises(ValueError, match="q_rank"):
        build_model(config_from_dict(copy.deepcopy(raw)), "float32")
    folder = tmp_path / "bare"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(raw))
    shutil.copy(model_dirs["A"] / "model.safetensors", folder / "model.safetensors")
    model = load_model(folder, "float32", device="cpu")
    assert model.config.layers[1].mixer["q_rank"] == 28


def test_plain_softmax_with_a_sink_of_score_zero():
    s = torch.tensor([[[0.5, 9.0], [1.0, -2.0]]], dtype=torch.float64)
    w = P.causal_scores_softmax(s, sink_one=True)
    assert torch.allclose(w[0, 0], torch.tensor([np.exp(0.5) / (1 + np.exp(0.5)), 0.0],
                                                dtype=torch.float64))
    den = 1 + np.exp(1.0) + np.exp(-2.0)
    assert torch.allclose(w[0, 1], torch.tensor([np.exp(1.0) / den, np.exp(-2.0) / den],
                                                dtype=torch.float64))
    assert torch.allclose(P.causal_scores_softmax(s, sink_one=False).sum(-1),
                          torch.ones(1, 2, dtype=torch.float64))


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
                                                       ("D", "changing_portions"),
                                                       ("E", "mixed")])
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


def test_a_file_may_hold_what_a_layer_without_feed_forward_leaves_unused(tmp_path, model_dirs):
    import shutil

    from kappai_amd.weights import WeightsError
    from kappai_amd.weights.safetensors_io import write_safetensors
    _, tensors = read_model_dir(model_dirs["A"])
    tensors["l2.norm2"] = torch.zeros(72, dtype=torch.bfloat16)
    tensors["l2.hc2.in"] = torch.zeros(3, dtype=torch.bfloat16)
    folder = tmp_path / "more"
    folder.mkdir()
    shutil.copy(model_dirs["A"] / "config.json", folder / "config.json")
    write_safetensors(folder / "model.safetensors", tensors)
    assert load_model(folder, "float32", device="cpu").bound
    tensors["l1.mix.q"] = torch.zeros(4, 72, dtype=torch.bfloat16)
    write_safetensors(folder / "model.safetensors", tensors)
    with pytest.raises(WeightsError, match="unexpected tensors .1.: l1.mix.q"):
        load_model(folder, "float32", device="cpu")
