"""The Dapipel decoder without a GPU: its configuration, the tensors its parts declare, the cache
bundle a layer asks for, and the engine's own logic (row tables, cache manager with bundles,
windows, state slots, step function, replay) against the plain implementation with the kernels
replaced by torch stand-ins."""
import copy

import pytest
import torch

import emulated_ops
import schedules
from replay_common import collect, make_requests
from tiny_dapipel import TINY, assert_matches_plain, write_tiny

from kappai_amd.cache import CacheBundle, CacheManager, FixedState, PagedKV
from kappai_amd.config import ConfigError, DapipelConfig, config_from_dict
from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
from kappai_amd.models import build_model, load_model

LENGTHS = {"P": [70, 45, 100, 37], "Q": [66, 35, 90], "R": [50, 81, 36], "S": [97, 40, 71]}
MIXED_LENGTHS = {"P": [70, 45, 100, 37, 83, 64, 29, 58], "Q": [66, 35, 90, 41, 23, 77, 50],
                 "R": [50, 81, 36, 67, 44, 72, 90], "S": [66, 40, 85, 37, 58, 49, 92]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("dapipel")
    return {name: write_tiny(name, base / name) for name in TINY}


def test_config_reads_every_size_from_the_file():
    raw = copy.deepcopy(TINY["P"][0])
    cfg = config_from_dict(raw)
    assert isinstance(cfg, DapipelConfig)
    assert (cfg.vocab_size, cfg.width, cfg.max_positions) == (301, 96, 400)
    assert cfg.max_position_embeddings == 400
    assert (cfg.embedding_scale, cfg.norm_eps, cfg.norm_groups, cfg.canon_taps) == (1.7, 1e-5, 3, 3)
    assert [l.type for l in cfg.layers] == ["mingru", "attention", "attention", "mingru"]
    assert cfg.layers[1].mixer == {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3,
                                   "diff": 0.4, "window": 20}
    assert cfg.layers[2].mixer["window"] is None and cfg.layers[2].mlp is None
    assert cfg.layers[0].mlp == {"kind": "moe", "ff": 40, "experts": 5, "top": 2}
    assert cfg.to_dict() == raw


@pytest.mark.parametrize("change,match", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].update(groups=5), "groups"),
    (lambda c: c["layers"][1].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv heads"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][3]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c.update(canon=None), "canon"),
])
def test_config_errors_name_the_key(change, match):
    raw = copy.deepcopy(TINY["P"][0])
    change(raw)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_tensor_names_and_shapes():
    model = build_model(config_from_dict(copy.deepcopy(TINY["P"][0])), "float32")
    shapes = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert shapes["embed"] == (301, 96) and shapes["pos"] == (400, 96)
    assert shapes["final.norm"] == (96,)
    assert shapes["l0.mix.z"] == (80, 96) and shapes["l0.mix.z.b"] == (80,)
    assert shapes["l0.mix.x.b"] == (80,) and "l0.mix.g.b" not in shapes
    assert shapes["l0.mix.o"] == (96, 80)
    assert shapes["l0.mlp.router"] == (5, 96) and shapes["l0.mlp.e4.down"] == (96, 40)
    assert shapes["l1.mix.q"] == (4 * 2 * 16, 96) and shapes["l1.mix.k"] == (2 * 2 * 16, 96)
    assert shapes["l1.mix.v"] == (2 * 24, 96) and shapes["l1.mix.o"] == (96, 4 * 24)
    assert shapes["l1.mix.lq1"] == (16,) and shapes["l1.canon2"] == (96, 3)
    assert "l2.norm2" not in shapes and "l2.canon2" not in shapes and "l2.canon1" in shapes
    assert not any(n.endswith(".weight") for n in shapes)


def test_a_layer_asks_for_a_bundle_and_the_manager_serves_every_member():
    model = build_model(config_from_dict(copy.deepcopy(TINY["P"][0])), "float32")
    specs = model.cache_specs()
    assert all(isinstance(s, CacheBundle) for s in specs)
    assert specs[1].member("mixer") == PagedKV(4, 32, 20)        # two maps a kv head, one size
    assert specs[2].member("mixer") == PagedKV(6, 32, None)
    assert specs[0].member("mixer") == FixedState((80,), "float32")
    assert specs[0].member("mixer_conv") == FixedState((2, 96), "float32")
    assert dict(specs[2].parts).keys() == {"mixer", "mixer_conv"}
    cm = CacheManager(specs, 16, 8, 2)
    cm.allocate_storage(torch.float32, "cpu")
    assert len(cm.paged_groups) == 2 and cm.paged_groups[0].spec.window == 20
    view = cm.view(1)
    assert view.part("mixer").pool("k").shape == (9, 4, 16, 32)
    assert view.part("ffn_conv").state.shape == (3, 2, 96)
    assert cm.view(0).part("mixer").state.shape == (3, 80)
    rc = cm.open("a")
    cm.extend(rc, 40)
    cm.commit(rc, 40)
    assert rc.blocks[0][0] == -1 and rc.blocks[1][0] >= 0    # the window gave its first page back
    assert cm.export_state(rc, (0, "mixer")).shape == (80,)
    assert set(cm.dump(rc)["caches"]) >= {(0, "mixer"), (1, "mixer"), (1, "ffn_conv")}
    cm.close(rc)
    cm.check()


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


@pytest.mark.parametrize("name,family", [(n, f) for n in "PQ" for f in
                                         ("whole", "prefill_then_decode", "changing_portions",
                                          "mixed")] + [("R", "mixed"), ("S", "mixed")])
def test_schedules_float32(monkeypatch, tmp_path, model_dirs, name, family):
    cfg = TINY[name][0]
    lengths = MIXED_LENGTHS[name] if family == "mixed" else LENGTHS[name]
    requests = make_requests(cfg["vocab"], lengths, seed=21)
    steps, index, peak = getattr(schedules, family)(requests)
    got = run_emulated(monkeypatch, model_dirs[name], steps, index, peak, tmp_path)
    assert len(got) == sum(len(t) for t in requests.values())
    assert_matches_plain(got, model_dirs[name], requests, "float32", (name, family))


def test_a_file_may_hold_the_norm_and_convolution_of_a_feed_forward_that_is_switched_off(
        tmp_path, model_dirs):
    """Layer 2 of configuration P has no feed-forward.  A checkpoint that holds ``l2.norm2`` and
    ``l2.canon2`` all the same loads (they are not read); any other stray tensor is an error."""
    from kappai_amd.weights import WeightsError
    from kappai_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
    import shutil
    f = SafetensorsFile(model_dirs["P"] / "model.safetensors")
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    tensors["l2.norm2"] = torch.ones(96, dtype=torch.bfloat16)
    tensors["l2.canon2"] = torch.zeros(96, 3, dtype=torch.bfloat16)
    folder = tmp_path / "more"
    folder.mkdir()
    shutil.copy(model_dirs["P"] / "config.json", folder / "config.json")
    write_safetensors(folder / "model.safetensors", tensors)
    model = load_model(folder, "float32", device="cpu")
    assert model.bound
    tensors["l1.norm3"] = torch.ones(96, dtype=torch.bfloat16)
    write_safetensors(folder / "model.safetensors", tensors)
    with pytest.raises(WeightsError, match="unexpected tensors .1.: l1.norm3"):
        load_model(folder, "float32", device="cpu")
