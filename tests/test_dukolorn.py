"""The Dukolorn decoder without a GPU: its configuration (also the sizes that only the tensors'
shapes give), the tensors its parts declare, the caches its layers ask for, the table of biases
by distance, and the engine's own logic (row tables, cache manager with bundles, windows, state
slots, step function, replay) against the plain implementation with the kernels replaced by
torch stand-ins."""
import copy
import json

import pytest
import torch

import emulated_ops
import schedules
from plain import dukolorn as P
from replay_common import collect, make_requests
from tiny_dukolorn import TINY, assert_matches_plain, write_tiny

from kappai_amd.cache import CacheBundle, CacheManager, FixedState, PagedKV
from kappai_amd.config import ConfigError, config_from_dict
from kappai_amd.config.dukolorn import DukolornConfig
from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
from kappai_amd.models import build_model, load_model

LENGTHS = {"U": [70, 45, 100, 37], "V": [66, 35, 90], "W": [50, 81, 36]}
MIXED_LENGTHS = {"U": [70, 45, 100, 37, 83, 64, 29, 58], "V": [66, 35, 90, 41, 23, 77, 50, 62, 88],
                 "W": [50, 81, 36, 67, 44, 72, 90, 33, 58]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("dukolorn")
    return {name: write_tiny(name, base / name) for name in TINY}


def test_config_reads_every_size_from_the_file():
    raw = copy.deepcopy(TINY["U"][0])
    cfg = config_from_dict(raw)
    assert isinstance(cfg, DukolornConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps, cfg.logit_scale) == (211, 72, 1e-5, 0.5)
    assert [l.type for l in cfg.layers] == ["parallel", "latent_attention", "channel_delta"]
    left = cfg.layers[0].mixer["left"]
    assert (left["heads"], left["kv_heads"], left["dim"], left["vdim"]) == (6, 2, 16, 24)
    assert (left["softcap"], left["bias_max"], left["buckets"]) == (8.0, 50.0, 12)
    assert (left["temp_coef"], left["temp_every"]) == (0.4, 16)
    assert cfg.layers[0].mixer["right"] == {"heads": 3, "dim": 8, "vdim": 16, "tau": 6.0,
                                            "decay_rank": 5}
    assert (cfg.layers[0].mixer["left_scale"], cfg.layers[0].mixer["right_scale"]) == (0.7, 1.3)
    m = cfg.layers[1].mixer
    assert (m["kv_rank"], m["rot_dim"], m["rot_dims"], m["rot_base"], m["window"]) == (
        20, 8, 8, 9000.0, 21)
    assert cfg.layers[2].mlp is None and cfg.layers[2].mixer["conv"] == 3
    assert config_from_dict(copy.deepcopy(TINY["V"][0])).layers[1].mixer["window"] is None
    assert cfg.to_dict() == raw


@pytest.mark.parametrize("change,match", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][1].update(type="attention"), "type"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["q_temp"].update(every=0), "every"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][0]["mixer"].pop("right_scale"), "right_scale"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=3), "q/k heads"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
])
def test_config_errors_name_the_key(change, match):
    raw = copy.deepcopy(TINY["U"][0])
    change(raw)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_sizes_that_the_file_leaves_out_come_from_the_tensors(tmp_path, model_dirs):
    """Without ``buckets``, ``decay_rank`` and ``gate_rank`` in config.json the model still loads:
    the shapes of ``rel``, ``a1`` and ``g1`` give them; and gives the same logits."""
    import shutil
    raw = copy.deepcopy(TINY["U"][0])
    raw["layers"][0]["mixer"]["left"].pop("buckets")
    raw["layers"][0]["mixer"]["right"].pop("decay_rank")
    raw["layers"][2]["mixer"].pop("decay_rank")
    raw["layers"][2]["mixer"].pop("gate_rank")
    with pytest.raises(ValueError, match="buckets"):
        build_model(config_from_dict(copy.deepcopy(raw)), "float32")
    folder = tmp_path / "bare"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(raw))
    shutil.copy(model_dirs["U"] / "model.safetensors", folder / "model.safetensors")
    model = load_model(folder, "float32", device="cpu")
    assert model.config.layers[0].mixer["left"]["buckets"] == 12
    assert model.config.layers[0].mixer["right"]["decay_rank"] == 5
    assert (model.config.layers[2].mixer["decay_rank"], model.config.layers[2].mixer["gate_rank"]) \
        == (6, 7)


def test_tensor_names_and_shapes():
    model = build_model(config_from_dict(copy.deepcopy(TINY["U"][0])), "float32")
    shapes = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert shapes["embed"] == (211, 72) and shapes["head"] == (211, 72)
    assert shapes["embed.norm"] == (72,) and shapes["final.norm"] == (72,)
    assert shapes["l0.mix.left.q"] == (96, 72) and shapes["l0.mix.left.k"] == (32, 72)
    assert shapes["l0.mix.left.v"] == (48, 72) and shapes["l0.mix.left.o"] == (72, 144)
    assert shapes["l0.mix.left.q.norm"] == (96,) and shapes["l0.mix.left.k.norm"] == (32,)
    assert shapes["l0.mix.left.rel"] == (12, 6) and shapes["l0.mix.left.sink"] == (6,)
    assert shapes["l0.mix.right.a1"] == (5, 72) and shapes["l0.mix.right.a2"] == (24, 5)
    assert shapes["l0.mix.right.a2.b"] == (24,) and shapes["l0.mix.right.norm"] == (16,)
    assert shapes["l0.mix.right.g"] == (48, 72) and shapes["l0.mix.right.o"] == (72, 48)
    assert shapes["l0.mlp.gate.b"] == (80,) and shapes["l0.mlp.down.b"] == (72,)
    assert shapes["l1.mix.q"] == (3 * 24, 72) and shapes["l1.mix.dkv"] == (28, 72)
    assert shapes["l1.mix.dkv.norm"] == (20,) and shapes["l1.mix.uk"] == (48, 20)
    assert shapes["l1.mix.uv"] == (72, 20) and shapes["l1.mix.sink"] == (3,)
    assert shapes["l2.mix.q"] == (16, 72) and shapes["l2.mix.v"] == (64, 72)
    assert shapes["l2.mix.q.conv"] == (16, 3) and shapes["l2.mix.v.conv"] == (64, 3)
    assert shapes["l2.mix.b"] == (4, 72) and shapes["l2.mix.A_log"] == (4,)
    assert shapes["l2.mix.dt_bias"] == (32,) and shapes["l2.mix.a2"] == (32, 6)
    assert shapes["l2.mix.g1"] == (7, 72) and shapes["l2.mix.g2"] == (64, 7)
    assert "l2.norm2" not in shapes and "l2.norm1" in shapes
    assert not any(n.endswith(".weight") or n.endswith(".bias") for n in shapes)


def test_what_the_layers_ask_of_the_cache_manager():
    model = build_model(config_from_dict(copy.deepcopy(TINY["U"][0])), "float32")
    specs = model.cache_specs()
    assert isinstance(specs[0], CacheBundle)
    assert specs[0].member("left") == PagedKV(2, 32, None)         # heads of 16 / 24 in one size
    assert specs[0].member("right") == FixedState((3, 16, 8), "float32")
    assert specs[1] == PagedKV(1, 32, 21)                           # latent 20 + 8 rotated places
    assert specs[2].member("state") == FixedState((4, 16, 8), "float32")
    assert specs[2].member("conv") == FixedState((2, 2 * 16 + 64), "float32")
    # one tap: the convolution keeps no history and the layer asks for its state alone
    v = build_model(config_from_dict(copy.deepcopy(TINY["V"][0])), "float32").cache_specs()
    assert v[0] == FixedState((1, 8, 24), "float32")
    cm = CacheManager(specs, 16, 8, 2)
    cm.allocate_storage(torch.float32, "cpu")
    assert len(cm.paged_groups) == 2 and cm.paged_groups[1].spec.window == 21
    rc = cm.open("a")
    cm.extend(rc, 40)
    cm.commit(rc, 40)
    assert rc.blocks[1][0] == -1 and rc.blocks[0][0] >= 0    # the window gave its first page back
    assert cm.view(0).part("right").state.shape == (3, 3, 16, 8)
    cm.close(rc)
    cm.check()


@pytest.mark.parametrize("rows,far", [(12, 50.0), (2, 7.0), (32, 200.0), (7, 19.5)])
def test_bias_by_distance_is_the_table_looked_up_by_bucket(rows, far):
    from kappai_amd.parts.scored_attention import distance_bias_columns
    table = torch.randn(rows, 3, generator=torch.Generator().manual_seed(rows))
    cols = distance_bias_columns(table, far)
    assert cols.shape[0] == 3 and cols.shape[1] >= far
    for n in list(range(cols.shape[1] + 40)):
        want = table[P.distance_bucket(n, rows, far)]
        assert torch.equal(cols[:, min(n, cols.shape[1] - 1)], want), n
    assert P.distance_bucket(int(far) + 1, rows, far) == rows - 1


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


@pytest.mark.parametrize("name,family", [("U", f) for f in
                                         ("whole", "prefill_then_decode", "changing_portions",
                                          "mixed")] + [("V", "mixed"), ("W", "mixed")])
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


def test_a_file_may_hold_the_second_norm_of_a_layer_without_feed_forward(tmp_path, model_dirs):
    import shutil

    from kappai_amd.weights import WeightsError
    from kappai_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
    f = SafetensorsFile(model_dirs["U"] / "model.safetensors")
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    tensors["l2.norm2"] = torch.zeros(72, dtype=torch.bfloat16)
    folder = tmp_path / "more"
    folder.mkdir()
    shutil.copy(model_dirs["U"] / "config.json", folder / "config.json")
    write_safetensors(folder / "model.safetensors", tensors)
    assert load_model(folder, "float32", device="cpu").bound
    tensors["l1.mix.k"] = torch.zeros(4, 72, dtype=torch.bfloat16)
    write_safetensors(folder / "model.safetensors", tensors)
    with pytest.raises(WeightsError, match="unexpected tensors .1.: l1.mix.k"):
        load_model(folder, "float32", device="cpu")
