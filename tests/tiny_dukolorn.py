"""Tiny Dukolorn configurations that differ in every size and option, and helpers that write them
as model folders with random weights and hold results to the plain implementation."""
from __future__ import annotations

import copy
import json

import numpy as np
import torch

from kappai_amd.config import config_from_dict
from kappai_amd.weights import write_random_model


def parallel(heads, kv_heads, dim, vdim, scale, softcap, buckets, bias_max, coef, every,
             r_heads, r_dim, r_vdim, tau, rank, left_scale, right_scale, mlp):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "softcap": softcap, "bias_max": bias_max, "buckets": buckets,
            "q_temp": {"coef": coef, "every": every}}
    right = {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": tau, "decay_rank": rank}
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left, "right": right, "left_scale": left_scale,
                      "right_scale": right_scale}}


def latent(heads, dim, rot_dim, vdim, rank, scale, base, dims, window, mlp):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
             "scale": scale, "rot": {"base": base, "dims": dims}}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank, mlp):
    return {"type": "channel_delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                      "decay_rank": decay_rank, "gate_rank": gate_rank}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(vocab, width, eps, logit_scale, layers):
    return {"architecture": "Dukolorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "logit_scale": logit_scale, "layers": layers}


# every mixer once; three query heads a kv head, values wider than keys on the left and narrower
# on the right; a table of 12 rows that ends at distance 50; a window of 21 (no multiple of a
# page); two q/k heads for four value heads in the delta rule, three taps
TINY_U = config(211, 72, 1e-5, 0.5, [
    parallel(6, 2, 16, 24, 0.2, 8.0, 12, 50.0, 0.4, 16, 3, 8, 16, 6.0, 5, 0.7, 1.3, dense(80)),
    latent(3, 16, 8, 24, 20, 0.21, 9000.0, 8, 21, dense(64)),
    delta(4, 2, 8, 16, 3, 6, 7, None),
])
INIT_U = dict(seed=31, std=0.15, norm_jitter=0.0)

# the delta rule first (one tap: no history; one head), a latent attention without a window whose
# rotation covers only part of the rotated places, a pair whose left side has one head, a cap so
# small that it bends every score, a table of two rows, temperature steps every 3 positions
TINY_V = config(97, 48, 1e-6, 1.0, [
    delta(1, 1, 24, 8, 1, 3, 2, dense(56)),
    latent(2, 8, 16, 8, 40, 0.3, 50.0, 12, None, None),
    parallel(1, 1, 24, 8, 0.3, 0.5, 2, 7.0, 1.5, 3, 2, 40, 8, 1.0, 4, 1.0, 0.25, dense(40)),
])
INIT_V = dict(seed=32, std=0.2, norm_jitter=0.0)

# keys wider than one lane group of the recurrence (72 and 136 key channels), five taps, a window
# of one key (a position sees itself and the sink), eight heads on eight kv heads
TINY_W = config(150, 64, 1e-5, 0.125, [
    latent(4, 8, 8, 16, 24, 0.25, 10000.0, 8, 1, dense(48)),
    parallel(8, 8, 8, 8, 0.35, 20.0, 6, 30.0, 0.2, 7, 1, 72, 24, 3.0, 8, 0.5, 0.5, None),
    delta(2, 2, 136, 8, 5, 4, 4, dense(32)),
    latent(2, 24, 8, 8, 16, 0.18, 300.0, 8, 33, None),
])
INIT_W = dict(seed=33, std=0.12, norm_jitter=0.0)

# sizes in between: attention heads of 48, 80 and 96 once widened (two kv heads of 32 / 48, five
# heads on a latent of 64 + 16, two on 64 + 32), four heads on one kv head, a window of 50, two
# taps, three q/k heads for six value heads, a table whose linear half ends at 16
TINY_X = config(500, 192, 1e-5, 0.7, [
    parallel(6, 3, 32, 48, 0.17, 15.0, 10, 100.0, 0.25, 50, 4, 24, 40, 4.0, 6, 0.9, 0.6,
             dense(256)),
    latent(5, 32, 16, 40, 64, 0.14, 5000.0, 16, 50, dense(200)),
    delta(6, 3, 48, 24, 2, 5, 5, None),
    latent(2, 16, 32, 16, 64, 0.2, 20000.0, 32, None, dense(128)),
    parallel(4, 1, 64, 64, 0.125, 50.0, 32, 64.0, 0.1, 40, 2, 64, 32, 16.0, 8, 1.0, 1.0, None),
])
INIT_X = dict(seed=34, std=0.08, norm_jitter=0.0)

TINY = {"U": (TINY_U, INIT_U), "V": (TINY_V, INIT_V), "W": (TINY_W, INIT_W),
        "X": (TINY_X, INIT_X)}


def write_tiny(name: str, folder, **overrides):
    cfg, init = TINY[name]
    return write_random_model(folder, config_from_dict(copy.deepcopy(cfg)), **{**init, **overrides})


def read_model_dir(model_dir):
    """(config dictionary, {name: tensor}) of a model folder, for the plain implementation."""
    from kappai_amd.weights.safetensors_io import SafetensorsFile
    cfg = json.loads((model_dir / "config.json").read_text())
    f = SafetensorsFile(model_dir / "model.safetensors")
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    return cfg, tensors


_plain_cache = {}


def plain_logits(model_dir, requests, rounding=None):
    """{id: float64 numpy [len, vocab]} from the plain implementation (cached per folder)."""
    from plain import dukolorn as plain
    key = (str(model_dir), json.dumps(requests, sort_keys=True), str(rounding))
    if key not in _plain_cache:
        cfg, t = read_model_dir(model_dir)
        _plain_cache[key] = {rid: plain.forward(cfg, t, toks, rounding=rounding).numpy()
                             for rid, toks in requests.items()}
    return _plain_cache[key]


def row_errors(got, ref):
    """{(id, pos): error of the row}: root mean square of the difference with its mean taken off,
    over the root mean square of all reference logits."""
    scale = float(np.sqrt(np.mean([np.mean(v * v) for v in ref.values()])))
    out = {}
    for (rid, pos), row in got.items():
        assert np.isfinite(row).all(), f"non-finite logits at {rid} position {pos}"
        d = row.astype(np.float64) - ref[rid][pos]
        d = d - d.mean()
        out[(rid, pos)] = float(np.sqrt((d * d).mean())) / scale
    return out


FP32_TOL = 2e-5


def assert_matches_plain(got, model_dir, requests, dtype, what=""):
    """float32: every row within FP32_TOL.  bfloat16: against what rounding the same values to
    bfloat16 costs the plain implementation itself.  Its root mean square row error is the yard:
    no row over six yards and at most one row in fifty over three, but for rows where the plain
    implementation's own rounding error is that large too (a few rows are far more sensitive than
    the rest; there a row may err by half as much again as the plain one)."""
    ref = plain_logits(model_dir, requests)
    errs = row_errors(got, ref)
    worst = max(errs, key=errs.get)
    if dtype == "float32":
        assert errs[worst] < FP32_TOL, (what, worst, errs[worst])
        return
    own = row_errors({k: plain_logits(model_dir, requests, torch.bfloat16)[k[0]][k[1]]
                      for k in got}, ref)
    yard = float(np.sqrt(np.mean(np.square(list(own.values())))))
    bad = [k for k, e in errs.items() if e > max(6 * yard, 1.5 * own[k])]
    over = [k for k, e in errs.items() if e > max(3 * yard, 1.5 * own[k])]
    assert not bad, (what, bad[:5], [errs[k] for k in bad[:5]], yard)
    assert len(over) <= max(1, len(errs) // 50), (what, len(over), len(errs), yard, over[:5])
