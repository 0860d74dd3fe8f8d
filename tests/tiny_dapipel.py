"""Tiny Dapipel configurations that differ in every size and option, and helpers that write them
as model folders with random weights."""
from __future__ import annotations

import copy

import numpy as np
import torch

from kappai_amd.config import config_from_dict
from kappai_amd.weights import write_random_model


def attention(heads, kv_heads, dim, vdim, window, scale, diff, mlp):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "diff": diff}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def mingru(width, mlp):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(vocab, width, positions, scale, eps, groups, taps, layers):
    return {"architecture": "Dapipel", "vocab": vocab, "width": width, "max_positions": positions,
            "embedding": {"scale": scale}, "norm": {"eps": eps, "groups": groups},
            "canon": {"taps": taps}, "layers": layers}


# a recurrent layer first, two query heads a kv head, values narrower than the maps' keys in one
# layer and wider in the other, a layer without feed-forward, two of five experts a token
TINY_P = config(301, 96, 400, 1.7, 1e-5, 3, 3, [
    mingru(80, moe(40, 5, 2)),
    attention(4, 2, 16, 24, 20, 0.3, 0.4, dense(112)),
    attention(3, 3, 24, 16, None, 0.2, 0.25, None),
    mingru(96, dense(72)),
])
INIT_P = dict(seed=11, std=0.08, norm_jitter=0.1)

# one group (the plain RMS norm), one tap (the convolution keeps no history), six heads on one kv
# head, a window of one key (a position sees itself only) beside one of 33, one expert a token
TINY_Q = config(200, 64, 300, 0.75, 1e-6, 1, 1, [
    attention(6, 1, 8, 8, 1, 0.35, 0.5, moe(24, 3, 1)),
    mingru(48, None),
    attention(2, 2, 24, 48, 33, 0.18, 0.7, dense(96)),
])
INIT_Q = dict(seed=12, std=0.1, norm_jitter=0.05)

# eight groups, five taps, only recurrent layers (no paged cache at all), all experts chosen
TINY_R = config(128, 128, 256, 1.0, 1e-4, 8, 5, [
    mingru(160, dense(64)),
    mingru(64, moe(48, 4, 4)),
])
INIT_R = dict(seed=13, std=0.07, norm_jitter=0.1)

# attention only, heads of 80 (values) on maps of 40, a window that is no multiple of a page
TINY_S = config(150, 56, 512, 2.0, 1e-5, 2, 2, [
    attention(2, 1, 40, 80, 37, 0.16, 0.65, dense(48)),
    attention(1, 1, 16, 16, 50, 0.25, 0.3, moe(32, 5, 2)),
])
INIT_S = dict(seed=14, std=0.1, norm_jitter=0.1)

# no experts (no router whose choice rounding could change): attention with two windows around a
# recurrent layer, five groups
TINY_T = config(180, 80, 512, 1.3, 1e-5, 5, 3, [
    attention(4, 2, 16, 32, 19, 0.25, 0.35, dense(64)),
    mingru(64, dense(48)),
    attention(2, 2, 24, 16, 41, 0.2, 0.55, None),
])
INIT_T = dict(seed=15, std=0.1, norm_jitter=0.1)

TINY = {"T": (TINY_T, INIT_T), "P": (TINY_P, INIT_P), "Q": (TINY_Q, INIT_Q), "R": (TINY_R, INIT_R),
        "S": (TINY_S, INIT_S)}


def write_tiny(name: str, folder, **overrides):
    cfg, init = TINY[name]
    return write_random_model(folder, config_from_dict(copy.deepcopy(cfg)), **{**init, **overrides})


_plain_cache = {}


def plain_logits(model_dir, requests, rounding=None):
    """{id: float64 numpy [len, vocab]} from the plain implementation (cached per folder)."""
    import json

    from plain import dapipel as plain
    key = (str(model_dir), json.dumps(requests, sort_keys=True), str(rounding))
    if key not in _plain_cache:
        cfg, t = plain.read_model_dir(model_dir)
        _plain_cache[key] = {rid: plain.forward(cfg, t, toks, rounding=rounding).numpy()
                             for rid, toks in requests.items()}
    return _plain_cache[key]


CLOSE_CALL = 0.01       # a router's margin below this may go the other way in bfloat16


def first_close_calls(model_dir, requests):
    """{id: the first position at which some router of the model makes a close call} (the
    request's length when none does).  From there on a bfloat16 run may have chosen another
    expert, which the recurrent state and the keys carry to every later position."""
    from plain import dapipel as plain
    cfg, t = plain.read_model_dir(model_dir)
    out = {}
    for rid, toks in requests.items():
        margins = []
        plain.forward(cfg, t, toks, margins=margins)
        first = len(toks)
        for m in margins:
            close = (m < CLOSE_CALL).nonzero().flatten()
            if close.numel():
                first = min(first, int(close[0]))
        out[rid] = first
    return out


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


def assert_matches_plain(got, model_dir, requests, dtype, what="", min_strict=1 / 6):
    """float32: every row within FP32_TOL.  bfloat16: against what rounding the same values to
    bfloat16 costs the plain implementation itself: no row over six times its root mean square
    row error and at most one row in fifty over three times, for the rows before a request's
    first close call of a router (at least ``min_strict`` of all rows must be such); the rows
    behind it must stay finite and within twice the logits' own size (another expert may have been
    chosen, rightly, and where one expert is chosen its whole output changes)."""
    ref = plain_logits(model_dir, requests)
    errs = row_errors(got, ref)
    worst = max(errs, key=errs.get)
    if dtype == "float32":
        assert errs[worst] < FP32_TOL, (what, worst, errs[worst])
        return
    own = row_errors({k: plain_logits(model_dir, requests, torch.bfloat16)[k[0]][k[1]]
                      for k in got}, ref)
    yard = float(np.sqrt(np.mean(np.square(list(own.values())))))
    close = first_close_calls(model_dir, requests)
    strict = {k: e for k, e in errs.items() if k[1] < close[k[0]]}
    assert len(strict) >= len(errs) * min_strict, (what, "too few rows before a close call",
                                                   len(strict))
    worst = max(strict, key=strict.get)
    over = [k for k, e in strict.items() if e > 3 * yard]
    assert strict[worst] < 6 * yard, (what, worst, strict[worst], yard)
    assert len(over) <= max(1, len(strict) // 50), (what, len(over), len(strict), yard, over[:5])
    assert max(errs.values()) < 2.0, (what, max(errs, key=errs.get), max(errs.values()))
