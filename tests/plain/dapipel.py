"""A plain, slow statement of the Dapipel decoder in float64 torch on the CPU: one function per
mechanism, whole sequences, no cache and no state.  It shares nothing with the product path; the
GPU tests hold the framework to it.

The model: token embedding times a scale plus a learned position row; layers of
``x += mixer(canon(norm(x))); x += ff(canon(norm(x)))`` where ``norm`` is an RMS norm in equal
groups, ``canon`` adds a short causal per-channel convolution of its input to it, the mixer is a
windowed differential attention or a minGRU, and the feed-forward is a gated dense layer (tanh
GELU) or a top-k mixture of SiLU-gated experts; a last norm and the embedding table as the head.

``rounding=torch.bfloat16`` rounds where a bfloat16 run rounds (matrix inputs and outputs), which
gives the yardstick for the error that rounding alone costs.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def _r(x: torch.Tensor, rounding) -> torch.Tensor:
    return x if rounding is None else x.to(rounding).to(F64)


def matmul(x, w, rounding=None):
    """``x [T, in] -> [T, out]`` with ``w [out, in]``; inputs rounded when a rounding is set."""
    return _r(x, rounding) @ _r(w.to(F64), rounding).T


def group_rms_norm(x, weight, groups: int, eps: float):
    T, D = x.shape
    parts = x.reshape(T, groups, D // groups)
    parts = parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(T, D) * weight.to(F64)


def canon(h, taps_w):
    """``h + conv(h)``: ``conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j]`` with zeros before the
    sequence starts."""
    T, D = h.shape
    n = taps_w.shape[1]
    w = taps_w.to(F64)
    out = h.clone()
    for j in range(n):
        back = n - 1 - j
        if back >= T:
            continue
        shifted = torch.zeros_like(h)
        shifted[back:] = h[:T - back]
        out = out + shifted * w[:, j]
    return out


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def diff_lambda(t: Dict[str, torch.Tensor], p: str, diff: float) -> float:
    a = float((t[p + "lq1"].to(F64) * t[p + "lk1"].to(F64)).sum())
    b = float((t[p + "lq2"].to(F64) * t[p + "lk2"].to(F64)).sum())
    return math.exp(a) - math.exp(b) + diff


def differential_attention(h, t, p, m: dict, eps: float, rounding=None):
    """Two softmax maps per head over the same values, ``o = a1 - lambda a2``, each head's ``o``
    divided by its root mean square and scaled by ``1 - diff``; keys further back than the window
    are not seen."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    window = m["mask"]["size"] if m.get("mask") else T + 1
    scale, diff = m["scale"], m["diff"]
    q = _r(matmul(h, t[p + "q"], rounding), rounding).reshape(T, H, 2, d)
    k = _r(matmul(h, t[p + "k"], rounding), rounding).reshape(T, G, 2, d)
    v = _r(matmul(h, t[p + "v"], rounding), rounding).reshape(T, G, dv)
    lam = diff_lambda(t, p, diff)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) & (i - j < window)
    out = torch.zeros(T, H, dv, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        maps = []
        for which in range(2):
            s = (q[:, head, which] @ k[:, g, which].T) * scale
            s = s.masked_fill(~seen, float("-inf"))
            maps.append(_r(torch.softmax(s, dim=-1) @ v[:, g], rounding))
        o = maps[0] - lam * maps[1]
        o = o / torch.sqrt((o * o).mean(dim=-1, keepdim=True) + eps)
        out[:, head] = o * (1.0 - diff)
    return matmul(out.reshape(T, H * dv), t[p + "o"], rounding)


def mingru_recurrence(pz, pu, pg, state: Optional[torch.Tensor] = None):
    """From the three projections (biases added): the gated states times the output gate
    [T, W], and the last state."""
    z = torch.sigmoid(pz)
    cand = torch.where(pu >= 0, pu + 0.5, torch.sigmoid(pu))
    gate = silu(pg)
    S = torch.zeros(z.shape[1], dtype=F64) if state is None else state.clone()
    ys = []
    for step in range(pz.shape[0]):
        S = (1.0 - z[step]) * S + z[step] * cand[step]
        ys.append(S * gate[step])
    return torch.stack(ys), S


def mingru(h, t, p, rounding=None):
    """``S_t = (1 - z_t) S_(t-1) + z_t c_t`` from a zero state; ``c = u + 1/2`` where ``u >= 0``,
    ``sigmoid(u)`` below; the output is ``W_o (S_t * silu(W_g h))``."""
    ys, _ = mingru_recurrence(matmul(h, t[p + "z"], rounding) + t[p + "z.b"].to(F64),
                              matmul(h, t[p + "x"], rounding) + t[p + "x.b"].to(F64),
                              matmul(h, t[p + "g"], rounding))
    return matmul(ys, t[p + "o"], rounding)


def dense_ff(h, t, p, rounding=None):
    a = gelu_tanh(matmul(h, t[p + "gate"], rounding)) * matmul(h, t[p + "up"], rounding)
    return matmul(a, t[p + "down"], rounding)


def moe_ff(h, t, p, experts: int, top: int, rounding=None, margins: Optional[list] = None):
    """Router logits over all experts, the ``top`` largest chosen, their weights the softmax over
    the chosen logits alone; every expert is a SiLU-gated feed-forward.  ``margins`` gets, per
    row, how far the last chosen logit lies above the first one left out, relative to the row's
    largest |logit| (a small margin is a close call that rounding may decide otherwise)."""
    logits = _r(h, rounding) @ t[p + "router"].to(F64).T
    best, chosen = torch.topk(logits, top, dim=-1)
    if margins is not None and top < experts:
        ranked = torch.sort(logits, dim=-1, descending=True).values
        margins.append((ranked[:, top - 1] - ranked[:, top]) / logits.abs().max(dim=-1).values)
    weights = torch.softmax(best, dim=-1)
    out = torch.zeros(h.shape[0], t[p + "e0.down"].shape[0], dtype=F64)
    for e in range(experts):
        for slot in range(top):
            rows = (chosen[:, slot] == e).nonzero().flatten()
            if rows.numel() == 0:
                continue
            x = h[rows]
            a = silu(matmul(x, t[p + f"e{e}.gate"], rounding)) * matmul(x, t[p + f"e{e}.up"],
                                                                        rounding)
            out[rows] += weights[rows, slot, None] * matmul(a, t[p + f"e{e}.down"], rounding)
    return out


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], rounding=None,
            layers_out: Optional[list] = None, margins: Optional[list] = None) -> torch.Tensor:
    """float64 logits [len(tokens), vocab] of one sequence from position 0.  ``layers_out``: a
    list that gets the residual stream after every layer; ``margins``: one that gets every
    router's margins (see ``moe_ff``)."""
    t = tensors
    eps, groups = config["norm"]["eps"], config["norm"]["groups"]
    ids = torch.tensor(tokens, dtype=torch.long)
    T = ids.shape[0]
    x = t["embed"].to(F64)[ids] * config["embedding"]["scale"] + t["pos"].to(F64)[:T]
    for li, layer in enumerate(config["layers"]):
        p = f"l{li}."
        h = canon(group_rms_norm(x, t[p + "norm1"], groups, eps), t[p + "canon1"])
        if layer["type"] == "attention":
            x = x + differential_attention(h, t, p + "mix.", layer["mixer"], eps, rounding)
        elif layer["type"] == "mingru":
            x = x + mingru(h, t, p + "mix.", rounding)
        else:
            raise ValueError(f"layer {li}: unknown mixer {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = canon(group_rms_norm(x, t[p + "norm2"], groups, eps), t[p + "canon2"])
            if mlp["kind"] == "dense":
                x = x + dense_ff(h, t, p + "mlp.", rounding)
            elif mlp["kind"] == "moe":
                x = x + moe_ff(h, t, p + "mlp.", mlp["router"]["experts"], mlp["router"]["top"],
                               rounding, margins)
            else:
                raise ValueError(f"layer {li}: unknown feed-forward {mlp['kind']!r}")
        if layers_out is not None:
            layers_out.append(x.clone())
    x = group_rms_norm(x, t["final.norm"], groups, eps)
    return matmul(x, t["embed"], rounding)


def read_model_dir(model_dir):
    """(config.json as a dictionary, {tensor name: torch tensor}) of a model folder."""
    import json
    from pathlib import Path

    from kappai_amd.weights.safetensors_io import SafetensorsFile
    cfg = json.loads((Path(model_dir) / "config.json").read_text())
    f = SafetensorsFile(Path(model_dir) / "model.safetensors")
    try:
        return cfg, {n: f.read(n) for n in f.names()}
    finally:
        f.close()
