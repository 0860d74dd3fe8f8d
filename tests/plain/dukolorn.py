"""A plain, slow statement of the Dukolorn decoder in float64 torch on the CPU: one function per
mechanism, whole sequences, no cache and no state.  It shares nothing with the product path; the
GPU tests hold the framework to it.

The model: an embedded row passes an RMS norm; every layer is ``x += n1(mixer(x))`` and, where the
layer has a feed-forward, ``x += n2(ff(x))``: the sublayers read the stream itself and the norm
sits on what they return.  Norm weights are stored around zero (``1 + w``).  Three mixers:

* ``parallel``: a softmax attention (norm over the whole query and key projection, a query
  temperature that grows with the position, capped scores, a learned bias by bucketed distance,
  a sink in the denominator) beside a gated linear attention with a decay per key channel; their
  outputs are added with two weights;
* ``latent_attention``: keys and values come from one low-rank latent per token, a rotated key
  part is shared by the heads, a sliding window, a sink;
* ``channel_delta``: the gated delta rule with short convolutions on q, k, v and a decay per head
  and key channel.

``rounding=torch.bfloat16`` rounds where a bfloat16 run rounds (inputs and outputs of matrix
products), which gives the yardstick for the error that rounding alone costs.
"""
from __future__ import annotations

import math
from typing import Dict

import torch

F64 = torch.float64


def _r(x: torch.Tensor, rounding) -> torch.Tensor:
    return x if rounding is None else x.to(rounding).to(F64)


def matmul(x, w, rounding=None, bias=None):
    """``x [T, in] -> [T, out]`` with ``w [out, in]``; inputs and the result rounded when a
    rounding is set."""
    y = _r(x, rounding) @ w.to(F64).T
    if bias is not None:
        y = y + bias.to(F64)
    return _r(y, rounding)


def rms(x, eps: float):
    return torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps: float):
    return x / rms(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps: float):
    return x / rms(x, eps) * w.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def distance_bucket(n: int, rows: int, bias_max: float) -> int:
    """Distances below half the table have a row each; larger ones share rows on a logarithmic
    scale that reaches the last row at ``bias_max``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(bias_max / half)
                                               * (rows - half))))


def sink_softmax(scores, sink):
    """Softmax over the last axis whose denominator also holds ``exp(sink)``; masked places are
    ``-inf``."""
    m = torch.maximum(scores.max(dim=-1, keepdim=True).values, sink)
    e = torch.exp(scores - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - m))


def biased_attention(h, t, p, m: dict, eps: float, rounding=None):
    """The softmax half of the parallel mixer."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = matmul(h, t[p + "q"], rounding)
    k = matmul(h, t[p + "k"], rounding)
    v = matmul(h, t[p + "v"], rounding).reshape(T, G, dv)
    q = norm_plain(q, t[p + "q.norm"], eps)                # over all heads' rows at once
    k = norm_plain(k, t[p + "k.norm"], eps)
    pos = torch.arange(T, dtype=F64)
    temp = 1.0 + m["q_temp"]["coef"] * torch.log(torch.floor((pos + 1) / m["q_temp"]["every"]) + 1)
    q = _r((q * temp[:, None]).reshape(T, H, d), rounding)
    k = _r(k.reshape(T, G, d), rounding)
    rel = t[p + "rel"].to(F64)
    B = rel.shape[0]
    bucket = torch.tensor([[distance_bucket(i - j, B, m["bias_max"]) if j <= i else 0
                            for j in range(T)] for i in range(T)])
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        cap = m.get("softcap")
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s + rel[bucket, hd]
        s = s.masked_fill(~causal, float("-inf"))
        out[:, hd] = sink_softmax(s, t[p + "sink"].to(F64)[hd]) @ v[:, g]
    return matmul(out.reshape(T, H * dv), t[p + "o"], rounding)


def gated_linear_attention(h, t, p, m: dict, eps: float, rounding=None):
    """The recurrent half of the parallel mixer: ``S <- diag(a) S + k v^T``, read out with q."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = matmul(h, t[p + "q"], rounding).reshape(T, H, d) * d ** -0.5
    k = matmul(h, t[p + "k"], rounding).reshape(T, H, d)
    v = matmul(h, t[p + "v"], rounding).reshape(T, H, dv)
    z = matmul(matmul(h, t[p + "a1"], rounding), t[p + "a2"], rounding, bias=t[p + "a2.b"])
    a = torch.exp(torch.nn.functional.logsigmoid(z) / m["tau"]).reshape(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        S = a[i][:, :, None] * S + k[i][:, :, None] * v[i][:, None, :]
        o[i] = torch.einsum("hdv,hd->hv", S, q[i])
    o = norm_plain(o, t[p + "norm"], eps).reshape(T, H * dv)
    o = o * silu(matmul(h, t[p + "g"], rounding))
    return matmul(o, t[p + "o"], rounding)


def parallel_mixer(h, t, p, m: dict, eps: float, rounding=None):
    return (m["left_scale"] * biased_attention(h, t, p + "left.", m["left"], eps, rounding)
            + m["right_scale"] * gated_linear_attention(h, t, p + "right.", m["right"], eps,
                                                        rounding))


def rotate_pairs(x, pos, dims: int, base: float):
    """Neighbouring pairs (2i, 2i+1) of the first ``dims`` entries of the last axis turn by
    ``pos * base^(-2i/dims)``; ``x`` is [T, ..., n]."""
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos.to(F64)[:, None] * base ** (-2.0 * i / dims)
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention(h, t, p, m: dict, eps: float, rounding=None):
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    window = m["mask"]["size"] if m.get("mask") else T + 1
    pos = torch.arange(T)
    q = matmul(h, t[p + "q"], rounding).reshape(T, H, d + dr)
    dkv = matmul(h, t[p + "dkv"], rounding)
    c = _r(norm_plain(dkv[:, :r], t[p + "dkv.norm"], eps), rounding)
    k_rot = rotate_pairs(dkv[:, r:], pos, m["rot"]["dims"], m["rot"]["base"])
    q_rot = rotate_pairs(q[:, :, d:], pos, m["rot"]["dims"], m["rot"]["base"])
    k_un = matmul(c, t[p + "uk"], rounding).reshape(T, H, d)
    v = matmul(c, t[p + "uv"], rounding).reshape(T, H, dv)
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & (i - j < window)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :d] @ k_un[:, hd].T + _r(q_rot[:, hd], rounding) @ _r(k_rot, rounding).T)
        s = (s * m["scale"]).masked_fill(~seen, float("-inf"))
        out[:, hd] = sink_softmax(s, t[p + "sink"].to(F64)[hd]) @ v[:, hd]
    return matmul(out.reshape(T, H * dv), t[p + "o"], rounding)


def conv_silu(x, w, rounding=None):
    """Causal per-channel convolution (the last column of ``w`` meets the current token, zeros
    before the start), then SiLU."""
    T, C = x.shape
    n = w.shape[1]
    w = w.to(F64)
    y = torch.zeros_like(x)
    for j in range(n):
        back = n - 1 - j
        if back < T:
            y[back:] += x[:T - back] * w[:, j]
    return _r(silu(y), rounding)


def channel_delta(h, t, p, m: dict, eps: float, rounding=None):
    """The gated delta rule: ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = conv_silu(matmul(h, t[p + "q"], rounding), t[p + "q.conv"], rounding).reshape(T, G, d)
    k = conv_silu(matmul(h, t[p + "k"], rounding), t[p + "k.conv"], rounding).reshape(T, G, d)
    v = conv_silu(matmul(h, t[p + "v"], rounding), t[p + "v.conv"], rounding).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(matmul(h, t[p + "b"], rounding))
    z = matmul(matmul(h, t[p + "a1"], rounding), t[p + "a2"], rounding) + t[p + "dt_bias"].to(F64)
    rate = torch.exp(t[p + "A_log"].to(F64))
    g = torch.exp(-rate[None, :, None] * softplus(z).reshape(T, H, d))
    gate = torch.sigmoid(matmul(matmul(h, t[p + "g1"], rounding), t[p + "g2"], rounding))
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    per = H // G
    for i in range(T):
        ki = k[i].repeat_interleave(per, dim=0)
        qi = q[i].repeat_interleave(per, dim=0)
        S = g[i][:, :, None] * S
        u = beta[i][:, None] * (v[i] - torch.einsum("hdv,hd->hv", S, ki))
        S = S + ki[:, :, None] * u[:, None, :]
        o[i] = torch.einsum("hdv,hd->hv", S, qi)
    o = (norm_plain(o, t[p + "norm"], eps)).reshape(T, H * dv) * gate
    return matmul(o, t[p + "o"], rounding)


def dense_feed_forward(h, t, p, rounding=None):
    gate = matmul(h, t[p + "gate"], rounding, bias=t[p + "gate.b"])
    up = matmul(h, t[p + "up"], rounding, bias=t[p + "up.b"])
    return matmul(silu(gate) * up, t[p + "down"], rounding, bias=t[p + "down.b"])


MIXERS = {"parallel": parallel_mixer, "latent_attention": latent_attention,
          "channel_delta": channel_delta}


def forward(config: dict, t: Dict[str, torch.Tensor], tokens, rounding=None, streams=None):
    """Logits [T, vocab] of one whole sequence.  ``streams``: a list that receives the residual
    stream after every layer."""
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = norm_one_plus(t["embed"].to(F64)[ids], t["embed.norm"], eps)
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](x, t, p + "mix.", layer["mixer"], eps, rounding)
        x = x + norm_one_plus(y, t[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = dense_feed_forward(x, t, p + "mlp.", rounding)
            x = x + norm_one_plus(y, t[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    x = norm_one_plus(x, t["final.norm"], eps)
    return matmul(x, t["head"], rounding) * config["logit_scale"]
