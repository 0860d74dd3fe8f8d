"""The Dukolorn decoder put together from parts.

The embedded rows pass an RMS norm; every layer is ``block.output_norm`` (the sublayers read the
stream itself, a norm sits on what they return) around one of three mixers: a scored softmax
attention beside a gated linear attention (``mixer.parallel``), a latent attention with a sliding
window, or the gated delta rule; a SiLU-gated dense feed-forward with biases, or none; a last
norm, a head of its own and a scale on the logits (folded into the last norm's weight).  Norm
weights are stored around zero.  Tensor names: ``embed``, ``embed.norm``, ``final.norm``,
``head`` and per layer ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``; no name ends in
``.weight``, biases end in ``.b``.
"""
from __future__ import annotations

import torch

from ..config.base import register_architecture
from ..config.dukolorn import ARCHITECTURE, DukolornConfig
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from .base import Model


def _need(value, what: str):
    if value is None:
        raise ValueError(f"config.json does not state {what}, and no tensor shapes were read "
                         "that could give it")
    return value


def _mixer(kind: str, m: dict, p: str, width: int, eps: float, dtype):
    if kind == "parallel":
        lt, rt = m["left"], m["right"]
        left = make_part(
            "mixer", "scored_attention", prefix=p + "left.", width=width, num_heads=lt["heads"],
            num_kv_heads=lt["kv_heads"], dim=lt["dim"], vdim=lt["vdim"], scale=lt["scale"],
            dtype=dtype, norm_eps=eps, whole_qk_norm=True, softcap=lt["softcap"],
            bias_buckets=_need(lt["buckets"], "mixer.left.buckets"), bias_far=lt["bias_max"],
            sink=True, temp_coef=lt["temp_coef"], temp_every=lt["temp_every"], weight_suffix="")
        right = make_part(
            "mixer", "gated_linear_attention", prefix=p + "right.", width=width,
            num_heads=rt["heads"], dim=rt["dim"], vdim=rt["vdim"], tau=rt["tau"],
            decay_rank=_need(rt["decay_rank"], "mixer.right.decay_rank"), norm_eps=eps,
            dtype=dtype, weight_suffix="", bias_suffix=".b")
        return make_part("mixer", "parallel", left=left, right=right,
                         left_scale=m["left_scale"], right_scale=m["right_scale"])
    if kind == "latent_attention":
        position = None
        if m["rot_dims"]:
            position = make_part("position_encoding", "rotary", head_dim=m["rot_dim"],
                                 theta=m["rot_base"], rot_dim=m["rot_dims"],
                                 pairing="interleaved")
        return make_part(
            "mixer", "latent_attention", prefix=p, width=width, num_heads=m["heads"],
            dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"], rank=m["kv_rank"],
            scale=m["scale"], norm_eps=eps, dtype=dtype, position=position, window=m["window"],
            sink=True, weight_suffix="")
    return make_part(
        "mixer", "gated_delta_rule", prefix=p, width=width, num_heads=m["heads"],
        num_qk_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], taps=m["conv"],
        decay_rank=_need(m["decay_rank"], "mixer.decay_rank"),
        gate_rank=_need(m["gate_rank"], "mixer.gate_rank"), norm_eps=eps, dtype=dtype,
        weight_suffix="")


def build_dukolorn(config: DukolornConfig, dtype: torch.dtype) -> Model:
    width, eps = config.width, config.norm_eps

    def norm(name, scale=1.0):
        return make_part("norm", "rmsnorm", name=name, width=width, eps=eps, dtype=dtype,
                         suffix="", weight_offset=1.0, weight_scale=scale)

    layers, unused = [], []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        mixer = _mixer(layer.type, layer.mixer, p + "mix.", width, eps, dtype)
        feed_forward = ffn_norm = None
        if layer.mlp is not None:
            feed_forward = make_part("feed_forward", "swiglu", prefix=p + "mlp.", width=width,
                                     hidden=layer.mlp["ff"], dtype=dtype, activation="silu",
                                     names={"gate": "gate", "up": "up", "down": "down"},
                                     weight_suffix="", bias=True, bias_suffix=".b")
            ffn_norm = norm(p + "norm2")
        else:
            unused.append(p + "norm2")
        layers.append(make_part("block", "output_norm", mixer=mixer, mixer_norm=norm(p + "norm1"),
                                feed_forward=feed_forward, ffn_norm=ffn_norm))
    embedding = TokenEmbedding("embed", config.vocab_size, width, suffix="")
    head = OutputHead("head", config.vocab_size, width, tied_to=None, suffix="")
    model = Model(config, dtype, embedding, layers, norm("final.norm", config.logit_scale), head,
                  embedding_norm=norm("embed.norm"))
    model.unused_tensor_names = unused
    return model


register_architecture(ARCHITECTURE, DukolornConfig, build_dukolorn)
