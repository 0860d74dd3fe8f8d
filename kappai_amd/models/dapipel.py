"""The Dapipel decoder put together from parts.

Embedding times a scale plus a learned position row; every layer is the pre-norm arrangement
with a short convolution in front of each sublayer (``block.conv_input``) around a windowed
differential attention or a minGRU and a tanh-GELU gated dense feed-forward, a mixture of
experts, or nothing; grouped RMS norms; the embedding table is the head.  Tensor names:
``embed``, ``pos``, ``final.norm`` and per layer ``l<i>.norm1|norm2|canon1|canon2``,
``l<i>.mix.*``, ``l<i>.mlp.*``; no name ends in ``.weight``.
"""
from __future__ import annotations

import torch

from ..config.base import register_architecture
from ..config.dapipel import ARCHITECTURE, DapipelConfig
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.input_conv import ShortInputConv
from .base import Model


def build_dapipel(config: DapipelConfig, dtype: torch.dtype) -> Model:
    width = config.width

    def norm(name):
        return make_part("norm", "group_rmsnorm", name=name, width=width, eps=config.norm_eps,
                         groups=config.norm_groups, dtype=dtype, suffix="")

    layers, unused = [], []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        m = layer.mixer
        if layer.type == "attention":
            mixer = make_part("mixer", "differential_attention", prefix=p + "mix.", width=width,
                              num_heads=m["heads"], num_kv_heads=m["kv_heads"], dim=m["dim"],
                              vdim=m["vdim"], scale=m["scale"], diff=m["diff"],
                              norm_eps=config.norm_eps, window=m["window"], dtype=dtype,
                              weight_suffix="")
        else:
            mixer = make_part("mixer", "mingru", prefix=p + "mix.", width=width, inner=m["width"],
                              dtype=dtype, weight_suffix="", bias_suffix=".b")
        feed_forward = None
        if layer.mlp is not None and layer.mlp["kind"] == "dense":
            feed_forward = make_part("feed_forward", "swiglu", prefix=p + "mlp.", width=width,
                                     hidden=layer.mlp["ff"], dtype=dtype, activation="gelu_tanh",
                                     names={"gate": "gate", "up": "up", "down": "down"},
                                     weight_suffix="")
        elif layer.mlp is not None:
            feed_forward = make_part("feed_forward", "moe", prefix=p + "mlp.", width=width,
                                     hidden=layer.mlp["ff"], experts=layer.mlp["experts"],
                                     top=layer.mlp["top"], dtype=dtype, weight_suffix="")
        has_ff = feed_forward is not None
        if not has_ff:
            # a layer without feed-forward reads no second norm and no second convolution; a
            # file that holds them all the same is no error
            unused += [p + "norm2", p + "canon2"]
        layers.append(make_part(
            "block", "conv_input",
            mixer_norm=norm(p + "norm1"),
            mixer_conv=ShortInputConv(p + "canon1", width, config.canon_taps, dtype),
            mixer=mixer,
            ffn_norm=norm(p + "norm2") if has_ff else None,
            ffn_conv=ShortInputConv(p + "canon2", width, config.canon_taps, dtype) if has_ff
            else None,
            feed_forward=feed_forward))
    embedding = TokenEmbedding("embed", config.vocab_size, width, suffix="")
    positions = make_part("position_encoding", "learned", name="pos",
                          max_positions=config.max_positions, width=width,
                          input_scale=config.embedding_scale)
    head = OutputHead("embed", config.vocab_size, width, tied_to=embedding, suffix="")
    model = Model(config, dtype, embedding, layers, norm("final.norm"), head,
                  embedding_position=positions)
    model.unused_tensor_names = unused
    return model


register_architecture(ARCHITECTURE, DapipelConfig, build_dapipel)
