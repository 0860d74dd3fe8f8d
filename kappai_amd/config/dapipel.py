"""Configuration of the Dapipel decoder: a list of layers, each with its mixer (a windowed
differential attention or a minGRU) and its feed-forward (dense, a mixture of experts, or none),
grouped RMS norms, a short convolution in front of every sublayer, scaled embeddings with learned
positions and the embedding table as the output head.

config.json names the design under ``architecture`` and nests its keys::

    {"architecture": "Dapipel", "vocab": V, "width": D, "max_positions": P,
     "embedding": {"scale": s}, "norm": {"eps": e, "groups": g}, "canon": {"taps": n},
     "layers": [{"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale",
                 "diff", "mask": {"size"}}, "mlp": {"kind": "dense", "ff": F}},
                {"type": "mingru", "mixer": {"width": W},
                 "mlp": {"kind": "moe", "expert": {"ff": F}, "router": {"experts", "top"}}},
                {"type": ..., "mixer": ..., "mlp": null}]}
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, KeyReader, ModelConfig

ARCHITECTURE = "Dapipel"

MIXER_TYPES = ("attention", "mingru")
MLP_KINDS = ("dense", "moe")


@dataclass
class DapipelLayer:
    type: str                                   # "attention" | "mingru"
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]               # None: the layer has no feed-forward


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.raw.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: required key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _layer(raw: Any, i: int) -> DapipelLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(raw, where)
    kind = raw.get("type")
    if kind not in MIXER_TYPES:
        raise ConfigError(f"{where}: type = {kind!r}; known: {', '.join(MIXER_TYPES)}")
    m = _sub(r, "mixer")
    if kind == "attention":
        mask = m.raw.get("mask")
        window = None
        if mask is not None:
            window = _sub(m, "mask").int("size")
            if window < 1:
                raise ConfigError(f"{where}: mixer.mask.size must be at least 1")
        mixer = {"heads": m.int("heads"), "kv_heads": m.int("kv_heads"), "dim": m.int("dim"),
                 "vdim": m.int("vdim"), "scale": m.float("scale"), "diff": m.float("diff"),
                 "window": window}
        if mixer["heads"] < 1 or mixer["kv_heads"] < 1 or mixer["heads"] % mixer["kv_heads"]:
            raise ConfigError(f"{where}: {mixer['heads']} heads cannot be shared out over "
                              f"{mixer['kv_heads']} kv heads")
        if mixer["dim"] < 1 or mixer["vdim"] < 1:
            raise ConfigError(f"{where}: mixer.dim and mixer.vdim must be positive")
    else:
        mixer = {"width": m.int("width")}
        if mixer["width"] < 1:
            raise ConfigError(f"{where}: mixer.width must be positive")
    mlp = None
    if raw.get("mlp") is not None:
        f = _sub(r, "mlp")
        mk = f.raw.get("kind")
        if mk not in MLP_KINDS:
            raise ConfigError(f"{where}: mlp.kind = {mk!r}; known: {', '.join(MLP_KINDS)}")
        if mk == "dense":
            mlp = {"kind": "dense", "ff": f.int("ff")}
        else:
            router = _sub(f, "router")
            mlp = {"kind": "moe", "ff": _sub(f, "expert").int("ff"),
                   "experts": router.int("experts"), "top": router.int("top")}
            if not 1 <= mlp["top"] <= mlp["experts"]:
                raise ConfigError(f"{where}: mlp.router.top ({mlp['top']}) must lie between 1 and "
                                  f"mlp.router.experts ({mlp['experts']})")
        if mlp["ff"] < 1:
            raise ConfigError(f"{where}: the feed-forward width must be positive")
    return DapipelLayer(kind, mixer, mlp)


@dataclass
class DapipelConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    max_positions: int = 0
    embedding_scale: float = 1.0
    norm_eps: float = 0.0
    norm_groups: int = 1
    canon_taps: int = 1
    layers: List[DapipelLayer] = field(default_factory=list)
    max_position_embeddings: int = 0
    eos_token_id: Optional[Union[int, List[int]]] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "DapipelConfig":
        r = KeyReader(raw)
        layers = r.list("layers")
        norm = _sub(r, "norm")
        cfg = cls(
            architecture=ARCHITECTURE,
            vocab_size=r.int("vocab"),
            width=r.int("width"),
            max_positions=r.int("max_positions"),
            embedding_scale=_sub(r, "embedding").float("scale"),
            norm_eps=norm.float("eps"),
            norm_groups=norm.int("groups"),
            canon_taps=_sub(r, "canon").int("taps"),
            layers=[_layer(x, i) for i, x in enumerate(layers)],
            eos_token_id=r.int_or_ints("eos_token_id", None),
            raw=copy.deepcopy(raw),
        )
        cfg.max_position_embeddings = cfg.max_positions
        cfg.validate()
        return cfg

    def validate(self) -> None:
        def need(cond, msg):
            if not cond:
                raise ConfigError("config.json: " + msg)

        need(self.vocab_size >= 1, "vocab must be positive")
        need(self.width >= 1, "width must be positive")
        need(self.max_positions >= 1, "max_positions must be positive")
        need(self.layers, "layers must name at least one layer")
        need(self.norm_eps > 0.0, "norm.eps must be positive")
        need(self.norm_groups >= 1 and self.width % self.norm_groups == 0,
             f"norm.groups ({self.norm_groups}) must divide width ({self.width})")
        need(self.canon_taps >= 1, "canon.taps must be at least 1")

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
