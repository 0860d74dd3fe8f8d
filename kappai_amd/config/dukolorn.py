"""Configuration of the Dukolorn decoder: a list of layers, each with one of three mixers and an
optional dense feed-forward; a norm sits on every sublayer's output and on the embedded rows.

config.json names the design under ``architecture`` and nests its keys::

    {"architecture": "Dukolorn", "vocab": V, "width": D, "logit_scale": s, "norm": {"eps": e},
     "layers": [
       {"type": "parallel",
        "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "bias_max",
                           "q_temp": {"coef", "every"}},
                  "right": {"heads", "dim", "vdim", "tau"},
                  "left_scale": a, "right_scale": b},
        "mlp": {"kind": "dense", "ff": F}},
       {"type": "latent_attention",
        "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale",
                  "rot": {"base", "dims"}, "mask": {"size"}}, "mlp": ...},
       {"type": "channel_delta",
        "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": null}]}

The ranks of the low-rank maps (``decay_rank``, ``gate_rank``) and the rows of the distance-bias
table (``left.buckets``) may be left out of the file: the tensors' shapes then give them
(``adopt_tensor_shapes``); a file for the random-weights mode states them.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, KeyReader, ModelConfig

ARCHITECTURE = "Dukolorn"

MIXER_TYPES = ("parallel", "latent_attention", "channel_delta")


@dataclass
class DukolornLayer:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]               # None: the layer has no feed-forward


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.raw.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: required key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _positive(where: str, **values) -> None:
    for name, v in values.items():
        if v < 1:
            raise ConfigError(f"{where}: mixer.{name} must be positive, got {v}")


def _parallel(m: KeyReader, where: str) -> Dict[str, Any]:
    left, right = _sub(m, "left"), _sub(m, "right")
    temp = left.raw.get("q_temp")
    lt = {"heads": left.int("heads"), "kv_heads": left.int("kv_heads"), "dim": left.int("dim"),
          "vdim": left.int("vdim"), "scale": left.float("scale"),
          "softcap": left.float("softcap", 0.0) or 0.0, "bias_max": left.float("bias_max"),
          "temp_coef": 0.0, "temp_every": 1, "buckets": left.int("buckets", None)}
    if temp is not None:
        t = _sub(left, "q_temp")
        lt["temp_coef"], lt["temp_every"] = t.float("coef"), t.int("every")
        if lt["temp_every"] < 1:
            raise ConfigError(f"{where}: mixer.left.q_temp.every must be at least 1")
    _positive(where + " left", heads=lt["heads"], kv_heads=lt["kv_heads"], dim=lt["dim"],
              vdim=lt["vdim"])
    if lt["heads"] % lt["kv_heads"]:
        raise ConfigError(f"{where}: {lt['heads']} heads cannot be shared out over "
                          f"{lt['kv_heads']} kv heads")
    if lt["bias_max"] <= 1.0:
        raise ConfigError(f"{where}: mixer.left.bias_max must be larger than 1")
    rt = {"heads": right.int("heads"), "dim": right.int("dim"), "vdim": right.int("vdim"),
          "tau": right.float("tau"), "decay_rank": right.int("decay_rank", None)}
    _positive(where + " right", heads=rt["heads"], dim=rt["dim"], vdim=rt["vdim"])
    if rt["tau"] <= 0.0:
        raise ConfigError(f"{where}: mixer.right.tau must be positive")
    return {"left": lt, "right": rt, "left_scale": m.float("left_scale"),
            "right_scale": m.float("right_scale")}


def _latent(m: KeyReader, where: str) -> Dict[str, Any]:
    rot = _sub(m, "rot")
    out = {"heads": m.int("heads"), "dim": m.int("dim"), "rot_dim": m.int("rot_dim"),
           "vdim": m.int("vdim"), "kv_rank": m.int("kv_rank"), "scale": m.float("scale"),
           "rot_base": rot.float("base"), "rot_dims": rot.int("dims"), "window": None}
    if m.raw.get("mask") is not None:
        out["window"] = _sub(m, "mask").int("size")
        if out["window"] < 1:
            raise ConfigError(f"{where}: mixer.mask.size must be at least 1")
    _positive(where, heads=out["heads"], dim=out["dim"], vdim=out["vdim"], kv_rank=out["kv_rank"])
    if out["rot_dim"] < 0 or out["rot_dims"] % 2 or not 0 <= out["rot_dims"] <= out["rot_dim"]:
        raise ConfigError(f"{where}: mixer.rot.dims ({out['rot_dims']}) must be even and at most "
                          f"mixer.rot_dim ({out['rot_dim']})")
    return out


def _delta(m: KeyReader, where: str) -> Dict[str, Any]:
    out = {"heads": m.int("heads"), "kv_heads": m.int("kv_heads"), "dim": m.int("dim"),
           "vdim": m.int("vdim"), "conv": m.int("conv"),
           "decay_rank": m.int("decay_rank", None), "gate_rank": m.int("gate_rank", None)}
    _positive(where, heads=out["heads"], kv_heads=out["kv_heads"], dim=out["dim"],
              vdim=out["vdim"], conv=out["conv"])
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{where}: {out['heads']} heads cannot be shared out over "
                          f"{out['kv_heads']} q/k heads")
    return out


def _layer(raw: Any, i: int) -> DukolornLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(raw, where)
    kind = raw.get("type")
    if kind not in MIXER_TYPES:
        raise ConfigError(f"{where}: type = {kind!r}; known: {', '.join(MIXER_TYPES)}")
    m = _sub(r, "mixer")
    mixer = {"parallel": _parallel, "latent_attention": _latent, "channel_delta": _delta}[kind](
        m, where)
    mlp = None
    if raw.get("mlp") is not None:
        f = _sub(r, "mlp")
        if f.raw.get("kind") != "dense":
            raise ConfigError(f"{where}: mlp.kind = {f.raw.get('kind')!r}; known: dense")
        mlp = {"kind": "dense", "ff": f.int("ff")}
        if mlp["ff"] < 1:
            raise ConfigError(f"{where}: the feed-forward width must be positive")
    return DukolornLayer(kind, mixer, mlp)


@dataclass
class DukolornConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 0.0
    logit_scale: float = 1.0
    layers: List[DukolornLayer] = field(default_factory=list)
    max_position_embeddings: int = 0
    eos_token_id: Optional[Union[int, List[int]]] = None
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "DukolornConfig":
        r = KeyReader(raw)
        cfg = cls(
            architecture=ARCHITECTURE,
            vocab_size=r.int("vocab"),
            width=r.int("width"),
            norm_eps=_sub(r, "norm").float("eps"),
            logit_scale=r.float("logit_scale", 1.0),
            layers=[_layer(x, i) for i, x in enumerate(r.list("layers"))],
            eos_token_id=r.int_or_ints("eos_token_id", None),
            raw=copy.deepcopy(raw),
        )
        if cfg.vocab_size < 1 or cfg.width < 1:
            raise ConfigError("config.json: vocab and width must be positive")
        if not cfg.layers:
            raise ConfigError("config.json: layers must name at least one layer")
        if cfg.norm_eps <= 0.0:
            raise ConfigError("config.json: norm.eps must be positive")
        return cfg

    def adopt_tensor_shapes(self, shapes: Dict[str, tuple]) -> None:
        """Fill in the sizes that the file leaves to the tensors: the rows of the distance-bias
        table, the ranks of the low-rank maps.  A size that config.json states is kept."""
        def rows(name: str, where: str):
            if name not in shapes or not shapes[name]:
                raise ConfigError(f"config.json: {where} is neither stated nor given by a tensor "
                                  f"'{name}'")
            return int(shapes[name][0])

        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.mix.", layer.mixer
            if layer.type == "parallel":
                if m["left"].get("buckets") is None:
                    m["left"]["buckets"] = rows(p + "left.rel", f"layers[{i}] mixer.left.buckets")
                if m["right"].get("decay_rank") is None:
                    m["right"]["decay_rank"] = rows(p + "right.a1",
                                                    f"layers[{i}] mixer.right.decay_rank")
            elif layer.type == "channel_delta":
                if m.get("decay_rank") is None:
                    m["decay_rank"] = rows(p + "a1", f"layers[{i}] mixer.decay_rank")
                if m.get("gate_rank") is None:
                    m["gate_rank"] = rows(p + "g1", f"layers[{i}] mixer.gate_rank")

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
