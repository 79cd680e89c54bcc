"""ZederaxConfig: the configuration of the Zederax architecture under its config.json keys.

config.json: ``architecture`` ("Zederax"), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list with one entry per
layer: ``type`` (the mixer: "attention"), ``mixer`` (its sizes and constants: ``heads``, ``kv_heads``, ``dim`` of a
query/key head, ``vdim`` of a value head, ``scale``, ``softcap``, ``mask.size`` the window, ``v_mix``) and ``mlp``
(``kind`` "dense" with its inner width ``ff``, or null for a layer without a feed-forward). Layers may differ in all of it.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .lm_config import ConfigError, LmConfig

MIXER_TYPES = ("attention",)
MLP_KINDS = ("dense",)


def _positive_int(v) -> bool:
    return isinstance(v, int) and not isinstance(v, bool) and v > 0


@LmConfig.register_subclass("zederax")
@dataclass(frozen=True)
class ZederaxConfig(LmConfig):
    vocab: int = 0
    width: int = 0
    norm_eps: float = 1e-6
    layers: Tuple[Dict[str, Any], ...] = ()
    initializer_range: float = 0.02

    def __post_init__(self):
        if not _positive_int(self.vocab) or not _positive_int(self.width):
            raise ConfigError(f"zederax: vocab and width must be positive integers, got {self.vocab!r} and {self.width!r}")
        if not (isinstance(self.norm_eps, (int, float)) and self.norm_eps > 0):
            raise ConfigError(f"zederax: norm.eps must be positive, got {self.norm_eps!r}")
        if not self.layers:
            raise ConfigError("zederax: the configuration lists no layers")
        mixed = None
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"zederax: layer {i} has type {layer.get('type') if isinstance(layer, dict) else layer!r}; known: {', '.join(MIXER_TYPES)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"zederax: layer {i} has no 'mixer' sizes")
            m.setdefault("kv_heads", m.get("heads"))  # left out: every head has keys and values of its own, of one size
            m.setdefault("vdim", m.get("dim"))
            for key in ("heads", "kv_heads", "dim", "vdim"):
                if not _positive_int(m.get(key)):
                    raise ConfigError(f"zederax: layer {i}: mixer.{key} must be a positive integer, got {m.get(key)!r}")
            if m["heads"] % m["kv_heads"] != 0:
                raise ConfigError(f"zederax: layer {i}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv_heads")
            if not isinstance(m.get("scale"), (int, float)) or isinstance(m.get("scale"), bool):
                raise ConfigError(f"zederax: layer {i}: mixer.scale must be a number, got {m.get('scale')!r}")
            cap = m.get("softcap")
            if cap is not None and not (isinstance(cap, (int, float)) and not isinstance(cap, bool) and cap > 0):
                raise ConfigError(f"zederax: layer {i}: mixer.softcap must be a positive number or absent, got {cap!r}")
            mask = m.get("mask")
            if mask is not None and not (isinstance(mask, dict) and (mask.get("size") is None or _positive_int(mask.get("size")))):
                raise ConfigError(f"zederax: layer {i}: mixer.mask must be {{'size': positive integer}}, got {mask!r}")
            if m.get("v_mix"):
                sizes = (m["kv_heads"], m["vdim"])
                if mixed is not None and sizes != mixed:
                    raise ConfigError(f"zederax: layer {i} mixes its values with the first such layer's, whose value heads differ "
                                      f"({mixed[0]} x {mixed[1]} against {sizes[0]} x {sizes[1]})")
                mixed = sizes
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"zederax: layer {i}: mlp.kind must be one of {', '.join(MLP_KINDS)}, got {mlp!r}")
                if not _positive_int(mlp.get("ff")):
                    raise ConfigError(f"zederax: layer {i}: mlp.ff must be a positive integer, got {mlp.get('ff')!r}")

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_hf_config(cls, hf_config: Dict[str, Any]) -> "ZederaxConfig":
        for required in ("vocab", "width", "layers"):
            if required not in hf_config:
                raise ConfigError(f"zederax: config.json lacks the key {required!r}")
        norm = hf_config.get("norm") or {}
        if not isinstance(norm, dict) or "eps" not in norm:
            raise ConfigError("zederax: config.json lacks norm.eps")
        layers = hf_config["layers"]
        if not isinstance(layers, (list, tuple)):
            raise ConfigError("zederax: 'layers' must be a list")
        extra = {"initializer_range": hf_config["initializer_range"]} if "initializer_range" in hf_config else {}
        return cls(vocab=hf_config["vocab"], width=hf_config["width"], norm_eps=norm["eps"], layers=tuple(copy.deepcopy(list(layers))), **extra)

    def to_hf_config(self) -> Dict[str, Any]:
        return {"architecture": "Zederax", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "layers": copy.deepcopy(list(self.layers)), "initializer_range": self.initializer_range}

    def __hash__(self):
        return hash((self.vocab, self.width, self.norm_eps, repr(self.layers)))

    def model_spec(self):
        from levanter_amd.models.zederax import zederax_model_spec

        return zederax_model_spec(self)
