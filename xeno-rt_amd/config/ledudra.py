"""Configuration of the Ledudra decoder: a stack of attention layers of two kinds.

config.json names the design under `architecture` and lists the layers; each entry gives `type` (which mixer), the
mixer's sizes and constants under `mixer`, and `mlp` (the feed-forward's sizes, or null for a layer without one).
Every size and constant is read from there; a key that a mixer may do without (a window, a rotation, its scaling,
the sharing of values) may be absent.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from . import ConfigError, _positive_int, _require

MIXER_TYPES = ("attention", "attention_2")
MLP_KINDS = ("dense",)


def _number(raw: dict, key: str, where: str) -> float:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json: {where}: '{key}' must be a number, found {value!r}")
    return float(value)


def _sizes(raw: dict, keys, where: str) -> None:
    for key in keys:
        value = raw.get(key)
        if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
            raise ConfigError(f"config.json: {where}: '{key}' must be a positive integer, found {value!r}")


def _check_mixer(kind: str, mixer: dict, where: str) -> None:
    _sizes(mixer, ("heads", "kv_heads", "dim", "vdim"), where)
    if mixer["heads"] % mixer["kv_heads"] != 0:
        raise ConfigError(f"config.json: {where}: {mixer['heads']} heads cannot share {mixer['kv_heads']} key/value heads")
    _number(mixer, "scale", where)
    mask = mixer.get("mask")
    if mask is not None:
        if not isinstance(mask, dict):
            raise ConfigError(f"config.json: {where}: 'mask' must give the window's size")
        _sizes(mask, ("size",), where + ".mask")
    if not isinstance(mixer.get("v_mix", False), bool):
        raise ConfigError(f"config.json: {where}: 'v_mix' is true or false")
    if kind == "attention":
        rot = mixer.get("rot")
        if rot is not None:
            if not isinstance(rot, dict):
                raise ConfigError(f"config.json: {where}: 'rot' must give the rotation's base and dims")
            _sizes(rot, ("dims",), where + ".rot")
            if rot["dims"] % 2 != 0 or rot["dims"] > mixer["dim"]:
                raise ConfigError(f"config.json: {where}.rot: {rot['dims']} rotated dims of a head of {mixer['dim']}: an even number within the head")
            if _number(rot, "base", where + ".rot") <= 1.0:
                raise ConfigError(f"config.json: {where}.rot: 'base' must exceed 1")
            scaling = rot.get("scaling")
            if scaling is not None:
                if not isinstance(scaling, dict):
                    raise ConfigError(f"config.json: {where}.rot: 'scaling' must give factor, original, fast and slow")
                for key in ("factor", "original", "fast", "slow"):
                    if _number(scaling, key, where + ".rot.scaling") <= 0:
                        raise ConfigError(f"config.json: {where}.rot.scaling: '{key}' must be positive")
    else:
        if _number(mixer, "bias_max", where) <= 0:
            raise ConfigError(f"config.json: {where}: 'bias_max' must be positive")
        if "bias_rows" in mixer:
            _sizes(mixer, ("bias_rows",), where)


@dataclass(frozen=True)
class LedudraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[dict, ...]            # as config.json lists them: {"type", "mixer", "mlp"}
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    # what the rest of the library asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict) -> "LedudraConfig":
        layers = _require(raw, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        kept, shared = [], None
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}: 'type' must be one of {MIXER_TYPES}")
            if not isinstance(layer.get("mixer"), dict):
                raise ConfigError(f"config.json: {where}: 'mixer' must give the mixer's sizes")
            _check_mixer(layer["type"], layer["mixer"], where + ".mixer")
            mixer = layer["mixer"]
            if mixer.get("v_mix"):
                width = mixer["kv_heads"] * mixer["vdim"]
                if shared is not None and shared != width:
                    raise ConfigError(f"config.json: {where}.mixer: values of {width} numbers a token cannot be mixed with the "
                                      f"{shared} of the first layer that shares its values")
                shared = width
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp: 'kind' must be one of {MLP_KINDS}")
                _sizes(mlp, ("ff",), where + ".mlp")
            kept.append(copy.deepcopy({"type": layer["type"], "mixer": mixer, "mlp": mlp}))
        norm = _require(raw, "norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        eos = raw.get("eos_token_id")
        eos = () if eos is None else tuple(eos) if isinstance(eos, list) else (eos,)
        return cls(architecture=str(raw.get("architecture") or raw["architectures"][0]), vocab=_positive_int(raw, "vocab"),
                   width=_positive_int(raw, "width"), norm_eps=_number(norm, "eps", "norm"),
                   residual_mult=_number(raw, "residual_mult", "config") if "residual_mult" in raw else 1.0,
                   layers=tuple(kept), eos_token_ids=tuple(int(e) for e in eos), bos_token_id=raw.get("bos_token_id"))

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "residual_mult": self.residual_mult, "layers": copy.deepcopy(list(self.layers))}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    def __hash__(self):
        return hash((self.architecture, self.vocab, self.width, len(self.layers)))

    # -- sizes that only the tensors give --------------------------------------------------------------------------
    @staticmethod
    def bias_table(index: int) -> str:
        """The tensor whose first dimension is the number of distance buckets of layer `index`."""
        return f"l{index}.mix.rel"

    def completed_from(self, shapes: Dict[str, tuple]) -> "LedudraConfig":
        """The same configuration with every 'bias_rows' that config.json left out read from the tensors' shapes."""
        layers = copy.deepcopy(list(self.layers))
        for index, layer in enumerate(layers):
            if layer["type"] != "attention_2" or "bias_rows" in layer["mixer"]:
                continue
            name = self.bias_table(index)
            if name not in shapes or len(shapes[name]) != 2:
                raise ConfigError(f"the checkpoint has no table '{name}' to read the number of distance buckets from")
            layer["mixer"]["bias_rows"] = int(shapes[name][0])
        return LedudraConfig(self.architecture, self.vocab, self.width, self.norm_eps, self.residual_mult, tuple(layers),
                             self.eos_token_ids, self.bos_token_id)
