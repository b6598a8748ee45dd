"""Configuration of the Sozopel decoder: a stack of layers that may each have another mixer.

config.json names the design under `architecture` and lists the layers; each entry gives `type` (which mixer), the
mixer's sizes under `mixer`, and `mlp` (the feed-forward's sizes, or null for a layer without one). Sizes that
config.json leaves to the tensors' shapes (the inner width of the low-rank projections that make a decay) are filled
in from the checkpoint's header by `completed_from` and then written under the mixer's key `rank`.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from . import ConfigError, _positive_int, _require

MIXER_TYPES = ("retention", "wkv", "parallel")
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
    if kind == "retention":
        _sizes(mixer, ("heads", "dim", "vdim"), where)
        decay = mixer.get("decay")
        if not isinstance(decay, list) or len(decay) != mixer["heads"] or not all(isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"config.json: {where}: 'decay' must list one number per head")
    elif kind == "wkv":
        _sizes(mixer, ("heads", "dim"), where)
    else:
        left, right = mixer.get("left"), mixer.get("right")
        if not isinstance(left, dict) or not isinstance(right, dict):
            raise ConfigError(f"config.json: {where}: a parallel mixer has 'left' and 'right'")
        _sizes(left, ("heads", "kv_heads", "dim", "vdim", "conv"), where + ".left")
        if left["heads"] % left["kv_heads"] != 0:
            raise ConfigError(f"config.json: {where}.left: {left['heads']} heads cannot share {left['kv_heads']} key/value heads")
        _number(left, "scale", where + ".left")
        if not isinstance(left.get("mask"), dict):
            raise ConfigError(f"config.json: {where}.left: 'mask' must give the window's size")
        _sizes(left["mask"], ("size",), where + ".left.mask")
        _sizes(right, ("heads", "dim", "vdim"), where + ".right")
        if _number(right, "tau", where + ".right") <= 0:
            raise ConfigError(f"config.json: {where}.right: 'tau' must be positive")
    for part in ([mixer] if kind != "parallel" else [mixer["right"]]):
        if "rank" in part:
            _sizes(part, ("rank",), where)


@dataclass(frozen=True)
class SozopelConfig:
    architecture: str
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    canon_taps: int
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
    def max_position_embeddings(self) -> int:
        return self.max_positions

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict) -> "SozopelConfig":
        layers = _require(raw, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        kept = []
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}: 'type' must be one of {MIXER_TYPES}")
            if not isinstance(layer.get("mixer"), dict):
                raise ConfigError(f"config.json: {where}: 'mixer' must give the mixer's sizes")
            _check_mixer(layer["type"], layer["mixer"], where + ".mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp: 'kind' must be one of {MLP_KINDS}")
                _sizes(mlp, ("ff",), where + ".mlp")
            kept.append(copy.deepcopy({"type": layer["type"], "mixer": layer["mixer"], "mlp": mlp}))
        norm, canon = _require(raw, "norm"), _require(raw, "canon")
        if not isinstance(norm, dict) or not isinstance(canon, dict):
            raise ConfigError("config.json: 'norm' and 'canon' must be objects")
        taps = _positive_int(canon, "taps")
        eos = raw.get("eos_token_id")
        eos = () if eos is None else tuple(eos) if isinstance(eos, list) else (eos,)
        return cls(architecture=str(raw.get("architecture") or raw["architectures"][0]), vocab=_positive_int(raw, "vocab"),
                   width=_positive_int(raw, "width"), max_positions=_positive_int(raw, "max_positions"),
                   norm_eps=_number(norm, "eps", "norm"), canon_taps=taps, layers=tuple(kept),
                   eos_token_ids=tuple(int(e) for e in eos), bos_token_id=raw.get("bos_token_id"))

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "max_positions": self.max_positions, "norm": {"eps": self.norm_eps}, "canon": {"taps": self.canon_taps},
               "layers": copy.deepcopy(list(self.layers))}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    def __hash__(self):
        return hash((self.architecture, self.vocab, self.width, len(self.layers)))

    # -- sizes that only the tensors give --------------------------------------------------------------------------
    @staticmethod
    def rank_tensor(index: int, kind: str) -> str:
        """The tensor whose first dimension is the inner width of layer `index`'s decay projection."""
        return f"l{index}.mix.w1" if kind == "wkv" else f"l{index}.mix.right.a1"

    def completed_from(self, shapes: Dict[str, tuple]) -> "SozopelConfig":
        """The same configuration with every 'rank' that config.json left out read from the tensors' shapes."""
        layers = copy.deepcopy(list(self.layers))
        for index, layer in enumerate(layers):
            if layer["type"] == "retention":
                continue
            part = layer["mixer"] if layer["type"] == "wkv" else layer["mixer"]["right"]
            if "rank" not in part:
                name = self.rank_tensor(index, layer["type"])
                if name not in shapes or len(shapes[name]) != 2:
                    raise ConfigError(f"the checkpoint has no matrix '{name}' to read the decay projection's inner width from")
                part["rank"] = int(shapes[name][0])
        return SozopelConfig(self.architecture, self.vocab, self.width, self.max_positions, self.norm_eps, self.canon_taps,
                             tuple(layers), self.eos_token_ids, self.bos_token_id)
