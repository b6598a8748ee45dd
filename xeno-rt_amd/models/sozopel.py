"""Sozopel: a decoder whose layers each have one of three mixers, described in parts.

Embedding plus a learnt vector per position; then the layers that config.json lists. A layer is pre-norm, with norms
whose gain is a single number, and every sublayer reads its normed input plus a short causal convolution of it over
time. The mixers:
  retention  linear attention with a fixed decay per head (parts/recurrent.py: Retention)
  wkv        time mixing with a decay per channel and token, a bonus for the current token and token shift (TimeMixWKV)
  parallel   a windowed softmax attention (grouped heads, short convolutions on q, k and v, a bias by distance, one more
             in the softmax's denominator) beside a gated linear attention; half the sum of their RMS-normed outputs
A layer may have a dense feed-forward with the activation xIELU, or none. Final norm, then the output head.
Tensor names: `embed`, `pos`, `l<i>.norm1|norm2|canon1|canon2`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config import ConfigError, register_architecture
from ..config.sozopel import SozopelConfig
from ..parts import (Attention, DenseMLP, DistanceSlopes, GatedLinearAttention, OutputHead, ParallelMixer, PositionedEmbedding,
                     PreNormBlock, Retention, ScalarRMSNorm, ShortConvolution, TimeMixWKV)
from .decoder import ModelSpec

SLOPE_SPAN = 8.0        # the distance bias of head h of H falls by 2^(-SLOPE_SPAN (h + 1) / H) a token


def _rank(part: dict, where: str) -> int:
    if "rank" not in part:
        raise ConfigError(f"{where}: the inner width of the decay's projection ('rank') is neither in the configuration "
                          "nor has it been read from a checkpoint's shapes")
    return int(part["rank"])


def _mixer(kind: str, m: dict, p: str, c: SozopelConfig):
    if kind == "retention":
        return Retention(p, c.width, m["heads"], m["dim"], m["vdim"], m["decay"], c.norm_eps, state_name="mix.state")
    if kind == "wkv":
        return TimeMixWKV(p, c.width, m["heads"], m["dim"], _rank(m, p), c.norm_eps, state_name="mix.state")
    left, right = m["left"], m["right"]
    q, kv, v = left["heads"] * left["dim"], left["kv_heads"] * left["dim"], left["kv_heads"] * left["vdim"]
    attention = Attention(
        p + "left.", c.width, left["heads"], left["kv_heads"], left["dim"], position=DistanceSlopes(left["heads"], SLOPE_SPAN),
        scale=left["scale"], window=left["mask"]["size"], value_dim=left["vdim"], sink=True,
        convolution=ShortConvolution([p + "left.q.conv", p + "left.k.conv", p + "left.v.conv"], [q, kv, v], left["conv"],
                                     state_name="mix.left.conv"),
        names={"q": "q", "k": "k", "v": "v", "o": "o"})
    linear = GatedLinearAttention(p + "right.", c.width, right["heads"], right["dim"], right["vdim"], right["tau"],
                                  _rank(right, p + "right."), c.norm_eps, state_name="mix.right.state")
    return ParallelMixer(attention, linear, c.width, p + "left.out", p + "right.out", c.norm_eps, scale=0.5)


def build_sozopel(config: SozopelConfig) -> ModelSpec:
    c = config
    embedding = PositionedEmbedding("", c.vocab, c.width, c.max_positions, name="embed", positions_name="pos")
    layers = []
    for index, layer in enumerate(c.layers):
        p = f"l{index}."
        mlp = layer["mlp"]
        layers.append(PreNormBlock(
            ScalarRMSNorm(p + "norm1", c.width, c.norm_eps),
            _mixer(layer["type"], layer["mixer"], p + "mix.", c),
            None if mlp is None else ScalarRMSNorm(p + "norm2", c.width, c.norm_eps),
            None if mlp is None else DenseMLP(p + "mlp.", c.width, mlp["ff"], "xielu"),
            mixer_input=ShortConvolution([p + "canon1"], [c.width], c.canon_taps, "canon1", plus_input=True),
            feed_forward_input=None if mlp is None else ShortConvolution([p + "canon2"], [c.width], c.canon_taps, "canon2",
                                                                         plus_input=True)))
    return ModelSpec(config=c, embedding=embedding, layers=layers, final_norm=ScalarRMSNorm("final.norm", c.width, c.norm_eps),
                     head=OutputHead("", c.vocab, c.width, name="head"))


register_architecture("Sozopel", SozopelConfig, build_sozopel)
