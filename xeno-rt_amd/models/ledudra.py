"""Ledudra: a decoder of attention layers of two kinds, each between norms before and after, described in parts.

Embedding; then the layers that config.json lists. A layer is x += m * post(sublayer(pre(x))) for the mixer and, if it
has one, for a gated feed-forward (silu), with layer norms (weight and bias) before and after each and one number m for
the whole model. What the mixer reads is first moved towards the normed row of the token before (`<layer>.shift`).
The mixers:
  attention    q, k, v and output projections with biases; the first rot.dims dims of every head of q and k rotated in
               pairs of neighbours, frequencies stretched for long contexts; the heads' scores of a (query, key) pair
               mixed by a matrix; the weight of a key inside the window is sigmoid(score + a number per head), not
               normalised over the keys; a gate per token and head on the heads' outputs
  attention_2  no biases; an RMS norm of every head of q and k; no rotation, but a learnt bias per head and bucket of
               distance on the scores; softmax over the window
In every layer that shares values but the first of them, the values are blended with those the first one made of the
same token. Final layer norm, then the output head.
Tensor names: `embed`, `l<i>.norm1|norm1b|norm2|norm2b` (biases with `.b`), `l<i>.shift`, `l<i>.mix.*`, `l<i>.mlp.*`,
`final.norm`, `head`.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.ledudra import LedudraConfig
from ..parts import (Attention, DistanceBuckets, Embedding, GatedMLP, LayerNorm, OutputHead, PairRotation, SandwichBlock,
                     SharedValues, TokenShift)
from .decoder import ModelSpec


def _norm(name: str, c: LedudraConfig) -> LayerNorm:
    return LayerNorm(name, name + ".b", c.width, c.norm_eps)


def _mixer(kind: str, m: dict, p: str, c: LedudraConfig, values) -> Attention:
    common = dict(scale=m["scale"], window=(m.get("mask") or {}).get("size"), value_dim=m["vdim"], values=values,
                  unread=() if values is not None else ("vmix",))
    if kind == "attention":
        rot = m.get("rot")
        position = None if rot is None else PairRotation(rot["dims"], rot["base"], neighbours=True, scaling=rot.get("scaling"))
        return Attention(p, c.width, m["heads"], m["kv_heads"], m["dim"], position=position, biases=True, weights="sigmoid",
                         head_mix="talk", score_bias="pb", output_gate="g",
                         names={"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                                "o_bias": "o.b"}, **common)
    table_rows = m.get("bias_rows")
    if table_rows is None:
        raise ValueError(f"{p}: the rows of the table of biases by distance are read from the checkpoint's shapes")
    return Attention(p, c.width, m["heads"], m["kv_heads"], m["dim"],
                     position=DistanceBuckets(p + "rel", m["heads"], table_rows, m["bias_max"]), qk_norm=True, qk_norm_eps=c.norm_eps,
                     names={"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}, **common)


def build_ledudra(config: LedudraConfig) -> ModelSpec:
    c = config
    shared, first = SharedValues(), True
    layers = []
    for index, layer in enumerate(c.layers):
        p = f"l{index}."
        values = None
        if layer["mixer"].get("v_mix"):
            values = shared.source("vmix") if first else shared.reader("vmix")
            first = False
        mlp = layer["mlp"]
        layers.append(SandwichBlock(
            _norm(p + "norm1", c), _mixer(layer["type"], layer["mixer"], p + "mix.", c, values), _norm(p + "norm1b", c),
            None if mlp is None else _norm(p + "norm2", c),
            None if mlp is None else GatedMLP(p + "mlp.", c.width, mlp["ff"], "silu", gate="gate", up="up", down="down"),
            None if mlp is None else _norm(p + "norm2b", c),
            residual_scale=c.residual_mult,
            mixer_input=TokenShift([p + "shift"], c.width, "shift", single=True)))
    return ModelSpec(config=c, embedding=Embedding("", c.vocab, c.width, name="embed"), layers=layers,
                     final_norm=_norm("final.norm", c), head=OutputHead("", c.vocab, c.width, name="head"))


register_architecture("Ledudra", LedudraConfig, build_ledudra)
