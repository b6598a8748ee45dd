"""Causal attention with grouped key/value heads over the cache.

The reference's attention (crates/xrt-models/src/llama.rs:447-577 decode,
:695-784 prefill): q, k, v projections without bias; optional RMSNorm of every
head of q and k with one weight [head_dim] each (:1025-1040), after the
projection and before the position encoding; keys (encoded) and values (raw)
appended to the cache; query head h reads key/value head h // group; a token at
position P sees keys 0..P; softmax of q.k * scale in float32; output projection
added to the residual stream.

Q, K and V are bound as one matrix [(n_heads + 2 n_kv_heads) head_dim][hidden], so
one product reads the normed activations once (the reference fuses the three
dispatches, llama.rs:447-464).

Beyond the reference's model, as options: values of a width of their own (`value_dim`), a short causal convolution
over time on every channel of q, k and v right after the projection (`convolution`, whose last inputs are kept per
sequence), a softmax with one more in its denominator (`sink`: a key of score 0 that has no value), a window, a
position encoding that biases the scores by distance, and tensor names of the caller's choice (`names`). With any of
the first three the step takes the general attention kernel, and the keys and values reach the cache through a
kernel of their own.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import CacheNeeds, KVSpec, Mixer, PositionEncoding, Runtime, WeightSpec, register_part


class Attention(Mixer):
    passes_norms = True

    @property
    def capturable(self) -> bool:
        return ((self.position is None or self.position.capturable)
                and (getattr(self, "convolution", None) is None or self.convolution.capturable))

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding] = None, qk_norm: bool = False,
                 qk_norm_eps: float = 0.0, scale: Optional[float] = None,
                 window: Optional[int] = None, value_dim: Optional[int] = None, sink: bool = False,
                 convolution=None, names: Optional[Dict[str, str]] = None):
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads != 0:
            raise ValueError(f"head counts {n_heads}/{n_kv_heads}: the first must be a multiple of the second")
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        self.sink = bool(sink)
        self.convolution = convolution
        self.general = self.sink or self.value_dim != head_dim or convolution is not None
        if head_dim <= 0 or (head_dim % 2 != 0 and not self.general):   # llama.rs:125-128 takes any size; the rotation pairs dims, so an even one
            raise ValueError(f"head_dim {head_dim} must be positive and even")
        if self.general and qk_norm:
            raise ValueError("attention with a sink, a convolution or values of another width takes no head norms")
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                      "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", **(names or {})}
        self.prefix = prefix
        self.hidden = hidden
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.position = position
        self.qk_norm = qk_norm
        self.qk_norm_eps = float(qk_norm_eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)  # llama.rs:506
        self.window = window
        self.q_width = n_heads * head_dim
        self.kv_width = n_kv_heads * head_dim
        self.v_width = n_kv_heads * self.value_dim
        self.w_qkv = None
        self.w_o = None
        self.q_norm = None
        self.k_norm = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, n = self.prefix, self.names
        specs = {
            p + n["q"]: WeightSpec((self.q_width, self.hidden)),
            p + n["k"]: WeightSpec((self.kv_width, self.hidden)),
            p + n["v"]: WeightSpec((self.v_width, self.hidden)),
            p + n["o"]: WeightSpec((self.hidden, self.n_heads * self.value_dim)),
        }
        if self.qk_norm:
            specs[p + n["q_norm"]] = WeightSpec((self.head_dim,), init="ones", kind="vector")
            specs[p + n["k_norm"]] = WeightSpec((self.head_dim,), init="ones", kind="vector")
        if self.convolution is not None:
            specs.update(self.convolution.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        needs = CacheNeeds(kv=KVSpec(self.n_kv_heads, self.head_dim, self.window,
                                     None if self.value_dim == self.head_dim else self.value_dim))
        return needs if self.convolution is None else needs.merged(self.convolution.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p, n = self.prefix, self.names
        if self.position is not None:
            self.position.bind(tensors, runtime)
        if self.general:
            if self.position is not None and self.position.rotation() is not None:
                raise ValueError("attention with a sink, a convolution or values of another width takes no rotation")
            if self.convolution is not None:
                self.convolution.bind(tensors, runtime)
            self.w_qkv = runtime.weight([tensors[p + n[name]] for name in "qkv"])
            self.w_o = runtime.weight(tensors[p + n["o"]])
            return
        # q and k heads that a rotation over the whole head turns: their pairs are kept side by side
        rotation = None if self.position is None else self.position.rotation()
        whole = rotation is not None and rotation.rope_dim == self.head_dim
        self.w_qkv = runtime.weight([tensors[p + n[name]] for name in "qkv"],
                                    "rotary", head_dim=self.head_dim,
                                    rotated_heads=self.n_heads + self.n_kv_heads if whole else 0)
        self.w_o = runtime.weight(tensors[p + n["o"]])
        if self.qk_norm:
            self.q_norm = runtime.vector(tensors[p + n["q_norm"]])
            self.k_norm = runtime.vector(tensors[p + n["k_norm"]])

    def _attend_general(self, h, batch, cache):
        """The heads' outputs [tokens, n_heads * value_dim] on the general path: projection, convolution over time, the keys and
        values into the cache, attention."""
        rt = self.runtime
        ops = rt.ops
        tokens = h.shape[0]
        qkv = rt.empty((tokens, self.q_width + self.kv_width + self.v_width))
        ops.linear(h, self.w_qkv, qkv)
        if self.convolution is not None:
            qkv = self.convolution.forward(qkv, batch, cache)
        if cache.writable:
            ops.kv_store(qkv[:, self.q_width:self.q_width + self.kv_width], qkv[:, self.q_width + self.kv_width:],
                         self.n_kv_heads, self.head_dim, self.value_dim, cache.kv, batch)
        slopes = None if self.position is None else self.position.score_slopes()
        out = rt.empty((tokens, self.n_heads * self.value_dim))
        ops.attention(qkv, self.n_heads, self.n_kv_heads, self.head_dim, cache.kv, batch, out, scale=self.scale, window=self.window,
                      distance_slopes=slopes, value_dim=self.value_dim, sink=self.sink)
        return out

    def forward_into(self, h, batch, cache, out: torch.Tensor) -> None:
        """The mixer's output into `out` (float32 [tokens, hidden]) instead of onto the residual stream: for an attention
        that is one of several mixers side by side."""
        if not self.general:
            raise NotImplementedError("only the general path writes its output aside")
        self.runtime.ops.linear(self._attend_general(h, batch, cache), self.w_o, out)

    def forward(self, h, batch, cache, residual: torch.Tensor, then=None):
        if self.general:
            self.runtime.ops.linear(self._attend_general(h, batch, cache), self.w_o, residual, accumulate=True)
            return None
        rt = self.runtime
        ops = rt.ops
        tokens = h.shape[0]
        kv = cache.kv
        qkv = rt.empty((tokens, self.q_width + 2 * self.kv_width))

        dims = (self.n_heads, self.n_kv_heads, self.head_dim)
        write_to = kv if cache.writable else None
        longest_run = int(getattr(batch, "max_count", 0) or 0)      # picks how the values are written; 0: unknown
        rotation = None if self.position is None else self.position.rotation()
        slopes = None if self.position is None else self.position.score_slopes()
        out = rt.empty((tokens, self.q_width))
        # A decode step of a model with head norms: the projection only, and the attention kernel finishes q, k and v
        # itself (norms, rotation, cache write) where it can; without head norms the projection's own kernel does that.
        finishes = getattr(ops, "attention_finishes_qkv", None)
        if (self.qk_norm and write_to is not None and slopes is None and (rotation is not None or self.position is None)
                and finishes is not None and finishes(qkv.dtype, *dims, batch, self.window, 0 if rotation is None else rotation.rope_dim,
                                                       None if rotation is None else rotation.table)):
            ops.linear(h, self.w_qkv, qkv)
            ops.attention(qkv, *dims, kv, batch, out, scale=self.scale,
                          finish=ops.QkvFinish(self.q_norm, self.k_norm, self.qk_norm_eps, None if rotation is None else rotation.table))
            return ops.linear(out, self.w_o, residual, accumulate=True,
                              then_norm=None if then is None else then.row_scale())
        if rotation is not None or self.position is None:
            # the projection, then in one pass (in the same kernel, where a step is short): head norms, rotation, cache write
            ops.linear_qkv(h, self.w_qkv, qkv, *dims, batch.positions, batch.slots,
                            q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps,
                            rope_theta=None if rotation is None else rotation.theta,
                            rope_dim=0 if rotation is None else rotation.rope_dim,
                            rope_scale=1.0 if rotation is None else rotation.scale,
                            kv=write_to, longest_run=longest_run)
        else:
            # any other position encoding: norms, then the encoding, then the cache write
            ops.linear(h, self.w_qkv, qkv)
            if self.qk_norm:
                ops.qkv_prepare(qkv, *dims, batch.positions, batch.slots,
                                q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps)
            self.position.apply(qkv, *dims, batch)
            if write_to is not None:
                ops.qkv_prepare(qkv, *dims, batch.positions, batch.slots, kv=write_to, longest_run=longest_run)

        ops.attention(qkv, *dims, kv, batch, out, scale=self.scale, window=self.window,
                      **({} if slopes is None else {"distance_slopes": slopes}))
        return ops.linear(out, self.w_o, residual, accumulate=True,
                          then_norm=None if then is None else then.row_scale())


register_part("mixer", "attention", Attention)
