"""Mixers whose memory is a matrix per head: S <- diag(decay) S + k v^T, read with the query.

Three of them, which differ in where the decay comes from and in what surrounds the recurrence:
  Retention             a fixed decay per head; k scaled by dim^-1/2; the heads' outputs divided by their root mean
                        square, gated by silu of a projection
  GatedLinearAttention  a decay per key channel and token, sigmoid(z)^(1/tau) with z from a low-rank projection with
                        bias; q scaled by dim^-1/2; the heads' outputs RMS-normed with a weight [vdim], gated
  TimeMixWKV            every projection reads its own mix of the token and the one before it; decay
                        exp(-exp(w0 + W2 tanh(W1 mix))) per key channel and token; the current token is read with a
                        bonus u before it enters the state; outputs divided by their root mean square, times a weight
                        over all heads, gated
The state [heads, dim, vdim] is float32 and so are decays, norms and gates' activations; projections run in the compute dtype.
All run through one kernel (`ops.linear_recurrence`), which walks a sequence's tokens in order from the state that
the steps before left, so a request gives the same result however it is cut into steps.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .base import CacheNeeds, Mixer, Runtime, StateSpec, WeightSpec, register_part
from .convolution import TokenShift


class _RecurrentMixer(Mixer):
    capturable = True

    def _project_into(self, out_or_residual, o, accumulate: bool):
        return self.runtime.ops.linear(o, self.w_o, out_or_residual, accumulate=accumulate)

    def forward(self, h, batch, cache, residual: torch.Tensor) -> None:
        """Adds the mixer's output to the float32 residual stream."""
        self._project_into(residual, self.mixed(h, batch, cache), True)

    def forward_into(self, h, batch, cache, out: torch.Tensor) -> None:
        """Writes the mixer's output to `out` (float32) instead: for a mixer that is one of several side by side."""
        self._project_into(out, self.mixed(h, batch, cache), False)


class Retention(_RecurrentMixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, decay: Sequence[float], eps: float,
                 state_name: str = "retention"):
        if len(decay) != heads:
            raise ValueError(f"retention: {len(decay)} decays for {heads} heads")
        self.prefix, self.hidden, self.heads, self.dim, self.vdim = prefix, hidden, heads, dim, vdim
        self.decay_values, self.eps, self.state_name = [float(d) for d in decay], float(eps), state_name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd, vd = self.prefix, self.hidden, self.heads * self.dim, self.heads * self.vdim
        return {p + "q": WeightSpec((kd, w)), p + "k": WeightSpec((kd, w)), p + "v": WeightSpec((vd, w)),
                p + "g": WeightSpec((vd, w)), p + "o": WeightSpec((w, vd))}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.vdim))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.w_in = runtime.weight([tensors[p + name] for name in "qkvg"])
        self.w_o = runtime.weight(tensors[p + "o"])
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=runtime.device)

    def mixed(self, h, batch, cache):
        rt = self.runtime
        kd, vd = self.heads * self.dim, self.heads * self.vdim
        qkvg = rt.empty((h.shape[0], 2 * kd + 2 * vd))
        rt.ops.linear(h, self.w_in, qkvg)
        o = rt.empty((h.shape[0], vd))
        rt.ops.linear_recurrence(qkvg[:, :kd], qkvg[:, kd:2 * kd], qkvg[:, 2 * kd:2 * kd + vd], cache.states[self.state_name], batch, o,
                                 self.heads, self.dim, self.vdim, self.decay, "per_head", k_scale=self.dim ** -0.5,
                                 norm_eps=self.eps, gate=qkvg[:, 2 * kd + vd:], gate_activation="silu")
        return o


class GatedLinearAttention(_RecurrentMixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, tau: float, low_rank: int, eps: float,
                 state_name: str = "gla"):
        self.prefix, self.hidden, self.heads, self.dim, self.vdim = prefix, hidden, heads, dim, vdim
        self.tau, self.low_rank, self.eps, self.state_name = float(tau), int(low_rank), float(eps), state_name

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd, vd = self.prefix, self.hidden, self.heads * self.dim, self.heads * self.vdim
        return {p + "q": WeightSpec((kd, w)), p + "k": WeightSpec((kd, w)), p + "v": WeightSpec((vd, w)),
                p + "g": WeightSpec((vd, w)), p + "o": WeightSpec((w, vd)),
                p + "a1": WeightSpec((self.low_rank, w)), p + "a2": WeightSpec((kd, self.low_rank)),
                p + "a2.b": WeightSpec((kd,), kind="vector"),
                p + "norm": WeightSpec((self.vdim,), init="ones", kind="vector")}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.vdim))),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.w_in = runtime.weight([tensors[p + name] for name in "qkvg"])
        self.w_a1 = runtime.weight(tensors[p + "a1"])
        self.w_a2 = runtime.weight(tensors[p + "a2"])
        self.a2_bias = runtime.vector(tensors[p + "a2.b"])
        self.norm_weight = runtime.vector(tensors[p + "norm"])
        self.w_o = runtime.weight(tensors[p + "o"])

    def mixed(self, h, batch, cache):
        rt = self.runtime
        tokens, kd, vd = h.shape[0], self.heads * self.dim, self.heads * self.vdim
        qkvg = rt.empty((tokens, 2 * kd + 2 * vd))
        rt.ops.linear(h, self.w_in, qkvg)
        low = rt.empty((tokens, self.low_rank))
        rt.ops.linear(h, self.w_a1, low)
        z = rt.empty((tokens, kd), torch.float32)                        # what the decay is made of stays float32
        rt.ops.linear(low, self.w_a2, z)
        o = rt.empty((tokens, vd))
        rt.ops.linear_recurrence(qkvg[:, :kd], qkvg[:, kd:2 * kd], qkvg[:, 2 * kd:2 * kd + vd], cache.states[self.state_name], batch, o,
                                 self.heads, self.dim, self.vdim, z, "sigmoid_power", decay_bias=self.a2_bias,
                                 decay_power=1.0 / self.tau, q_scale=self.dim ** -0.5, norm_eps=self.eps,
                                 norm_weight=self.norm_weight, gate=qkvg[:, 2 * kd + vd:], gate_activation="silu")
        return o


class TimeMixWKV(_RecurrentMixer):
    READERS = ("r", "k", "v", "g", "w")

    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, low_rank: int, eps: float, state_name: str = "wkv"):
        self.prefix, self.hidden, self.heads, self.dim = prefix, hidden, heads, dim
        self.low_rank, self.eps, self.state_name = int(low_rank), float(eps), state_name
        self.shift = TokenShift([prefix + "mu." + reader for reader in self.READERS], hidden, state_name + ".before")

    @property
    def capturable(self) -> bool:
        return self.shift.capturable

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, kd = self.prefix, self.hidden, self.heads * self.dim
        specs = {p + name: WeightSpec((kd, w)) for name in "rkvg"}
        specs.update({p + "w1": WeightSpec((self.low_rank, w)), p + "w2": WeightSpec((kd, self.low_rank)),
                      p + "w0": WeightSpec((kd,), kind="vector"),
                      p + "u": WeightSpec((self.heads, self.dim), kind="vector"),
                      p + "norm": WeightSpec((kd,), init="ones", kind="vector"), p + "o": WeightSpec((w, kd))})
        specs.update(self.shift.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(states=((self.state_name, StateSpec((self.heads, self.dim, self.dim))),)).merged(self.shift.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.shift.bind(tensors, runtime)
        self.w_r, self.w_k, self.w_v, self.w_g = (runtime.weight(tensors[p + name]) for name in "rkvg")
        self.w_1 = runtime.weight(tensors[p + "w1"])
        self.w_2 = runtime.weight(tensors[p + "w2"])
        self.w0 = runtime.vector(tensors[p + "w0"])
        self.bonus = runtime.vector(tensors[p + "u"])
        self.norm_weight = runtime.vector(tensors[p + "norm"])
        self.w_o = runtime.weight(tensors[p + "o"])

    def mixed(self, h, batch, cache):
        rt = self.runtime
        tokens, kd = h.shape[0], self.heads * self.dim
        mixes = self.shift.forward(h, batch, cache)                      # [5, tokens, hidden]: r, k, v, g, w
        rkvg = [rt.empty((tokens, kd)) for _ in range(4)]
        for mix, weight, out in zip(mixes, (self.w_r, self.w_k, self.w_v, self.w_g), rkvg):
            rt.ops.linear(mix, weight, out)
        low = rt.empty((tokens, self.low_rank), torch.float32)
        rt.ops.linear(mixes[4], self.w_1, low)
        squashed = rt.empty((tokens, self.low_rank))
        rt.ops.activation(low, squashed, "tanh")
        z = rt.empty((tokens, kd), torch.float32)
        rt.ops.linear(squashed, self.w_2, z)
        o = rt.empty((tokens, kd))
        rt.ops.linear_recurrence(rkvg[0], rkvg[1], rkvg[2], cache.states[self.state_name], batch, o, self.heads, self.dim, self.dim,
                                 z, "exp_neg_exp", decay_bias=self.w0, bonus=self.bonus, norm_eps=self.eps,
                                 norm_weight=self.norm_weight, gate=rkvg[3], gate_activation="silu")
        return o


register_part("mixer", "retention", Retention)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "time_mix_wkv", TimeMixWKV)
