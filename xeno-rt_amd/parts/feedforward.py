"""Dense gated feed-forward: x + W_down (act(W_gate y) * (W_up y)), no biases.

The reference's SwiGLU block (crates/xrt-models/src/llama.rs:582-601) with
silu(z) = z / (1 + exp(-z)) (crates/xrt-kernels/src/cpu/silu.rs:1-3, 22-24).
Gate and up are bound as one matrix [2I][H] so that one product reads the
normed activations once, as the reference fuses the two dispatches
(llama.rs:584-594).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import FeedForward, Runtime, WeightSpec, register_part


class GatedMLP(FeedForward):
    capturable = True
    passes_norms = True

    ACTIVATIONS = ("silu",)

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu",
                 gate: str = "gate_proj.weight", up: str = "up_proj.weight", down: str = "down_proj.weight"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation must be one of {self.ACTIVATIONS}, found {activation!r}")
        self.prefix = prefix
        self.hidden = hidden
        self.intermediate = intermediate
        self.activation = activation
        self.gate_name, self.up_name, self.down_name = prefix + gate, prefix + up, prefix + down
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, i = self.hidden, self.intermediate
        return {
            self.gate_name: WeightSpec((i, h)),
            self.up_name: WeightSpec((i, h)),
            self.down_name: WeightSpec((h, i)),
        }

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.w_gate_up = runtime.weight([tensors[self.gate_name], tensors[self.up_name]], "gated", gated_n=self.intermediate)
        self.w_down = runtime.weight(tensors[self.down_name])

    def forward_into(self, h, batch, out: torch.Tensor) -> None:
        """The feed-forward's output into `out` (float32 [tokens, hidden]) instead of onto the residual stream: for a
        block that puts a norm between the two."""
        rt = self.runtime
        act = rt.empty((h.shape[0], self.intermediate))
        rt.ops.linear_glu(h, self.w_gate_up, act, activation=self.activation)
        rt.ops.linear(act, self.w_down, out)

    def forward(self, h, batch, residual: torch.Tensor, then=None):
        rt = self.runtime
        tokens = h.shape[0]
        act = rt.empty((tokens, self.intermediate))
        rt.ops.linear_glu(h, self.w_gate_up, act, activation=self.activation)
        return rt.ops.linear(act, self.w_down, residual, accumulate=True,
                             then_norm=None if then is None else then.row_scale())


class DenseMLP(FeedForward):
    """x + W_down act(W_up y), no gate and no biases. act: "silu", "tanh", or "xielu", which has two learnt numbers
    (p, q) in the tensor `act`: z > 0: softplus(p) z^2 + z / 2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2.
    The activation reads the product's float32 sums and rounds once, to the compute dtype."""
    capturable = True

    ACTIVATIONS = ("silu", "tanh", "xielu")

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "xielu",
                 up: str = "up", down: str = "down", act: Optional[str] = "act"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation must be one of {self.ACTIVATIONS}, found {activation!r}")
        self.hidden, self.intermediate, self.activation = hidden, intermediate, activation
        self.up_name, self.down_name = prefix + up, prefix + down
        self.act_name = prefix + act if activation == "xielu" else None
        self.w_up = self.w_down = self.act_params = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {self.up_name: WeightSpec((self.intermediate, self.hidden)),
                 self.down_name: WeightSpec((self.hidden, self.intermediate))}
        if self.act_name is not None:
            specs[self.act_name] = WeightSpec((2,), kind="vector")
        return specs

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.w_up = runtime.weight(tensors[self.up_name])
        self.w_down = runtime.weight(tensors[self.down_name])
        if self.act_name is not None:
            self.act_params = runtime.vector(tensors[self.act_name])

    def forward(self, h, batch, residual: torch.Tensor) -> None:
        rt = self.runtime
        sums = rt.empty((h.shape[0], self.intermediate), torch.float32)
        rt.ops.linear(h, self.w_up, sums)
        act = rt.empty((h.shape[0], self.intermediate))
        rt.ops.activation(sums, act, self.activation, self.act_params)
        rt.ops.linear(act, self.w_down, residual, accumulate=True)


register_part("feed_forward", "gated_mlp", GatedMLP)
register_part("feed_forward", "dense_mlp", DenseMLP)
