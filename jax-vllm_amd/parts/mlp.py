"""Gated feed-forward.  Reference: ``jllm/model/common.py:69-76``:
``down( silu(gate(x)) * up(x) )``, no biases (SwiGLU); the gate's activation is a parameter, one
of ``ops.kernels.GATE_ACTIVATIONS``.  gate and up are one matrix product against
one weight whose rows alternate gate row j, up row j, so that a gate value and its up value
come out next to each other: for few rows the activation is that product's epilogue, for
many rows a kernel over adjacent pairs.  The activation runs in float."""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class GatedMLP:
    replayable = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"GatedMLP has kernels for {sorted(K.GATE_ACTIVATIONS)}, not for {activation!r}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.w_gate_up = self.w_down = None
        self.partial_out = True     # whether the result may be a float stack of partial products (the next norm adds them)

    def tensors(self) -> dict:
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": TensorSpec((i, h)),
            "up_proj.weight": TensorSpec((i, h)),
            "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        self.w_gate_up = torch.stack([g, u], dim=1).reshape(2 * g.shape[0], g.shape[1]).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def takes_unscaled_rows(self, n_rows: int) -> bool:
        """x goes into the gate/up product and nowhere else: the norm before may leave its scale to that product."""
        return K.linear_takes_unscaled_rows(n_rows, self.w_gate_up, gate_pairs=True)

    def forward(self, x, ctx=None) -> torch.Tensor:
        z = K.linear(x, self.w_gate_up, gate_pairs=self.activation)    # gate and up rows alternate in the fused weight
        return K.linear(z, self.w_down, partial_ok=self.partial_out)   # the next norm adds the partial products


class DenseMLP:
    """A feed-forward without a gate: ``down( act(up(x) + b_up) ) + b_down``; the activation is one of
    ``ops.kernels.PLAIN_ACTIVATIONS`` ("gelu" is the erf form), computed in float; the biases are optional."""

    replayable = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu", bias: bool = True):
        if activation not in K.PLAIN_ACTIVATIONS or activation is None:
            raise ValueError(f"DenseMLP has kernels for {sorted(a for a in K.PLAIN_ACTIVATIONS if a)}, not for {activation!r}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation, self.bias = activation, bool(bias)
        self.w_up = self.w_down = self.b_up = self.b_down = None

    def tensors(self) -> dict:
        h, i = self.hidden_size, self.intermediate_size
        t = {"up_proj.weight": TensorSpec((i, h)), "down_proj.weight": TensorSpec((h, i))}
        if self.bias:
            t["up_proj.bias"] = TensorSpec((i,), role="vector")
            t["down_proj.bias"] = TensorSpec((h,), role="vector")
        return t

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.w_up, self.w_down = tensors["up_proj.weight"], tensors["down_proj.weight"]
        if self.bias:
            self.b_up, self.b_down = tensors["up_proj.bias"], tensors["down_proj.bias"]

    def forward(self, x, ctx=None) -> torch.Tensor:
        z = K.linear(x, self.w_up)
        K.bias_act(z, self.b_up, self.activation)
        y = K.linear(z, self.w_down, partial_ok=True)       # the next norm adds the partial products
        # the second bias is left to whoever takes the output: a block that norms it adds the bias in that kernel
        return K.BiasedOutput(y, self.b_down) if self.b_down is not None else y


register_part("feed_forward", "gated_mlp", GatedMLP)
register_part("feed_forward", "dense_mlp", DenseMLP)
