"""Linear attention with a per-head decay and a matrix state per request (no reference counterpart).

    q, k = silu(W_q h), silu(W_k h)  [heads, dim];   v = silu(W_v h)  [heads, vdim]
    S_t = decay[h] * S_(t-1) + k_t v_t^T;            o_t = S_t^T q_t
    out = W_o ( norm(concat_h o_t) * sigmoid(W_g h) )

The state S [heads, dim, vdim] is float, starts at zero and lives in the request's state slot between
steps; nothing is kept per token.  One product makes q, k, v and the gate; the activation is applied
where the recurrence kernel loads them; the recurrence's output stays float until its norm.
"""
from __future__ import annotations

from typing import Sequence

import torch

from ..ops import kernels as K
from .spec import LayerMemory, StateSpec, StepContext, TensorSpec, register_part


class LightningAttention:
    replayable = True     # slots, request borders and tokens come from the device; the kernel choice does not depend on values

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_dim: int, decay: Sequence[float],
                 norm_eps: float):
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(num_heads), int(head_dim), int(v_dim)
        self.decay_values = [float(d) for d in decay]
        if len(self.decay_values) != self.heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.heads} heads")
        self.eps = float(norm_eps)

    def tensors(self) -> dict:
        H, hid = self.heads, self.hidden_size
        return {
            "q_proj.weight": TensorSpec((H * self.dim, hid)),
            "k_proj.weight": TensorSpec((H * self.dim, hid)),
            "v_proj.weight": TensorSpec((H * self.vdim, hid)),
            "gate.weight": TensorSpec((H * self.vdim, hid)),
            "o_proj.weight": TensorSpec((hid, H * self.vdim)),
            "norm.weight": TensorSpec((H * self.vdim,), role="vector", init="norm"),
        }

    def cache_spec(self):
        return None

    def state_spec(self):
        return StateSpec((self.heads, self.dim, self.vdim), "float32")

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        self.w_in = torch.cat([tensors[k + ".weight"] for k in ("q_proj", "k_proj", "v_proj", "gate")], dim=0).contiguous()
        self.w_o, self.norm_weight = tensors["o_proj.weight"], tensors["norm.weight"]
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.w_o.device)

    def forward(self, x, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        H, d, dv = self.heads, self.dim, self.vdim
        proj = K.linear(x, self.w_in)
        plan = None
        if not ctx.captured and ctx.max_q_len >= K.LIGHTNING_CHUNK_MIN_TOKENS and K.lightning_chunks_possible(d):
            # prompt portions: chunks side by side (the list of chunks is the same for every such layer of the step)
            plan = ctx.plans.get("lightning_chunks")
            if plan is None:
                plan = ctx.plans["lightning_chunks"] = K.lightning_chunk_plan(ctx.q_lens_host, x.device)
        o = K.lightning_attention(proj, 0, H * d, 2 * H * d, mem.state, ctx.slot_ids, ctx.cu_seqlens, self.decay,
                                  H, d, dv, plan)
        y = K.gated_rmsnorm(o, proj[:, 2 * H * d + H * dv:], self.norm_weight, self.eps)
        return K.linear(y, self.w_o, partial_ok=True)


register_part("mixer", "lightning_attention", LightningAttention)
