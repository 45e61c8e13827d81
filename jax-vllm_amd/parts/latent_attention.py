"""Attention through a low-rank latent, over a paged cache of that latent (no reference counterpart).

A token's keys and values of ALL heads are functions of one vector per token:

    c      = norm(W_dkv h)[:rank]                       the latent, cached
    k_rot  = rotate(W_dkv h [rank:])                    one rotated key part shared by the heads, cached
    k[h]   = [W_uk[h] c | k_rot],   v[h] = W_uv[h] c
    q[h]   = W_uq[h] norm(W_dq h) = [q_plain | q_rot], q_rot rotated
    score  = (q_plain . W_uk[h] c + q_rot . k_rot) * scale,   causal, optionally a sliding window
    out    = W_o ( concat_h(softmax . v[h]) * sigmoid(W_g h) )      (the gate is an option)

Since q_plain . (W_uk[h] c) = (W_uk[h]^T q_plain) . c and sum_j p_j W_uv[h] c_j = W_uv[h] sum_j p_j c_j,
the cached vector e = [c | k_rot] serves as key AND value of one shared kv head of size rank + rot: the
paged attention kernels of grouped-query attention run unchanged (one kv head, ``heads`` q heads), on a
query [W_uk[h]^T q_plain | q_rot], and W_uv[h] is applied to the first ``rank`` elements of their result.
The same arithmetic serves prompts and decoded tokens, so logits do not depend on how a prompt is cut.
The cache keeps e in the two layouts those kernels read (``parts.spec.kv_cache_spec``).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .spec import LayerMemory, PagedCacheSpec, PartSpec, StepContext, TensorSpec, build_part, is_replayable, kv_cache_spec, register_part


class LatentAttention:
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, v_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, position: Optional[PartSpec] = None,
                 window: Optional[int] = None, output_gate: bool = True):
        self.hidden_size, self.heads = int(hidden_size), int(num_heads)
        self.dim, self.rot, self.vdim = int(head_dim), int(rot_dim), int(v_dim)
        self.q_rank, self.rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(norm_eps)
        self.window = int(window) if window else None
        self.output_gate = bool(output_gate)
        self.position = build_part("position", position) if position is not None and self.rot else None
        rotation = self.position.as_rotation() if self.position is not None else None
        if rotation is not None and rotation[1]:
            raise ValueError("the latent attention kernels rotate half-split pairs (i, i + dims/2) only")
        self.rot_dims = int(rotation[0]) if rotation is not None else 0
        if self.rot_dims > self.rot:
            raise ValueError(f"{self.rot_dims} rotated dimensions do not fit a key part of {self.rot}")
        # what the paged attention kernels see: one kv head of the cached vector's size
        self.nq, self.nkv, self.d = self.heads, 1, self.rank + self.rot
        self.q_row_stride = self.heads * self.d

    @property
    def replayable(self) -> bool:
        return self.position is None or is_replayable(self.position)

    def tensors(self) -> dict:
        H, hid = self.heads, self.hidden_size
        t = {
            "q_down.weight": TensorSpec((self.q_rank, hid)),
            "q_norm.weight": TensorSpec((self.q_rank,), role="vector", init="norm"),
            "q_up.weight": TensorSpec((H * (self.dim + self.rot), self.q_rank)),
            "kv_down.weight": TensorSpec((self.rank + self.rot, hid)),
            "kv_norm.weight": TensorSpec((self.rank,), role="vector", init="norm"),
            "k_up.weight": TensorSpec((H * self.dim, self.rank)),
            "v_up.weight": TensorSpec((H * self.vdim, self.rank)),
            "o_proj.weight": TensorSpec((hid, H * self.vdim)),
        }
        if self.output_gate:
            t["gate.weight"] = TensorSpec((H * self.vdim, hid))
        return t

    def cache_spec(self) -> Optional[PagedCacheSpec]:
        return kv_cache_spec(1, self.d, self.window)

    def state_spec(self):
        return None

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        H = self.heads
        down = [tensors["q_down.weight"], tensors["kv_down.weight"]]
        if self.output_gate:
            down.append(tensors["gate.weight"])
        self.w_down = torch.cat(down, dim=0).contiguous()       # one product for everything that reads the input
        self.gate_at = self.q_rank + self.rank + self.rot
        self.q_norm, self.kv_norm = tensors["q_norm.weight"], tensors["kv_norm.weight"]
        self.w_q_up = tensors["q_up.weight"]
        self.w_k_up_t = tensors["k_up.weight"].view(H, self.dim, self.rank).transpose(1, 2).contiguous()   # [H, rank, dim]
        self.w_v_up = tensors["v_up.weight"].view(H, self.vdim, self.rank).contiguous()
        self.w_o = tensors["o_proj.weight"]
        if self.position is not None:
            self.position.bind({}, dtype, self.w_o.device)

    def forward(self, x, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        n, H, E = x.shape[0], self.heads, self.d
        cos_sin = self.position.rotation_table(ctx) if self.rot_dims else None
        proj = K.linear(x, self.w_down)
        writes = mem.writes
        cq = K.latent_prepare(proj, self.q_rank, self.rank, self.rot, self.rot_dims, self.q_norm, self.kv_norm, self.eps,
                              cos_sin, ctx.slot_mappings[mem.group] if writes else None,
                              mem.pages["k"] if writes else None, mem.pages["v"] if writes else None, ctx.page_size)
        q = K.linear(cq, self.w_q_up)
        qe = torch.empty((n, H * E), dtype=x.dtype, device=x.device)
        K.head_linear(qe, E, q, self.dim + self.rot, self.w_k_up_t)             # W_uk[h]^T q_plain
        if self.rot:
            K.latent_query_rope(q, qe, H, self.dim, self.rot, self.rot_dims, self.rank, cos_sin)
        att = torch.empty((n, H * E), dtype=x.dtype, device=x.device)
        from . import attention_backend

        attention_backend.run(self, att, qe, ctx, mem)
        o = torch.empty((n, H * self.vdim), dtype=x.dtype, device=x.device)
        K.head_linear(o, self.vdim, att, E, self.w_v_up, gate=proj[:, self.gate_at:] if self.output_gate else None)
        return K.linear(o, self.w_o, partial_ok=True)


register_part("mixer", "latent_attention", LatentAttention)
