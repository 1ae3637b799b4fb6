"""Softmax attention whose keys and values are expanded from one small latent vector per token.

Per token the layer projects ``heads`` queries, each ``[plain (P) | turned (R)]``, and one vector
``[latent (C) | turned key part (R)]``.  The latent is RMS-normed (with a weight); head h's plain key is
``W_uk[h] c`` and its value ``W_uv[h] c``; the turned key part is shared by all heads; queries' and the key's turned
parts rotate with the position.  The score of query t and key j is ``(q_plain . k_plain + q_turned . k_turned) * scale``
over all ``j <= t``, softmax; the heads' outputs are multiplied by ``sigmoid(W_g x)`` and projected by ``W_o``.

Only the normed latent and the turned key part are cached, and the expansions are never applied to the cache:
since ``q_plain . (W_uk[h] c) = (W_uk[h]^T q_plain) . c``, a query is folded into the latent space once, and since
``sum_j p_j W_uv[h] c_j = W_uv[h] sum_j p_j c_j`` the value expansion is applied once to the head's weighted sum of
latents.  To the paged attention kernels this is one key head of ``R + C`` numbers (padded to a head size they take)
shared by all query heads, whose value is the cache entry itself: the layer reuses them as they are, in both
precisions.  The per-head folding and unfolding are block-diagonal products (``ops.block_linear``).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.manager import PagedKV
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.tensors import TensorSpec
from .attention import attend
from .base import Part, build_part, register_part
from .linear import linear


def positions_bound(batch) -> int:
    """Positions a step's rotation tables have to reach: its longest context, or, for a step that is captured and
    replayed with other contexts, the bound it was captured for."""
    return batch.static_plan.max_keys if batch.static_plan is not None else batch.max_context


class LatentAttention(Part):
    graph_safe = True  # (a captured step's rotation tables reach the bound the step was captured for)

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 scale: float, eps: float, position: PartSpec) -> None:
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim),
                            ("value_dim", value_dim), ("kv_rank", kv_rank)):
            if value < 1:
                raise ValueError(f"{name} must be positive, got {value}")
        if rot_dim < 0 or rot_dim % 2:
            raise ValueError(f"the turned part of a head must be even, got {rot_dim}")
        if not scale > 0 or not eps > 0:
            raise ValueError("scale and eps must be positive")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.rot_dim = rot_dim
        self.value_dim = value_dim
        self.kv_rank = kv_rank
        self.scale = float(scale)
        self.eps = float(eps)
        self.position = build_part("position", position)
        entry = rot_dim + kv_rank
        # the cache entry is as wide as a head of the attention kernels: the next size their matrix-core forms take
        self.entry_dim = next((size for size in ops.MFMA_HEAD_DIMS if size >= entry), None)
        if self.entry_dim is None:
            raise ValueError(f"a cache entry of {entry} numbers is more than the attention kernels' {ops.MFMA_HEAD_DIMS[-1]}")

    def cache_need(self) -> PagedKV:
        return PagedKV(1, self.entry_dim, None)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, p, r, v, c, hidden = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank, self.hidden_size
        return {
            prefix + "q": TensorSpec((h * (p + r), hidden)),
            prefix + "dkv": TensorSpec((c + r, hidden)),
            prefix + "dkv.norm": TensorSpec((c,), init="norm", keeps_float32=True),
            prefix + "uk": TensorSpec((h * p, c)),
            prefix + "uv": TensorSpec((h * v, c)),
            prefix + "g": TensorSpec((h * v, hidden)),
            prefix + "o": TensorSpec((hidden, h * v)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        h, p, r, v, c = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank
        self.w_in = torch.cat([tensors[prefix + "q"], tensors[prefix + "dkv"], tensors[prefix + "g"]], dim=0).contiguous()
        self.latent_weight = tensors[prefix + "dkv.norm"].contiguous()
        # fold: [heads, C, P] so that (q_plain of head h) @ fold[h].T lies in the latent space
        self.w_fold = tensors[prefix + "uk"].reshape(h, p, c).transpose(1, 2).contiguous()
        # unfold: [heads, V, entry] reads the latent part of a head's weighted sum of cache entries
        unfold = torch.zeros((h, v, self.entry_dim), dtype=dtype, device=device)
        unfold[:, :, r: r + c] = tensors[prefix + "uv"].reshape(h, v, c)
        self.w_unfold = unfold.contiguous()
        self.w_o = tensors[prefix + "o"].contiguous()

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        h, p, r, c, width = self.num_heads, self.head_dim, self.rot_dim, self.kv_rank, self.entry_dim
        if batch.max_context > self.position.max_position and self.position.rotates:
            raise ValueError(f"position {batch.max_context - 1} is beyond the rotary table of {self.position.max_position}")
        queries = h * (p + r)
        proj = linear(x, self.w_in)
        rows = ops.latent_rows(proj[:, : queries + c + r], self.latent_weight, h, p, r, c, width, self.eps)
        ops.block_linear(proj, self.w_fold, a_block=p + r, out=rows, out_offset=r, c_block=width)
        turns = bool(r) and self.position.rotates
        cos, sin = self.position.tables(x.device, positions_bound(batch))
        ops.rope_kv_write(rows, cos, sin, batch.positions, batch.seq_of_token, batch.seq_slot, view.block_table,
                          view.k_pool, view.v_pool, h, 1, width, rotate=turns, write_kv=writes,
                          rotary_dim=r if turns else None)
        context = attend(rows, batch, view, h, 1, width, None, self.scale)
        gated = ops.block_linear(context, self.w_unfold, gate=proj, gate_offset=queries + c + r)
        return linear(gated, self.w_o)


register_part("mixer", "latent_attention", LatentAttention)
