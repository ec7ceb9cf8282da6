"""Attention over one compressed row per position, without rotation.

Every position keeps a latent c = rmsnorm(W_dkv x) of ``kv_rank`` numbers, and nothing else.  Head h has matrices of its
own that would expand it, k_h = W_uk,h c and v_h = W_uv,h c; the score of query position i and key position j <= i is
(q_h,i . k_h,j) * scale, the softmax is the ordinary one, the concatenated heads are multiplied element by element by
sigmoid(W_g x) and go through the output product.

The keys and values are never expanded.  Since q . (W_uk c) = (W_uk^T q) . c, each head's key matrix is folded into its
query (one product per head, ``ops.head_gemm``), and since sum_j p_j W_uv c_j = W_uv sum_j p_j c_j, each head's value
matrix is applied to its weighted sum of latents afterwards (a second product per head, whose epilogue applies the output
gate).  In between runs the library's attention over the paged cache as for any mixer with one key/value head shared by
all query heads, of width ``kv_rank`` rounded up to a multiple of 16 (the added columns are zeros in the folded queries
and in the cache): the cache holds the latent as a key row and, transposed, as a value row, the layouts that the
attention kernels' operands take.  A prompt and a decoded token take the same path, so a position's result does not
depend on how its sequence was cut into steps.

``shares_latent``: the mixer has no W_dkv; its schedule entry reads the cache of an earlier entry (another layer's
latents, written earlier in the same step) with its own W_uk, W_uv, queries, gate and output product.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import CacheNeed, ParamSpec, Part, register_part
from .rope import NoRotation


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, kv_rank: int, scale: float,
                 eps: float, shares_latent: bool = False, gate_activation: str = "sigmoid"):
        if min(num_heads, head_dim, value_dim, kv_rank) < 1:
            raise ValueError("heads, widths and the latent's size must be positive")
        if kv_rank > 512:
            raise ValueError(f"a latent of {kv_rank} numbers is beyond the 512 that the attention kernels take as a head")
        if gate_activation not in ops.GATES:
            raise ValueError(f"unknown activation {gate_activation!r}; known: {', '.join(sorted(ops.GATES))}")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.kv_rank, self.scale, self.eps, self.shares_latent = kv_rank, float(scale), eps, shares_latent
        self.gate_activation = gate_activation
        self.width = -(-kv_rank // 16) * 16          # the latent's width in the cache and in the attention kernels
        for name in self.param_specs():
            setattr(self, name, None)
        self.in_weight = self.fold_weight = self.expand_weight = None      # made by prepare()
        self._no_rotation = NoRotation()

    def param_specs(self):
        H, K, V, R, W = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.hidden_size
        specs = {"q_weight": ParamSpec((H * K, W)), "uk_weight": ParamSpec((H * K, R)), "uv_weight": ParamSpec((H * V, R)),
                 "g_weight": ParamSpec((H * V, W)), "out_weight": ParamSpec((W, H * V))}
        if not self.shares_latent:
            specs.update({"dkv_weight": ParamSpec((R, W)), "dkv_norm": ParamSpec((R,), role="scale")})
        return specs

    def cache_need(self) -> CacheNeed:
        return CacheNeed(1, self.width)

    def state_need(self):
        return None

    def prepare(self, device, act):
        if self.in_weight is not None:
            return
        H, K, V, R, Rp = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.width
        first = [self.q_weight] + ([] if self.shares_latent else [self.dkv_weight]) + [self.g_weight]
        self.in_weight = torch.cat(first).contiguous()          # q | (latent) | gate: one product of the layer's input
        # W_uk,h^T [R, K] per head, rows R .. Rp - 1 zeros: the folded query's padding is zero
        fold = self.uk_weight.new_zeros((H, Rp, K))
        fold[:, :R] = self.uk_weight.view(H, K, R).transpose(1, 2)
        self.fold_weight = fold.contiguous()
        # W_uv,h [V, R] per head, columns R .. Rp - 1 zeros
        expand = self.uv_weight.new_zeros((H, V, Rp))
        expand[:, :, :R] = self.uv_weight.view(H, V, R)
        self.expand_weight = expand.contiguous()
        for name in ("q_weight", "dkv_weight", "g_weight", "uk_weight", "uv_weight"):
            setattr(self, name, None)

    def forward(self, normed, ctx, entry):
        b, kv = ctx.batch, ctx.kv(entry)
        H, K, V, R, Rp = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.width
        T = normed.shape[0]
        proj = ops.gemm(normed, self.in_weight, ctx.act)                    # float32 [T, q | (latent) | gate]
        q = proj[:, :H * K]
        gate = proj[:, proj.shape[1] - H * V:]
        if kv.owns != (not self.shares_latent):
            raise ValueError("a latent attention keeps a cache of its own exactly if it has a latent of its own")
        if kv.owns:
            # folded queries, then the normed latent twice (the key row and the value row), as the cache write reads them
            rows = torch.empty((T, (H + 2) * Rp), dtype=torch.float32, device=normed.device)
            ops.head_gemm(q, self.fold_weight, ctx.act, out=rows[:, :H * Rp])
            ops.latent_norm(proj[:, H * K:H * K + R], self.dkv_norm, self.eps, rows[:, H * Rp:], 2, Rp, ctx.act)
            folded = ops.rope_kv_write(rows, b.positions, b.slot_of_token, kv.table, self._no_rotation.table(ctx.device), 0, 0,
                                       kv.k_pages, kv.v_pages, kv.layer_offset, kv.page_size, kv.page_stride, H, 1, Rp,
                                       ctx.act, runs=b.runs())
        else:
            folded = ops.head_gemm(q, self.fold_weight, ctx.act, out_act=True)
        mixed = ops.attention(folded, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                              kv.page_size, kv.page_stride, H, 1, Rp, None, self.scale, ctx.act, runs=b.runs())
        out = ops.head_gemm(mixed, self.expand_weight, ctx.act, out_act=True, gate=gate, activation=self.gate_activation)
        return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)
