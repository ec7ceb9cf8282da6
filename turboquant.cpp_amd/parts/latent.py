"""Attention over one compressed row per position, without rotation.

Every position keeps a latent c = rmsnorm(W_dkv x) of ``kv_rank`` numbers, and nothing else.  Head h has matrices of its
own that would expand it, k_h = W_uk,h c and v_h = W_uv,h c; the score of query position i and key position j <= i is
(q_h,i . k_h,j) * scale, the softmax is the ordinary one, the concatenated heads are multiplied element by element by
sigmoid(W_g x) and go through the output product.

In the folded form the keys and values are never expanded.  Since q . (W_uk c) = (W_uk^T q) . c, each head's key matrix is folded into its
query (one product per head, ``ops.head_gemm``), and since sum_j p_j W_uv c_j = W_uv sum_j p_j c_j, each head's value
matrix is applied to its weighted sum of latents afterwards (a second product per head, whose epilogue applies the output
gate).  In between runs the library's attention over the paged cache as for any mixer with one key/value head shared by
all query heads, of width ``kv_rank`` rounded up to a multiple of 16 (the added columns are zeros in the folded queries
and in the cache): the cache holds the latent as a key row and, transposed, as a value row, the layouts that the
attention kernels' operands take.  Decoded tokens and portions of prompts that go on from earlier tokens take this form:
it reads ``kv_rank`` numbers per position whatever the number of heads.

A step whose sequences all start at their first token takes the other, expanded form, since per pair of positions the folded form
costs heads x 2 ``kv_rank`` multiply-adds and the expanded one heads x (dim + vdim): one product expands the step's
latents into every head's keys and values, which are laid into pages that live for the step only
(``StepBatch.own_pages``), and the library's attention runs over them with as many key/value heads as heads; the output
gate is applied to its result.  The latents go into the cache all the same, for the steps that follow.  Both forms are
the same function of the same rounded latents; they differ in the rounding of what comes after.

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
        if max(head_dim, value_dim) > 512:
            raise ValueError(f"heads of {max(head_dim, value_dim)} are beyond the 512 that the attention kernels take")
        if gate_activation not in ops.GATES:
            raise ValueError(f"unknown activation {gate_activation!r}; known: {', '.join(sorted(ops.GATES))}")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.kv_rank, self.scale, self.eps, self.shares_latent = kv_rank, float(scale), eps, shares_latent
        self.gate_activation = gate_activation
        self.width = -(-kv_rank // 16) * 16          # the latent's width in the cache and in the attention kernels
        # the width at which a head's queries, gates and outputs are laid out: the expanded form's attention has keys and
        # values of one width, a multiple of 16; the added rows and columns of the matrices are zeros
        self.head_width = -(-max(head_dim, value_dim) // 16) * 16
        for name in self.param_specs():
            setattr(self, name, None)
        self.in_weight = self.fold_weight = self.expand_weight = self.kv_weight = None      # made by prepare()
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
        H, K, V, R, Rp, D = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.width, self.head_width

        def heads_padded(t, n):          # [H * n, ...] -> [H * D, ...], rows n .. D - 1 of every head zeros
            if n == D:
                return t
            out = t.new_zeros((H, D) + tuple(t.shape[1:]))
            out[:, :n] = t.view(H, n, *t.shape[1:])
            return out.view(H * D, *t.shape[1:])

        first = [heads_padded(self.q_weight, K)] + ([] if self.shares_latent else [self.dkv_weight]) + [heads_padded(self.g_weight, V)]
        self.in_weight = torch.cat(first).contiguous()          # q | (latent) | gate: one product of the layer's input
        # W_uk,h^T [R, K] per head, rows R .. Rp - 1 and columns K .. D - 1 zeros: the folded query's padding is zero
        fold = self.uk_weight.new_zeros((H, Rp, D))
        fold[:, :R, :K] = self.uk_weight.view(H, K, R).transpose(1, 2)
        self.fold_weight = fold.contiguous()
        # W_uv,h [V, R] per head, rows V .. D - 1 and columns R .. Rp - 1 zeros
        expand = self.uv_weight.new_zeros((H, D, Rp))
        expand[:, :V, :R] = self.uv_weight.view(H, V, R)
        self.expand_weight = expand.contiguous()
        # every head's keys, then every head's values, from a latent: [2 H D, Rp]
        kv = self.uk_weight.new_zeros((2, H, D, Rp))
        kv[0, :, :K, :R] = self.uk_weight.view(H, K, R)
        kv[1, :, :V, :R] = self.uv_weight.view(H, V, R)
        self.kv_weight = kv.view(2 * H * D, Rp).contiguous()
        if V != D:
            out = self.out_weight.new_zeros((self.hidden_size, H, D))
            out[:, :, :V] = self.out_weight.view(self.hidden_size, H, V)
            self.out_weight = out.view(self.hidden_size, H * D).contiguous()
        for name in ("q_weight", "dkv_weight", "g_weight", "uk_weight", "uv_weight"):
            setattr(self, name, None)

    def forward(self, normed, ctx, entry):
        b, kv = ctx.batch, ctx.kv(entry)
        H, R, Rp, D = self.num_heads, self.kv_rank, self.width, self.head_width
        T = normed.shape[0]
        proj = ops.gemm(normed, self.in_weight, ctx.act)                    # float32 [T, q | (latent) | gate]
        q = proj[:, :H * D]
        gate = proj[:, proj.shape[1] - H * D:]
        if kv.owns != (not self.shares_latent):
            raise ValueError("a latent attention keeps a cache of its own exactly if it has a latent of its own")
        no_angles = self._no_rotation.table(ctx.device)
        if not b.is_decode and b.is_fresh and not ctx.capturing:
            return self._expanded(proj, q, gate, ctx, kv, no_angles)
        if kv.owns:
            # folded queries, then the normed latent twice (the key row and the value row), as the cache write reads them
            rows = torch.empty((T, (H + 2) * Rp), dtype=torch.float32, device=normed.device)
            ops.head_gemm(q, self.fold_weight, ctx.act, out=rows[:, :H * Rp])
            ops.latent_norm(proj[:, H * D:H * D + R], self.dkv_norm, self.eps, rows[:, H * Rp:], 2, Rp, ctx.act)
            folded = ops.rope_kv_write(rows, b.positions, b.slot_of_token, kv.table, no_angles, 0, 0,
                                       kv.k_pages, kv.v_pages, kv.layer_offset, kv.page_size, kv.page_stride, H, 1, Rp,
                                       ctx.act, runs=b.runs())
        else:
            folded = ops.head_gemm(q, self.fold_weight, ctx.act, out_act=True)
        mixed = ops.attention(folded, kv.k_pages, kv.v_pages, kv.layer_offset, b.positions, b.slot_of_token, kv.table,
                              kv.page_size, kv.page_stride, H, 1, Rp, None, self.scale, ctx.act, runs=b.runs())
        out = ops.head_gemm(mixed, self.expand_weight, ctx.act, out_act=True, gate=gate, activation=self.gate_activation)
        return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)

    def _expanded(self, proj, q, gate, ctx, kv, no_angles):
        """A step of whole prompts: every head's keys and values from the step's latents, in pages of the step's own."""
        b = ctx.batch
        H, R, Rp, D = self.num_heads, self.kv_rank, self.width, self.head_width
        T = proj.shape[0]
        runs = b.runs()
        shared = ("latents", kv.k_pages.data_ptr(), kv.layer_offset)     # the same for every entry that reads this cache
        if kv.owns:
            rows = torch.empty((T, 2 * Rp), dtype=torch.float32, device=proj.device)
            ops.latent_norm(proj[:, H * D:H * D + R], self.dkv_norm, self.eps, rows, 2, Rp, ctx.act)
            ops.rope_kv_write(rows, b.positions, b.slot_of_token, kv.table, no_angles, 0, 0, kv.k_pages, kv.v_pages,
                              kv.layer_offset, kv.page_size, kv.page_stride, 0, 1, Rp, ctx.act, runs=runs)
            latents = b.scratch[shared] = ops.act_rows(rows[:, :Rp], None, None, ctx.act)       # as the cache holds them
        else:
            latents = b.scratch[shared]
        table, n_pages = b.own_pages(kv.page_size)
        stride = H * kv.page_size * D
        # (cleared: a page's places behind a sequence's last token are multiplied by weights of zero, and must be numbers)
        pages = torch.zeros((2, n_pages, stride), dtype=latents.dtype, device=proj.device)
        ops.rope_kv_write(ops.gemm(latents, self.kv_weight, ctx.act), b.positions, b.slot_of_token, table, no_angles, 0, 0,
                          pages[0], pages[1], 0, kv.page_size, stride, 0, H, D, ctx.act, runs=runs)
        mixed = ops.attention(ops.act_rows(q, None, None, ctx.act), pages[0], pages[1], 0, b.positions, b.slot_of_token, table,
                              kv.page_size, stride, H, H, D, None, self.scale, ctx.act, runs=runs)
        return ops.gemm(ops.gate_rows(mixed, gate, self.gate_activation, ctx.act), self.out_weight, ctx.act, partial_sums=True)
