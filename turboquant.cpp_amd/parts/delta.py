"""Recurrent mixers: the gated delta rule with one decay per head and key channel (``ChannelDeltaRule``), and with one decay
per head (``HeadDeltaRule``, at the end of this file).

Per head, a state S [dim, vdim] that starts at zero and is carried from token to token of a sequence:

    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

q and k ([kv_heads, dim]) and v ([heads, vdim]) are projections without bias that pass a short causal convolution over
time, one filter per channel (zeros before the start, the last tap is the current token's), and silu; q and k are
then scaled to unit length per head (x / sqrt(sum x^2 + 1e-6)), q also by dim^-1/2.  Head h reads q/k head
h // (heads / kv_heads).  beta = sigmoid(W_b x) per head; g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 x) + dt_bias)) per
head and key channel.  Each head's o is divided by its root mean square over vdim (``eps``), multiplied by a weight
per value channel (shared by the heads) and by sigmoid(W_g2 (W_g1 x)), and the heads go through the output product.

The sequence's state is one row of float32 per slot (``StateNeed``): S, then the convolution's last taps - 1 inputs of
every channel.  Decays, gates, norms and the recurrence are float32 on both libraries; the products are the
activation type's.  Six launches a prompt step: the product of all first projections, ``delta_prep``, the second product
of decay and gate (one product over a block-diagonal matrix of both), ``delta_scan`` (which, in a step of many tokens,
first works out all decays in a launch of their own), ``delta_out``, the output product.  Four a decode step:
``delta_decode`` stands for the three in the middle.
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import ParamSpec, Part, StateNeed, register_part


@register_part("mixer", "channel_delta")
class ChannelDeltaRule(Part):
    graph_safe = True       # what changes from step to step is read from the batch's device arrays only

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, conv_taps: int,
                 rank_a: int, rank_g: int, eps: float):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"a key width of {head_dim} is beyond the 256 that the recurrence's kernel takes")
        if not 1 <= conv_taps <= 64:
            raise ValueError(f"{conv_taps} taps are beyond the 64 that the convolution's kernel takes")
        self.hidden_size, self.eps = hidden_size, eps
        self.dims = ops.DeltaDims(num_heads, num_kv_heads, head_dim, value_dim, conv_taps, rank_a, rank_g)
        for name in self.param_specs():
            setattr(self, name, None)
        self.in_weight = self.low_weight = self.conv = None     # made by prepare()

    def param_specs(self):
        d, W = self.dims, self.hidden_size
        qk, v = d.kv_heads * d.dim, d.heads * d.vdim
        return {
            "q_weight": ParamSpec((qk, W)), "k_weight": ParamSpec((qk, W)), "v_weight": ParamSpec((v, W)),
            "q_conv": ParamSpec((qk, d.taps), role="scale"), "k_conv": ParamSpec((qk, d.taps), role="scale"),
            "v_conv": ParamSpec((v, d.taps), role="scale"),
            "b_weight": ParamSpec((d.heads, W)),
            "a1_weight": ParamSpec((d.rank_a, W)), "a2_weight": ParamSpec((d.heads * d.dim, d.rank_a)),
            "g1_weight": ParamSpec((d.rank_g, W)), "g2_weight": ParamSpec((v, d.rank_g)),
            "a_log": ParamSpec((d.heads,), role="scale"), "dt_bias": ParamSpec((d.heads * d.dim,), role="bias"),
            "out_norm": ParamSpec((d.vdim,), role="scale"),
            "out_weight": ParamSpec((W, v)),
        }

    def cache_need(self):
        return None

    def state_need(self) -> StateNeed:
        return StateNeed((self.dims.state_floats,), torch.float32)

    def prepare(self, device, act):
        if self.in_weight is not None:
            return
        d = self.dims
        # all products of the layer's input as one, and the two second products as one over a block-diagonal matrix
        # (its zeros add nothing to any sum)
        self.in_weight = torch.cat([self.q_weight, self.k_weight, self.v_weight, self.b_weight, self.a1_weight,
                                    self.g1_weight]).contiguous()
        a2, g2 = self.a2_weight, self.g2_weight
        low = a2.new_zeros((a2.shape[0] + g2.shape[0], d.rank_a + d.rank_g))
        low[:a2.shape[0], :d.rank_a] = a2
        low[a2.shape[0]:, d.rank_a:] = g2
        self.low_weight = low
        # what enters float arithmetic only
        self.conv = torch.cat([self.q_conv, self.k_conv, self.v_conv]).float().contiguous()
        self.a_log, self.dt_bias = self.a_log.float().contiguous(), self.dt_bias.float().contiguous()
        self.out_norm = self.out_norm.float().contiguous()
        for name in ("q_weight", "k_weight", "v_weight", "b_weight", "a1_weight", "g1_weight", "a2_weight", "g2_weight",
                     "q_conv", "k_conv", "v_conv"):
            setattr(self, name, None)

    def forward(self, normed, ctx, entry):
        b, d = ctx.batch, self.dims
        state = ctx.state(entry)
        runs = b.runs()
        proj = ops.gemm(normed, self.in_weight, ctx.act)
        qn, kn, vc, beta, low = ops.delta_prep(proj, b.slot_of_token, state, self.conv, d, ctx.act)
        if b.is_decode and ops.delta_decode_fits(d):
            # one token per sequence: second products, decays, recurrence, norm, gate and new convolution state in one launch
            out = ops.delta_decode(qn, kn, vc, beta, low, self.low_weight, self.a_log, self.dt_bias, self.out_norm, self.eps,
                                   proj, runs, state, d, ctx.act)
            return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)
        ag = ops.gemm(low, self.low_weight, ctx.act)
        o = ops.delta_scan(qn, kn, vc, beta, ag, self.a_log, self.dt_bias, runs, state, d, ctx.act)
        out = ops.delta_out(o, ag, self.out_norm, self.eps, proj, runs, state, d, ctx.act)
        return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)


@register_part("mixer", "head_delta")
class HeadDeltaRule(Part):
    """The gated delta rule with one decay per head: the recurrence, convolutions, unit lengths and beta of
    :class:`ChannelDeltaRule`, with

        g = exp(-exp(A_log_h) softplus(W_a x + dt_bias_h))      one number per head and token,

    which scales the head's whole state before the token's write, and a gate that is a full projection: each head's
    read-out is divided by its root mean square over vdim (``eps``), multiplied by a weight per value channel (shared by
    the heads) and by ``gate_activation`` of W_g x (``silu`` or ``sigmoid``), and the heads go through the output product.

    The state is laid out as there.  Five launches a prompt step: the product of all projections (q, k, v, b, a, gate:
    one matrix), ``delta_prep_h`` (which also works out the decays), ``delta_scan_h``, ``delta_out_h``, the output
    product; four a decode step, ``delta_decode_h`` standing for the two in the middle.
    """
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, conv_taps: int,
                 eps: float, gate_activation: str = "silu"):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"a key width of {head_dim} is beyond the 256 that the recurrence's kernel takes")
        if not 1 <= conv_taps <= 64:
            raise ValueError(f"{conv_taps} taps are beyond the 64 that the convolution's kernel takes")
        if gate_activation not in ops.GATES:
            raise ValueError(f"unknown activation {gate_activation!r}; known: {', '.join(sorted(ops.GATES))}")
        self.hidden_size, self.eps, self.gate_activation = hidden_size, eps, gate_activation
        self.dims = ops.DeltaDims(num_heads, num_kv_heads, head_dim, value_dim, conv_taps, 0, 0, head_decay=True)
        for name in self.param_specs():
            setattr(self, name, None)
        self.in_weight = self.conv = None     # made by prepare()

    def param_specs(self):
        d, W = self.dims, self.hidden_size
        qk, v = d.kv_heads * d.dim, d.heads * d.vdim
        return {
            "q_weight": ParamSpec((qk, W)), "k_weight": ParamSpec((qk, W)), "v_weight": ParamSpec((v, W)),
            "q_conv": ParamSpec((qk, d.taps), role="scale"), "k_conv": ParamSpec((qk, d.taps), role="scale"),
            "v_conv": ParamSpec((v, d.taps), role="scale"),
            "b_weight": ParamSpec((d.heads, W)), "a_weight": ParamSpec((d.heads, W)), "g_weight": ParamSpec((v, W)),
            "a_log": ParamSpec((d.heads,), role="scale"), "dt_bias": ParamSpec((d.heads,), role="bias"),
            "out_norm": ParamSpec((d.vdim,), role="scale"),
            "out_weight": ParamSpec((W, v)),
        }

    def cache_need(self):
        return None

    def state_need(self) -> StateNeed:
        return StateNeed((self.dims.state_floats,), torch.float32)

    def prepare(self, device, act):
        if self.in_weight is not None:
            return
        self.in_weight = torch.cat([self.q_weight, self.k_weight, self.v_weight, self.b_weight, self.a_weight,
                                    self.g_weight]).contiguous()
        # what enters float arithmetic only
        self.conv = torch.cat([self.q_conv, self.k_conv, self.v_conv]).float().contiguous()
        self.a_log, self.dt_bias = self.a_log.float().contiguous(), self.dt_bias.float().contiguous()
        self.out_norm = self.out_norm.float().contiguous()
        for name in ("q_weight", "k_weight", "v_weight", "b_weight", "a_weight", "g_weight", "q_conv", "k_conv", "v_conv"):
            setattr(self, name, None)

    def forward(self, normed, ctx, entry):
        b, d = ctx.batch, self.dims
        state = ctx.state(entry)
        runs = b.runs()
        proj = ops.gemm(normed, self.in_weight, ctx.act)
        qn, kn, vc, beta, dec = ops.delta_prep_h(proj, b.slot_of_token, state, self.conv, self.a_log, self.dt_bias, d, ctx.act)
        if b.is_decode and ops.delta_decode_fits(d):
            out = ops.delta_decode_h(qn, kn, vc, beta, self.a_log, self.dt_bias, self.out_norm, self.eps, proj,
                                     self.gate_activation, runs, state, d, ctx.act)
        else:
            o = ops.delta_scan_h(qn, kn, vc, beta, dec, runs, state, d, ctx.act)
            out = ops.delta_out_h(o, self.out_norm, self.eps, proj, self.gate_activation, runs, state, d, ctx.act)
        return ops.gemm(out, self.out_weight, ctx.act, partial_sums=True)
