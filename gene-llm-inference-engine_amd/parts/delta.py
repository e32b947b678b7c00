"""The gated delta rule as a mixer (`config.spec.GatedDeltaSpec` states the recurrence; the kernels are `csrc/recurrent.hip`).

One product with the stacked matrix [q; k; v; output gate; a; b] gives the 32-bit projections of a step's rows.  One kernel
makes of them what the rule reads: q, k and v through their short convolutions (a request's rows before this step come from
its state) and SiLU, q and k as unit vectors, the decays and step sizes.  One kernel keeps every request's last rows for the
next step's convolutions (in a step of single rows the kernel before it does that on its way).  One kernel steps the memories over every request's rows, in order, from the request's state slot
and back into it.  One kernel divides every head's read-out by its root mean square, multiplies by the norm's weights and by
SiLU of the output gate, and stores the rows as the output product reads them.  Everything between the projections and the
output product is 32-bit, whatever the compute dtype.

A request's state: the memories S [head][key_dim][value_dim] and the convolutions' last taps - 1 inputs, one run of 32-bit
numbers in the slot the cache manager gives it (zeroed when the request opens).  The runs of rows that belong to one request
are found on the device, so a captured pass may contain the mixer."""
from __future__ import annotations

import torch

from ..cache.needs import StateNeed
from ..kernels import ops
from ..weights.loader import TensorNeed
from .attention import _pad_rows
from .base import Mixer, register_mixer
from .linear import activation_dtype_for, linear, linear_onto, takes_handed_norm


class GatedDelta(Mixer):
    graph_safe = True
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next
    can_overwrite = True

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and takes_handed_norm(self.w_in, n_rows)

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if s.n_heads % s.n_kv_heads:
            raise ValueError("gated delta rule: the number of heads must be a multiple of the number of query/key heads")
        if not 0 < s.key_dim <= ops.DELTA_MAX_KEY_DIM:
            raise ValueError(f"gated delta rule: key_dim = {s.key_dim} is outside what the kernel takes (1 to {ops.DELTA_MAX_KEY_DIM})")
        if not 1 <= s.conv_taps <= ops.DELTA_MAX_TAPS:
            raise ValueError(f"gated delta rule: {s.conv_taps} taps are outside what the kernel takes (1 to {ops.DELTA_MAX_TAPS})")
        qk, vv, h = s.n_kv_heads * s.key_dim, s.n_heads * s.value_dim, s.n_heads
        # the convolved columns first and side by side: q, k, v
        self.offsets = dict(conv=0, g=2 * qk + vv, a=2 * qk + 2 * vv, b=2 * qk + 2 * vv + h)
        self.w_in = _pad_rows(torch.cat([tensors[n] for n in (s.q_proj, s.k_proj, s.v_proj, s.gate_proj, s.a_proj, s.b_proj)], dim=0).contiguous())
        self.taps = torch.cat([tensors[n] for n in (s.q_conv, s.k_conv, s.v_conv)], dim=0).float().contiguous()
        self.a_log = tensors[s.a_log].float().contiguous()
        self.dt_bias = tensors[s.dt_bias].float().contiguous()
        self.out_norm = tensors[s.out_norm]
        self.w_o = tensors[s.o_proj]
        self.in_dtype = activation_dtype_for(self.w_in, dtype)
        self.mid_dtype = activation_dtype_for(self.w_o, dtype)

    def weights_read_per_step(self):
        return [self.w_in, self.taps, self.a_log, self.dt_bias, self.out_norm, self.w_o]

    # The first product's matrix, for a block that makes the first products of several parts in one (`ParallelBlock`): it then
    # hands the part its rows of that product (`forward(..., projected=)`) and the part keeps a view of the common matrix.
    def input_weight(self):
        return self.w_in

    def use_input_weight(self, view):
        self.w_in = view

    @classmethod
    def tensor_needs(cls, spec):
        s, d = spec, spec.hidden_size
        qk, vv = s.n_kv_heads * s.key_dim, s.n_heads * s.value_dim
        return [TensorNeed(s.q_proj, (qk, d)), TensorNeed(s.q_conv, (qk, s.conv_taps)), TensorNeed(s.k_proj, (qk, d)), TensorNeed(s.k_conv, (qk, s.conv_taps)),
                TensorNeed(s.v_proj, (vv, d)), TensorNeed(s.v_conv, (vv, s.conv_taps)), TensorNeed(s.b_proj, (s.n_heads, d)), TensorNeed(s.a_log, (s.n_heads,)),
                TensorNeed(s.out_norm, (s.value_dim,), "norm"), TensorNeed(s.a_proj, (s.n_heads, d)), TensorNeed(s.dt_bias, (s.n_heads,)),
                TensorNeed(s.gate_proj, (vv, d)), TensorNeed(s.o_proj, (d, vv))]

    @classmethod
    def cache_need(cls, spec):
        return StateNeed((ops.delta_state_floats(spec.n_heads, spec.n_kv_heads, spec.key_dim, spec.value_dim, spec.conv_taps),), torch.float32)

    def forward(self, h, residual, ctx, cache, then=None, overwrite=False, projected=None):
        s, T, o, dev = self.spec, ctx.n_rows, self.offsets, ctx.device
        H, G, dk, dv = s.n_heads, s.n_kv_heads, s.key_dim, s.value_dim
        vv = H * dv
        proj = projected
        if proj is None:
            proj = torch.empty((T, self.w_in.shape[0]), dtype=torch.float32, device=dev)
            linear(h, self.w_in, proj)
        seg_start, seg_len = ops.segments(ctx)
        qkv = torch.empty((T, 2 * G * dk + vv), dtype=torch.float32, device=dev)
        gates = torch.empty((T, 2 * H), dtype=torch.float32, device=dev)
        single_rows = ctx.max_seg_len == 1            # (a step's shape, which a captured pass shares with its replays)
        ops.delta_prepare(proj, o["conv"], o["a"], o["b"], self.taps, self.a_log, self.dt_bias, ctx.row_slot, ctx.row_pos, cache.state, qkv, gates,
                          H, G, dk, dv, dk ** -0.5, single_rows)
        if not single_rows:
            ops.delta_tail(proj, o["conv"], s.conv_taps, seg_start, seg_len, ctx.row_slot, cache.state, H, G, dk, dv)
        read = torch.empty((T, vv), dtype=torch.float32, device=dev)
        ops.delta_scan(qkv, gates, seg_start, seg_len, ctx.row_slot, cache.state, read, H, G, dk, dv)
        mid = torch.empty((T, vv), dtype=self.mid_dtype, device=dev)
        ops.head_norm_gate(read, proj[:, o["g"]:o["g"] + vv], self.out_norm, s.norm_eps, mid, H, dv, gate_activation="silu")
        if overwrite:
            linear(mid, self.w_o, residual)
            return None
        return linear_onto(mid, self.w_o, residual, then)


register_mixer("gated_delta", GatedDelta)
