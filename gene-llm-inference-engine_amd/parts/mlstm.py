"""The matrix-memory mixer (mLSTM): per head a memory S [key_dim, value_dim] with a normaliser and exponential input and forget
gates whose logarithms are kept bounded by a running maximum (`config.spec.MlstmSpec` states the recurrence; the kernel is
`csrc/recurrent.hip`).

One product with the stacked matrix [q; k; v; output gate; i; f] gives the 32-bit projections of a step's rows; one kernel
steps every request's memories over its rows of this step, in order, from the state slot of the request and back into it;
one kernel divides every head's output by its root mean square, multiplies by the norm's weights and the sigmoid of the output
gate and stores the rows as the output product reads them.  The memories, the gates and everything between the projections
and the output product are 32-bit, whatever the compute dtype.

The runs of rows that belong to one request are found on the device from the rows' slots and positions, so a captured pass
may contain the mixer: nothing but the number of requests comes from the host."""
from __future__ import annotations

import torch

from ..cache.needs import StateNeed
from ..kernels import ops
from ..weights.loader import TensorNeed
from .attention import _pad_rows
from .base import Mixer, register_mixer
from .linear import activation_dtype_for, linear, linear_onto


class Mlstm(Mixer):
    graph_safe = True
    accepts_deferred_norm = True      # its input goes into `linear` only
    can_overwrite = True              # `forward(..., overwrite=True)` stores its result in `residual` instead of adding onto it

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if not 0 < s.key_dim <= ops.mlstm_max_key_dim():
            raise ValueError(f"mlstm: key_dim = {s.key_dim} is outside what the kernel takes (1 to {ops.mlstm_max_key_dim()})")
        qk, vv, h = s.n_heads * s.key_dim, s.n_heads * s.value_dim, s.n_heads
        self.offsets = dict(q=0, k=qk, v=2 * qk, g=2 * qk + vv, i=2 * qk + 2 * vv, f=2 * qk + 2 * vv + h)
        self.w_in = _pad_rows(torch.cat([tensors[n] for n in (s.q_proj, s.k_proj, s.v_proj, s.gate_proj, s.i_proj, s.f_proj)], dim=0).contiguous())
        self.i_bias = tensors[s.i_bias].float().contiguous()
        self.f_bias = tensors[s.f_bias].float().contiguous()
        self.out_norm = tensors[s.out_norm]
        self.w_o = tensors[s.o_proj]
        self.in_dtype = activation_dtype_for(self.w_in, dtype)
        self.mid_dtype = activation_dtype_for(self.w_o, dtype)

    @classmethod
    def tensor_needs(cls, spec):
        s, d = spec, spec.hidden_size
        qk, vv = s.n_heads * s.key_dim, s.n_heads * s.value_dim
        return [TensorNeed(s.q_proj, (qk, d)), TensorNeed(s.k_proj, (qk, d)), TensorNeed(s.v_proj, (vv, d)), TensorNeed(s.gate_proj, (vv, d)),
                TensorNeed(s.o_proj, (d, vv)), TensorNeed(s.out_norm, (vv,), "norm"), TensorNeed(s.i_proj, (s.n_heads, d)), TensorNeed(s.i_bias, (s.n_heads,)),
                TensorNeed(s.f_proj, (s.n_heads, d)), TensorNeed(s.f_bias, (s.n_heads,))]

    @classmethod
    def cache_need(cls, spec):
        return StateNeed((ops.mlstm_state_floats(spec.n_heads, spec.key_dim, spec.value_dim),), torch.float32)

    def forward(self, h, residual, ctx, cache, overwrite=False):
        s, T, o = self.spec, ctx.n_rows, self.offsets
        vv = s.n_heads * s.value_dim
        proj = torch.empty((T, self.w_in.shape[0]), dtype=torch.float32, device=ctx.device)
        linear(h, self.w_in, proj)
        seg_start, seg_len = ops.segments(ctx)
        sums = torch.empty((T, vv), dtype=torch.float32, device=ctx.device)          # the heads' S^T q, and what to divide them by
        divisors = torch.empty((T, s.n_heads), dtype=torch.float32, device=ctx.device)
        ops.mlstm_scan(proj, (o["q"], o["k"], o["v"], o["i"], o["f"]), self.i_bias, self.f_bias, s.gate_cap, s.key_dim ** -0.5, seg_start, seg_len,
                       ctx.row_slot, cache.state, sums, divisors, s.n_heads, s.key_dim, s.value_dim)
        mid = torch.empty((T, vv), dtype=self.mid_dtype, device=ctx.device)
        ops.head_norm_gate(sums, proj[:, o["g"]:o["g"] + vv], self.out_norm, s.norm_eps, mid, s.n_heads, s.value_dim, den=divisors)
        if overwrite:
            linear(mid, self.w_o, residual)
        else:
            linear_onto(mid, self.w_o, residual)


register_mixer("mlstm", Mlstm)
