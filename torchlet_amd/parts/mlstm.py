"""Matrix-memory recurrence (the mLSTM of xLSTM) with a fixed-size state per request.

Per head, with ``q = W_q h * dim**-0.5``, ``k = W_k h``, ``v = W_v h``, a log input gate ``i = cap(W_i h + b_i)`` and a log
forget gate ``f = logsigmoid(cap(W_f h + b_f))``, ``cap(z) = c * tanh(z / c)``, the state ``S [dim, vdim]``, ``n [dim]`` and a
running maximum ``m`` (all zero for a new request) move token by token::

    m' = max(f + m, i);   S' = exp(f + m - m') S + exp(i - m') k v^T;   n' = exp(f + m - m') n + exp(i - m') k
    o  = S'^T q / (max(|n' . q|, exp(-m')) + denom_eps)

and the mixer's output is ``W_o (concat_heads(o / rms(o)) * w_norm * sigmoid(W_g h))``.  The state lives in 32-bit in the
cache manager's slot of the request; gates, decays and the quotient are 32-bit under every engine, the projections run in
the compute dtype.  One kernel runs the recurrence for every request of the step from where its state stands, so a
portion of n tokens is n single steps by construction.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_FLOAT32, KEEP_STORED, MIXERS, Mixer, StateNeed, WeightSpec


@MIXERS.register("mlstm")
class MLSTM(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden, self.heads, self.dim, self.vdim = spec.hidden, spec.heads, spec.dim, spec.vdim
        self.qk_width, self.v_width = spec.heads * spec.dim, spec.heads * spec.vdim
        self.qscale = float(spec.dim) ** -0.5 if spec.query_scale is None else float(spec.query_scale)
        self.state_width = spec.dim * spec.vdim + spec.dim + 1          # S, n and m of one head
        self.w_in = self.w_gates = self.b_gates = self.w_norm = self.w_o = None

    def state_need(self):
        return StateNeed(shape=(self.heads, self.state_width), dtype=torch.float32)

    def kernel_libraries(self):
        return ["recurrent"]

    def weight_specs(self):
        H = self.hidden
        return {
            "q": WeightSpec((self.qk_width, H)), "k": WeightSpec((self.qk_width, H)),
            "v": WeightSpec((self.v_width, H)), "g": WeightSpec((self.v_width, H)),
            "o": WeightSpec((H, self.v_width)),
            "norm": WeightSpec((self.v_width,), keep=KEEP_STORED, init="one_plus_normal"),
            "i": WeightSpec((self.heads, H)), "i.b": WeightSpec((self.heads,), keep=KEEP_FLOAT32),
            "f": WeightSpec((self.heads, H)), "f.b": WeightSpec((self.heads,), keep=KEEP_FLOAT32),
        }

    def load_weights(self, tensors):
        # one matrix for queries, keys, values and the output gate, one for the two gates of the recurrence, whose
        # product leaves in 32-bit (with its bias added there)
        self.w_in = self._place(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0), KEEP_COMPUTE)
        self.w_gates = self._place(torch.cat((tensors["i"], tensors["f"]), dim=0), KEEP_COMPUTE)
        self.b_gates = self._place(torch.cat((tensors["i.b"].float(), tensors["f.b"].float())), KEEP_FLOAT32)
        self.w_norm = self._place(tensors["norm"], KEEP_STORED)
        self.w_o = self._place(tensors["o"], KEEP_COMPUTE)

    def forward(self, h, ctx, cache):
        T = h.shape[0]
        proj = torch.empty((T, 2 * self.qk_width + 2 * self.v_width), dtype=self.dtype, device=h.device)
        ops.linear(h, self.w_in, None, proj)
        gates = torch.empty((T, 2 * self.heads), dtype=torch.float32, device=h.device)
        ops.linear(h, self.w_gates, self.b_gates, gates)
        o = torch.empty((T, self.v_width), dtype=torch.float32, device=h.device)
        ops.mlstm_scan(proj, self.qk_width, 2 * self.qk_width, gates, cache.state, ctx.slots, ctx.req_indptr, o,
                       self.heads, self.dim, self.vdim, self.spec.gate_cap, self.qscale, float(self.spec.denom_eps))
        y = torch.empty((T, self.v_width), dtype=self.dtype, device=h.device)
        ops.gated_head_norm(o, proj[:, 2 * self.qk_width + self.v_width:], self.w_norm, float(self.spec.norm_eps), y, self.heads, self.vdim)
        if self.dtype == torch.bfloat16 and ops.linear_partials_pay(T, self.hidden, self.v_width):
            return ops.linear_partials(y, self.w_o)      # few rows against a narrow matrix: the next norm adds the slabs up
        out = torch.empty((T, self.hidden), dtype=self.dtype, device=h.device)
        ops.linear(y, self.w_o, None, out)
        return out
