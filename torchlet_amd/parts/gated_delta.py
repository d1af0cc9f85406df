"""The gated delta rule with a fixed-size state per request.

Per token, with ``q = W_q h`` and ``k = W_k h`` (``kv_heads x dim``) and ``v = W_v h`` (``heads x vdim``): each channel of q, k and v
passes a causal convolution over the last ``conv`` tokens (zeros before the start of the sequence) and silu; q and k become unit
vectors per head (``x / sqrt(sum x^2 + unit_eps)``), q times ``dim ** -0.5``; ``beta = sigmoid(W_b h)`` and ``g = exp(-exp(A_log) *
softplus(W_a h + dt_bias))`` per head.  Head ``i`` (reading q/k head ``i // (heads / kv_heads)``) moves its state ``S [dim, vdim]``::

    S <- g S;    u = beta (v - S^T k);    S <- S + k u^T;    o = S^T q

and the mixer's output is ``W_o (concat_heads(o / rms(o) * w_norm) * silu(W_g h))``.  A request's slot holds the states of all
heads and the last ``conv - 1`` inputs of every convolved channel, in 32-bit, zero when the slot is handed out.  The unit norms, the
gates, the decays, the state and the per-head norm are 32-bit under every engine; the projections run in the compute dtype (the two
per-head gates leave their product in 32-bit).  One kernel runs the recurrence for every request of the step from where its state
stands, token by token, so a portion of n tokens is n single steps by construction.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..config.base import ConfigError
from .base import KEEP_COMPUTE, KEEP_FLOAT32, MIXERS, StagedMixer, StateNeed, WeightSpec, register_init_law


@register_init_law("log_decay")
def _init_log_decay(shape, gen, device, std):
    """Logarithms of decay rates between about 0.02 and 1."""
    return torch.log(torch.rand(shape, generator=gen, device=device, dtype=torch.float32) * 0.98 + 0.02)


@register_init_law("conv_taps")
def _init_conv_taps(shape, gen, device, std):
    """Convolution taps of order one over their number."""
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * (1.0 / shape[-1])


@MIXERS.register("gated_delta")
class GatedDelta(StagedMixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.heads % spec.kv_heads:
            raise ConfigError(f"gated delta rule: {spec.heads} heads are not a multiple of {spec.kv_heads} query/key heads")
        if spec.conv < 1 or spec.conv > ops.DELTA_MAX_TAPS:
            raise ConfigError(f"gated delta rule: convolutions of 1 to {ops.DELTA_MAX_TAPS} taps are built, not {spec.conv}")
        if spec.dim > ops.DELTA_MAX_DIM:
            raise ConfigError(f"gated delta rule: built for up to {ops.DELTA_MAX_DIM} query/key dimensions per head, not {spec.dim}")
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim, self.taps = spec.hidden, spec.heads, spec.kv_heads, spec.dim, spec.vdim, spec.conv
        self.qk_width, self.v_width = spec.kv_heads * spec.dim, spec.heads * spec.vdim
        self.channels = 2 * self.qk_width + self.v_width                 # convolved channels: q, k, v
        self.in_width = self.channels + self.v_width                     # ... and the output gate
        self.mix_width = self.v_width
        self.qscale = float(spec.dim) ** -0.5 if spec.query_scale is None else float(spec.query_scale)
        self.state_floats = spec.heads * spec.dim * spec.vdim            # the heads' states; the convolutions' tails follow
        self.w_gates = self.w_conv = self.a_log = self.dt_bias = self.w_norm = None

    def state_need(self):
        return StateNeed(shape=(self.state_floats + (self.taps - 1) * self.channels,), dtype=torch.float32)

    def kernel_libraries(self):
        return ["recurrent"]

    def weight_specs(self):
        H = self.hidden
        return {
            "q": WeightSpec((self.qk_width, H)), "q.conv": WeightSpec((self.qk_width, self.taps), keep=KEEP_FLOAT32, init="conv_taps"),
            "k": WeightSpec((self.qk_width, H)), "k.conv": WeightSpec((self.qk_width, self.taps), keep=KEEP_FLOAT32, init="conv_taps"),
            "v": WeightSpec((self.v_width, H)), "v.conv": WeightSpec((self.v_width, self.taps), keep=KEEP_FLOAT32, init="conv_taps"),
            "b": WeightSpec((self.heads, H)), "a": WeightSpec((self.heads, H)),
            "A_log": WeightSpec((self.heads,), keep=KEEP_FLOAT32, init="log_decay"),
            "dt_bias": WeightSpec((self.heads,), keep=KEEP_FLOAT32),
            "norm": WeightSpec((self.vdim,), keep=KEEP_FLOAT32, init="one_plus_normal"),
            "g": WeightSpec((self.v_width, H)), "o": WeightSpec((H, self.v_width)),
        }

    def load_weights(self, tensors):
        # one matrix for what is read in the activation dtype (queries, keys, values, the output gate), one for the two per-head
        # gates of the recurrence, whose product leaves in 32-bit
        self.w_in = self._place(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0), KEEP_COMPUTE)
        self.w_gates = self._place(torch.cat((tensors["b"], tensors["a"]), dim=0), KEEP_COMPUTE)
        self.w_conv = self._place(torch.cat([tensors[f"{n}.conv"].float() for n in "qkv"], dim=0), KEEP_FLOAT32)
        self.a_log = self._place(tensors["A_log"], KEEP_FLOAT32)
        self.dt_bias = self._place(tensors["dt_bias"], KEEP_FLOAT32)
        self.w_norm = self._place(tensors["norm"], KEEP_FLOAT32)
        self.w_o = self._place(tensors["o"], KEEP_COMPUTE)

    def mix(self, proj, h, ctx, cache, out, gain=1.0):
        T = h.shape[0]
        gates = torch.empty((T, 2 * self.heads), dtype=torch.float32, device=h.device)
        ops.linear(h, self.w_gates, None, gates)
        qkv = torch.empty((T, self.channels), dtype=torch.float32, device=h.device)
        # convolutions (from the slot's tails, which move on), silu, unit vectors; the raw gates become beta and the decay in place
        ops.delta_prepare(proj, self.w_conv, gates, self.a_log, self.dt_bias, cache.state, self.state_floats, ctx.slots, ctx.req_indptr,
                          ctx.token_req, qkv, self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.qscale, float(self.spec.unit_eps))
        o = torch.empty((T, self.v_width), dtype=torch.float32, device=h.device)
        ops.delta_scan(qkv, gates, cache.state, ctx.slots, ctx.req_indptr, o, self.heads, self.kv_heads, self.dim, self.vdim,
                       max_new_tokens=ctx.max_new_tokens)
        ops.gated_head_norm(o, proj[:, self.channels:], self.w_norm, float(self.spec.norm_eps), out, self.heads, self.vdim,
                            gate="silu", gain=gain)
