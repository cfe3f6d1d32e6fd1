"""A state-space mixer with a scalar decay per head and token (the Mamba-2 recurrence) behind a short convolution.

One projection of the input gives ``[z | x | B | C | dt]``: a gate ``z`` and the recurrence's input ``x`` (``heads x
head_dim`` each), ``B`` and ``C`` (``groups x state``; head ``h`` uses group ``h // (heads / groups)``) and one step
size per head. ``x``, ``B`` and ``C`` pass one causal convolution per channel with a bias, then silu. Then

    dt_t = softplus(dt_t + dt_bias)        S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T        y_t = S_t^T C_t + D x_t

per head (``S`` is ``state x head_dim``). The heads' ``y`` side by side are multiplied by ``silu(z)`` and then divided,
in ``norm_parts`` equal runs, by each run's root mean square, times a weight (the gate comes before the norm), and
projected back.

The state (``S`` and the convolution's last ``taps - 1`` inputs) is float32 in the state store, zero when a sequence
starts. The step sizes keep the float32 accumulators of their projection, and softplus, both exponentials, the
recurrence, the gate and the norm are float arithmetic in both precisions. A step may bring any number of rows per
sequence; the kernels walk them in order from the state the step before left, a long sequence as segments side by side
(the recurrence is linear in the state: a segment's effect is the product of its decays and the state it reaches from
zero).
"""

from __future__ import annotations

import torch

from ..cache.spec import StateNeed
from ..csrc import ops
from ..weights.spec import VECTOR
from . import register_part
from .base import Mixer, StepContext, matrix
from .conv import conv_need, short_conv
from .linear import linear


class StateSpaceMixer(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, state_size: int, groups: int, conv_taps: int,
                 norm_parts: int, norm_eps: float):
        self.hidden, self.n_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.n_state, self.groups, self.taps, self.norm_parts = int(state_size), int(groups), int(conv_taps), int(norm_parts)
        self.norm_eps = float(norm_eps)
        self.inner = self.n_heads * self.head_dim
        if self.groups <= 0 or self.n_heads % self.groups:
            raise ValueError(f"{num_heads} heads do not share {groups} groups evenly")
        if self.norm_parts <= 0 or self.inner % self.norm_parts:
            raise ValueError(f"{self.inner} channels do not split into {norm_parts} equal parts for the norm")
        if not 0 < self.n_state <= ops.SSM_MAX_STATE:
            raise ValueError(f"the state takes 1..{ops.SSM_MAX_STATE} rows, got {state_size}")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"the convolution takes 1..{ops.CONV_MAX_TAPS} taps, got {conv_taps}")
        self.conv_channels = self.inner + 2 * self.groups * self.n_state
        self.w_in = self.w_dt = self.w_o = self.conv_w = self.conv_b = None
        self.dt_bias = self.a_log = self.d_skip = self.out_norm = None

    def tensor_specs(self):
        return {"in_proj": matrix((self.inner + self.conv_channels + self.n_heads, self.hidden)),
                "conv": matrix((self.conv_channels, self.taps)), "conv_bias": ((self.conv_channels,), VECTOR, "normal"),
                "dt_bias": ((self.n_heads,), VECTOR, "normal"), "a_log": ((self.n_heads,), VECTOR, "normal"),
                "d_skip": ((self.n_heads,), VECTOR, "ones"), "out_norm": ((self.inner,), VECTOR, "ones"),
                "o_proj": matrix((self.hidden, self.inner))}

    def load(self, tensors):
        w = tensors["in_proj"]
        cut = self.inner + self.conv_channels
        self.w_in = w[:cut].contiguous()              # z | x | B | C, in the activation dtype
        self.w_dt = w[cut:].contiguous()              # the step sizes: their product keeps its float32 accumulators
        self.w_o = tensors["o_proj"]
        self.conv_w, self.conv_b = tensors["conv"].float().contiguous(), tensors["conv_bias"].float().contiguous()
        self.conv_wt = self.conv_w.t().contiguous()
        for name in ("dt_bias", "a_log", "d_skip", "out_norm"):
            setattr(self, name, tensors[name].float().contiguous())

    def cache_need(self):
        need = {"state": StateNeed((self.n_heads, self.n_state, self.head_dim))}
        if self.taps > 1:
            need["tail"] = conv_need(self.taps, self.conv_channels)
        return need

    def kernel_modules(self, dtype):
        return ("gemm", "conv", "ssm")

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        rows, GN = h.shape[0], self.groups * self.n_state
        proj = linear(h, self.w_in)
        dt_raw = linear(h, self.w_dt, out_dtype=torch.float32)
        xbc = short_conv(proj, self.inner, self.conv_channels, self.conv_w, ctx, line.get("tail"), writes_cache,
                         out_bias=self.conv_b, silu=True, weight_t=self.conv_wt)
        # a long prompt runs as segments side by side (the rows of sequences that sit out are then not visited)
        segments = ctx.segments() if writes_cache else None
        y = torch.empty((rows, self.inner), dtype=torch.float32, device=h.device)
        ops.ssm_scan(xbc, 0, self.inner, self.inner + GN, dt_raw, self.dt_bias, self.a_log, self.d_skip, ctx.seq_slot,
                     ctx.cu_rows, ctx.q_len, ctx.n_seqs, line["state"].state, y, self.n_heads, self.head_dim,
                     self.n_state, self.groups, writes_cache, segments=segments)
        out = torch.empty((rows, self.inner), dtype=h.dtype, device=h.device)
        ops.gate_part_norm(y, proj, 0, self.out_norm, ctx.row_slot, out, self.norm_parts, self.norm_eps)
        return linear(out, self.w_o, allow_partials=True)

    def flops(self, rows, spans):
        """The projections, the convolution, and per token and head the update of the state and its read-out."""
        return super().flops(rows, spans) + 2.0 * rows * self.conv_channels * self.taps + \
            6.0 * rows * self.n_heads * self.n_state * self.head_dim


register_part("state_space", StateSpaceMixer)
