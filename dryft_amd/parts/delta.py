"""The gated delta rule: a matrix state per head that is corrected towards each token's value along its key.

``q`` and ``k`` (``num_kv_heads x key_dim``; head ``h`` uses ``h // (heads / kv_heads)``) and ``v`` (``heads x
value_dim``) are projections of the input without biases; each passes a short causal convolution per channel and
silu. ``q`` and ``k`` are made unit vectors per head, ``x / sqrt(sum(x^2) + unit_eps)``, ``q`` also times
``key_dim^-1/2``. With ``beta = sigmoid(W_b h)`` and ``g = exp(-exp(A_log) softplus(W_a h + dt_bias))`` per head,

    S <- g S;    u = beta (v - S^T k);    S <- S + k u^T;    o = S^T q

in this order, so the read-out sees the token's own write. Each head's ``o`` is divided by its root mean square, times
a weight shared by the heads, times ``silu(W_g h)``, and projected back.

The state (``S`` and the convolution's last ``taps - 1`` inputs) is float32 in the state store, zero when a sequence
starts. The two gates keep the float32 accumulators of their projections; sigmoid, softplus, both exponentials, the
unit lengths, the recurrence and the read-out's norm are float arithmetic in both precisions. A long sequence of a step
is walked as segments side by side: a token maps every column of the state alike, ``c -> g (I - beta k k^T) c + beta k
v_c``, so a segment's effect is the product of its tokens' maps and the state it reaches from zero.
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


class GatedDeltaMixer(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, conv_taps: int,
                 norm_eps: float, unit_eps: float = 1e-6):
        self.hidden, self.n_heads, self.n_kv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim, self.taps = int(key_dim), int(value_dim), int(conv_taps)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        if self.n_kv <= 0 or self.n_heads % self.n_kv:
            raise ValueError(f"{num_heads} heads cannot share {num_kv_heads} key heads evenly")
        if not 0 < self.key_dim <= ops.DELTA_MAX_DIM:
            raise ValueError(f"key_dim must lie in 1..{ops.DELTA_MAX_DIM}, got {key_dim}")
        if not 0 < self.value_dim <= ops.WKV_MAX_DIM:
            raise ValueError(f"value_dim must lie in 1..{ops.WKV_MAX_DIM}, got {value_dim}")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"the convolution takes 1..{ops.CONV_MAX_TAPS} taps, got {conv_taps}")
        self.qk_dim, self.v_dim = self.n_kv * self.key_dim, self.n_heads * self.value_dim
        self.conv_channels = 2 * self.qk_dim + self.v_dim
        self.w_in = self.w_gates = self.w_o = self.conv_w = self.dt_bias = self.a_log = self.out_norm = None

    def tensor_specs(self):
        t = self.taps
        return {"q_proj": matrix((self.qk_dim, self.hidden)), "k_proj": matrix((self.qk_dim, self.hidden)),
                "v_proj": matrix((self.v_dim, self.hidden)), "g_proj": matrix((self.v_dim, self.hidden)),
                "q_conv": matrix((self.qk_dim, t)), "k_conv": matrix((self.qk_dim, t)), "v_conv": matrix((self.v_dim, t)),
                "a_proj": matrix((self.n_heads, self.hidden)), "b_proj": matrix((self.n_heads, self.hidden)),
                "dt_bias": ((self.n_heads,), VECTOR, "normal"), "a_log": ((self.n_heads,), VECTOR, "normal"),
                "out_norm": ((self.value_dim,), VECTOR, "ones"), "o_proj": matrix((self.hidden, self.v_dim))}

    def load(self, tensors):
        self.w_in = torch.cat([tensors[n] for n in ("q_proj", "k_proj", "v_proj", "g_proj")], dim=0).contiguous()
        self.w_gates = torch.cat([tensors["a_proj"], tensors["b_proj"]], dim=0).contiguous()
        self.w_o = tensors["o_proj"]
        self.conv_w = torch.cat([tensors[n].float() for n in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.conv_wt = self.conv_w.t().contiguous()                         # tap by tap, for 8 channels a thread
        self.dt_bias, self.a_log = tensors["dt_bias"].float().contiguous(), tensors["a_log"].float().contiguous()
        self.out_norm = tensors["out_norm"].float().repeat(self.n_heads).contiguous()      # one weight for every head

    def cache_need(self):
        need = {"memory": StateNeed((self.n_heads, self.key_dim, self.value_dim))}
        if self.taps > 1:
            need["tail"] = conv_need(self.taps, self.conv_channels)
        return need

    def kernel_modules(self, dtype):
        return ("gemm", "conv", "delta", "wkv")

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        rows = h.shape[0]
        proj = linear(h, self.w_in)                                        # q | k | v | gate, in the activation dtype
        gates = linear(h, self.w_gates, out_dtype=torch.float32)            # a | b stay float32 from here on
        qkv = short_conv(proj, 0, self.conv_channels, self.conv_w, ctx, line.get("tail"), writes_cache, silu=True,
                         weight_t=self.conv_wt)
        # the rows of sequences that sit out are not visited by the walk; the read-out norms whatever they hold
        o_raw = ctx.kept_zeros((rows, self.v_dim), torch.float32) if ctx.some_sit_out() else \
            torch.empty((rows, self.v_dim), dtype=torch.float32, device=h.device)
        # a long prompt runs as segments side by side
        segments = ctx.segments() if writes_cache else None
        ops.delta_steps(qkv, 0, self.qk_dim, 2 * self.qk_dim, gates, 0, self.n_heads, self.dt_bias, self.a_log,
                        ctx.seq_slot, ctx.cu_rows, ctx.q_len, ctx.n_seqs, line["memory"].state, o_raw, self.n_heads,
                        self.n_kv, self.key_dim, self.value_dim, self.key_dim ** -0.5, self.unit_eps, writes_cache,
                        segments=segments)
        out = torch.empty((rows, self.v_dim), dtype=h.dtype, device=h.device)
        ops.wkv_out(o_raw, proj[:, self.conv_channels:], self.out_norm, out, self.n_heads, self.value_dim, self.norm_eps)
        return linear(out, self.w_o, allow_partials=True)

    def flops(self, rows, spans):
        """The projections, the convolution, and per token and head the state's decay, correction and read-out."""
        return super().flops(rows, spans) + 2.0 * rows * self.conv_channels * self.taps + \
            7.0 * rows * self.n_heads * self.key_dim * self.value_dim


register_part("gated_delta", GatedDeltaMixer)
