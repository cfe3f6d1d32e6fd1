"""A matrix state per head with a decay that depends on the token (RWKV-style time mixing).

With ``h'`` the previous token's input (zeros before the first token), each of r, k, v, g, w reads a blend of its
own, ``h + (h' - h) * mu``. ``r, k, v`` are projections of their blends (heads x dim), ``gate = silu(W_g .)``, and the
decay is ``w = exp(-exp(W_up tanh(W_down .) + bias))`` per head and key channel. Per head, with a bonus ``u`` for the
token at hand: ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``. Each head's
``o`` is divided by its root mean square, weighted, gated, and projected back.

The state (``S`` and the previous token's input) is float32 in the state store, zero when a sequence starts. What
enters the recurrence besides the projections is float arithmetic in both precisions: the decay from the float
accumulators of its first projection on (tanh, the second product, both exponentials), the bonus, the read-out and
its norm. A step may bring any number of rows per sequence; the kernels walk them in order from the state the step
before left, so a prompt, a portion of one and a single token are the same code.
"""

from __future__ import annotations

import torch

from ..cache.spec import StateNeed
from ..csrc import ops
from ..weights.spec import VECTOR
from . import register_part
from .base import Mixer, StepContext, matrix
from .linear import linear

_BLENDS = ("r", "k", "v", "g", "w")


class WKVMixer(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float, decay_rank: int | None = None):
        self.hidden, self.n_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        if not 0 < self.head_dim <= ops.WKV_MAX_DIM:
            raise ValueError(f"head_dim must lie in 1..{ops.WKV_MAX_DIM}, got {head_dim}")
        self.inner = self.n_heads * self.head_dim
        self.decay_rank = int(decay_rank) if decay_rank else None     # None: whatever the checkpoint holds
        self.norm_eps = float(norm_eps)
        self.mu = self.w_r = self.w_k = self.w_v = self.w_g = self.w_down = self.w_up = self.w_o = None
        self.decay_bias = self.bonus = self.out_norm = None

    def tensor_specs(self):
        rank = self.decay_rank or -1
        specs = {f"mu_{n}": ((self.hidden,), VECTOR, "normal") for n in _BLENDS}
        specs.update({"r_proj": matrix((self.inner, self.hidden)), "k_proj": matrix((self.inner, self.hidden)),
                      "v_proj": matrix((self.inner, self.hidden)), "g_proj": matrix((self.inner, self.hidden)),
                      "decay_down": matrix((rank, self.hidden)), "decay_up": matrix((self.inner, rank)),
                      "decay_bias": ((self.inner,), VECTOR, "normal"),
                      "bonus": ((self.n_heads, self.head_dim), VECTOR, "normal"),
                      "out_norm": ((self.inner,), VECTOR, "ones"), "o_proj": matrix((self.hidden, self.inner))})
        return specs

    def load(self, tensors):
        self.mu = torch.stack([tensors[f"mu_{n}"].float() for n in _BLENDS]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (tensors[n + "_proj"] for n in ("r", "k", "v", "g"))
        self.w_down, self.w_up, self.w_o = tensors["decay_down"], tensors["decay_up"].contiguous(), tensors["o_proj"]
        if self.w_down.shape[0] != self.w_up.shape[1]:
            raise ValueError(f"the decay's two projections disagree on its rank: {tuple(self.w_down.shape)} and "
                             f"{tuple(self.w_up.shape)}")
        self.decay_bias = tensors["decay_bias"].float().contiguous()
        self.bonus = tensors["bonus"].float().contiguous()
        self.out_norm = tensors["out_norm"].float().contiguous()

    def cache_need(self):
        return {"memory": StateNeed((self.n_heads, self.head_dim, self.head_dim)), "previous": StateNeed((self.hidden,))}

    def kernel_modules(self, dtype):
        return ("gemm", "wkv")

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        rows = h.shape[0]
        blends = torch.empty((len(_BLENDS), rows, self.hidden), dtype=h.dtype, device=h.device)
        ops.wkv_blend(h, line["previous"].state, self.mu, ctx.row_slot, ctx.row_seq, ctx.row_pos, ctx.seq_start, blends)
        r, k, v, g = (linear(blends[i], w) for i, w in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)))
        low = linear(blends[4], self.w_down, out_dtype=torch.float32)      # the decay stays float32 from here on
        decay = torch.empty((rows, self.inner), dtype=torch.float32, device=h.device)
        ops.wkv_decay(low, self.w_up, self.decay_bias, decay)
        # a long prompt runs as segments side by side (the rows of sequences that sit out are then not visited)
        segments = ctx.segments(ops.WKV_GROUP) if writes_cache else None
        if segments is not None and ctx.some_sit_out():
            o_raw = ctx.kept_zeros((rows, self.inner), torch.float32)
        else:
            o_raw = torch.empty((rows, self.inner), dtype=torch.float32, device=h.device)
        ops.wkv_steps(r, k, v, decay, self.bonus, ctx.seq_slot, ctx.cu_rows, ctx.q_len, ctx.n_seqs,
                      line["memory"].state, o_raw, h, line["previous"].state, self.n_heads, self.head_dim,
                      writes_cache, segments=segments)
        out = torch.empty((rows, self.inner), dtype=h.dtype, device=h.device)
        ops.wkv_out(o_raw, g, self.out_norm, out, self.n_heads, self.head_dim, self.norm_eps)
        return linear(out, self.w_o, allow_partials=True)

    def flops(self, rows, spans):
        """The projections, and per token and head the update of the state and its read-out."""
        return super().flops(rows, spans) + 5.0 * rows * self.n_heads * self.head_dim * self.head_dim


register_part("wkv", WKVMixer)
