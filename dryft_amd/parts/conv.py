"""A short causal convolution over time on every channel of a projection, for mixers that have one.

``y[t, c] = act(sum_j w[c, j] * u[t - taps + 1 + j, c] + b[c])`` with zeros before a sequence's start; the last column
of ``w`` meets the current token. The last ``taps - 1`` inputs of a sequence are part of its state (``conv_need``,
float32 in the state store, zero when a sequence starts), so a prompt, a portion of one and a single token are the
same code. A bias of the projection itself (``in_bias``) is added to the inputs on their way in, and is therefore part
of what the state holds. Float arithmetic, rounded once.
"""

from __future__ import annotations

import torch

from ..cache.spec import StateNeed
from ..csrc import ops
from .base import StepContext


def conv_need(taps: int, channels: int) -> StateNeed | None:
    return StateNeed((int(taps) - 1, int(channels))) if taps > 1 else None


def short_conv(u: torch.Tensor, col: int, channels: int, weight: torch.Tensor, ctx: StepContext, tail_line,
               writes_cache: bool, *, in_bias=None, out_bias=None, silu: bool = False, weight_t=None) -> torch.Tensor:
    """The convolution of columns ``col .. col + channels`` of ``u`` over this step's rows, ``[rows, channels]`` in the
    dtype of ``u``; ``weight`` is float32 ``[channels, taps]``, ``weight_t`` (optional) the same tap by tap, ``[taps,
    channels]``, for the kernel that takes 8 channels a thread. With ``writes_cache`` the sequences' tails move on."""
    taps = weight.shape[1]
    tail = tail_line.state if taps > 1 else None
    out = torch.empty((u.shape[0], channels), dtype=u.dtype, device=u.device)
    ops.causal_conv(u, col, channels, in_bias, weight, out_bias, silu, ctx.row_slot, ctx.row_seq, ctx.row_pos,
                    ctx.seq_start, tail, out, weight_t=weight_t)
    if writes_cache and taps > 1:
        ops.conv_tail(u, col, channels, in_bias, taps, ctx.seq_slot, ctx.cu_rows, ctx.q_len, ctx.n_seqs, tail)
    return out
