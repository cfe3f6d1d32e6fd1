"""Attention whose queries, keys and values come through low-rank latents.

``c_q = rmsnorm(W_dq h)``, ``q = W_uq c_q`` laid out head by head as ``[dim plain, rot_dim rotated]``. ``W_dkv h`` gives
``kv_rank + rot_dim`` numbers: the first ``kv_rank``, normed, are the latent ``c``; the last ``rot_dim`` (not normed)
are one rotated key part that all heads share. Per head the plain key is ``W_uk c``, the value ``W_uv c``, and the
score ``(q_plain . k_plain + q_rot . k_rot) * scale``. The rotation pairs feature ``i`` with ``i + dims/2`` of the
rotated part's first ``dims`` features. A row sees itself and the ``window - 1`` tokens before it; ``exp(sink_h)``
joins each head's softmax denominator; each head's output is multiplied by ``sigmoid(W_g h)_h``.

What is kept per sequence. The latent and the rotated key part would do; this part keeps every head's key
``[plain | rotated]`` and value in the paged cache instead, because the window bounds what a sequence holds anyway
and the attention kernels of the library read such pages (head widths up to 256, which ``kv_rank + rot_dim`` as
the width of a single shared head soon exceeds). Where the matrix cores serve the step (bfloat16, key width a
multiple of 16) the values' pages are as wide as the keys', the columns beyond ``value_dim`` staying zero.

Other forms, by constructor arguments: no sink (``sink=False``: an ordinary softmax); a gate per output feature
instead of one per head (``gate="element"``: ``sigmoid(W_g h)`` is as wide as the concatenated heads); and, with a
position encoding over neighbouring pairs (``PairRotaryPositions``), feature ``2i`` of the rotated part turns with
feature ``2i + 1``.

Float arithmetic in both precisions: both latent norms, the rotation with float32 tables, scores, softmax with its
sink, the gate's sigmoid.
"""

from __future__ import annotations

import torch

from ..cache.spec import KVNeed
from ..cache.store import KVLine
from ..csrc import ops
from ..limits import MATRIX_CORE_HEAD_STEP, MAX_HEAD_DIM
from ..weights.spec import VECTOR
from . import register_part
from .attention import GQAAttention
from .base import Mixer, StepContext, matrix
from .linear import linear
from .rope import PairRotaryPositions


class LatentAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, positions: str | None = None, window: int | None = None,
                 sink: bool = True, gate: str = "head"):
        if gate not in ("head", "element"):
            raise ValueError(f"gate is 'head' or 'element', got {gate!r}")
        self.has_sink, self.element_gate = bool(sink), gate == "element"
        self.hidden, self.n_heads = int(hidden_size), int(num_heads)
        self.plain, self.rot_dim, self.value_dim = int(head_dim), int(rot_dim), int(value_dim)
        self.key_dim = self.plain + self.rot_dim
        if not (0 < self.key_dim <= MAX_HEAD_DIM and 0 < self.value_dim <= MAX_HEAD_DIM):
            raise ValueError(f"key and value widths must lie in 1..{MAX_HEAD_DIM}, got {self.key_dim} and {value_dim}")
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.positions, self.window = positions, (int(window) if window else None)
        self.w_down = self.w_uq = self.w_ukv = self.w_o = self.q_norm = self.kv_norm = self.sink = None

    def tensor_specs(self):
        H = self.n_heads
        specs = {"q_down": matrix((self.q_rank, self.hidden)), "q_norm": ((self.q_rank,), VECTOR, "ones"),
                "q_up": matrix((H * self.key_dim, self.q_rank)),
                "kv_down": matrix((self.kv_rank + self.rot_dim, self.hidden)), "kv_norm": ((self.kv_rank,), VECTOR, "ones"),
                "k_up": matrix((H * self.plain, self.kv_rank)), "v_up": matrix((H * self.value_dim, self.kv_rank)),
                "g_proj": matrix((H * self.value_dim if self.element_gate else H, self.hidden)),
                "o_proj": matrix((self.hidden, H * self.value_dim))}
        if self.has_sink:
            specs["sink"] = ((H,), VECTOR, "normal")
        return specs

    def load(self, tensors):
        # one product for everything that reads h: the queries' latent | the latent and the rotated key part | gates
        self.w_down = torch.cat([tensors["q_down"], tensors["kv_down"], tensors["g_proj"]], dim=0).contiguous()
        self.w_uq = tensors["q_up"]
        self.w_ukv = torch.cat([tensors["k_up"], tensors["v_up"]], dim=0).contiguous()
        self.w_o = tensors["o_proj"]
        self.q_norm, self.kv_norm = tensors["q_norm"].float().contiguous(), tensors["kv_norm"].float().contiguous()
        if self.has_sink:
            self.sink = tensors["sink"].float().contiguous()

    def _matrix_cores(self) -> bool:
        return self.compute_dtype == torch.bfloat16 and self.key_dim % MATRIX_CORE_HEAD_STEP == 0 and \
            self.value_dim <= self.key_dim

    def _page_value_dim(self) -> int:
        return self.key_dim if self._matrix_cores() else self.value_dim

    def cache_need(self):
        dv = self._page_value_dim()
        return KVNeed(self.n_heads, self.key_dim, self.window, dv if dv != self.key_dim else None)

    def kernel_modules(self, dtype):
        return ("gemm", "latent", "attn_rows") + (("attn_mfma",) if dtype == torch.bfloat16 else ())

    def forward(self, h: torch.Tensor, ctx: StepContext, line: KVLine, writes_cache: bool):
        rows, H, D, Dv = h.shape[0], self.n_heads, self.key_dim, self.value_dim
        cos = sin = None
        rot, pairs = 0, False
        if self.positions:
            table = ctx.positions[self.positions]
            if ctx.max_kv_len > table.n_positions:
                raise ValueError(f"position tables cover {table.n_positions} positions, the step reaches {ctx.max_kv_len}")
            cos, sin, rot, pairs = table.cos, table.sin, table.dims, isinstance(table, PairRotaryPositions)
        down = linear(h, self.w_down)                               # c_q | c | rotated key part | gates
        c_q = torch.empty((rows, self.q_rank), dtype=h.dtype, device=h.device)
        c_kv = torch.empty((rows, self.kv_rank), dtype=h.dtype, device=h.device)
        ops.rms_segments(down, 0, self.q_norm, c_q, self.q_rank, self.kv_norm, c_kv, self.norm_eps)
        q_raw = linear(c_q, self.w_uq)
        kv = linear(c_kv, self.w_ukv)                               # plain keys of all heads | values of all heads
        q = torch.empty((rows, H, D), dtype=h.dtype, device=h.device)
        page_dv = self._page_value_dim()
        ops.latent_rope_kv(q_raw, kv, down, self.q_rank + self.kv_rank, cos, sin, rot, ctx.row_slot, ctx.row_pos, q,
                           line.k, line.v, line.page_table, writes_cache, H, self.plain, self.rot_dim, Dv, page_dv,
                           pairs=pairs)
        window = self.window or 0
        if self._matrix_cores() and ctx.max_q_len == 1:
            out = torch.empty((rows, H, D), dtype=h.dtype, device=h.device)
            splits = self.decode_splits(ctx.n_seqs, ctx.max_kv_len)
            part_o = torch.empty((ctx.n_seqs, H, splits, D), dtype=torch.float32, device=h.device)
            part_ml = torch.empty((ctx.n_seqs, H, splits, 2), dtype=torch.float32, device=h.device)
            ops.attn_split_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, ctx.kv_len, ctx.n_seqs,
                                part_o, part_ml, splits, out, H, H, D, self.scale, window, sink=self.sink)
        elif self._matrix_cores():
            # the tiled kernel never visits the rows of sequences that sit out; they must hold something finite
            out = ctx.kept_zeros((rows, H, D), h.dtype) if ctx.some_sit_out() else \
                torch.empty((rows, H, D), dtype=h.dtype, device=h.device)
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu, ctx.seq_start,
                                 ctx.n_seqs, max_tiles, out, H, H, D, self.scale, window, sink=self.sink)
        else:
            out = torch.empty((rows, H, page_dv), dtype=h.dtype, device=h.device)
            ops.attn_rows(q, line.k, line.v, line.page_table, ctx.row_slot, ctx.row_pos, out, H, H, D, self.scale,
                          window, v_dim=page_dv, sink=self.sink, exact_p=True)
        gated = torch.empty((rows, H * Dv), dtype=h.dtype, device=h.device)
        ops.head_gate(out, down, self.q_rank + self.kv_rank + self.rot_dim, gated, H, Dv, per_element=self.element_gate)
        return linear(gated, self.w_o, allow_partials=True)

    def decode_splits(self, n_seqs: int, max_kv_len: int) -> int:
        return GQAAttention.decode_splits(self, n_seqs, max_kv_len)

    @property
    def n_kv(self) -> int:
        return self.n_heads

    def flops(self, rows, spans):
        seen = 0
        for start, q in spans:
            first, last = start + 1, start + q
            if self.window:
                full = max(0, min(last, self.window) - first + 1)
                seen += (2 * first + full - 1) * full // 2 + (q - full) * self.window
            else:
                seen += (first + last) * q // 2
        return super().flops(rows, spans) + 2.0 * self.n_heads * (self.key_dim + self.value_dim) * seen


register_part("latent_attention", LatentAttention)
