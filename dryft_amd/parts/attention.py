"""Grouped-query attention over the paged cache.

Per row: ``q, k, v`` from one fused projection (reference: engine/dryft_qwen3/weights.py:93-96);
optional RMSNorm over each q and k head (one weight per head width, before the rotation,
model.py:165-166); optional rotary positions; append k and v to the cache line (model.py:170-171);
causal scores ``(q . k) / sqrt(head_dim)`` against every cached key of the sequence up to the row's
own position (or the last ``window`` of them), query head ``h`` reading kv head ``h // group``
(model.py:172-177, 254-257); output projection (model.py:179). No biases.

Options other designs use, all off by default: values of another width than the keys (``value_dim``); a
capped score, ``s <- softcap * tanh(s / softcap)``; a sink per query head (tensor ``sink``), whose ``exp`` joins
the softmax's denominator and nothing else; an output gate, the heads' outputs times ``sigmoid(W_g h)`` before
the output projection (tensor ``g_proj``, fused into the q/k/v product); attention weights kept in float
(``float_weights``); biases on the q, k, v and output projections (``bias``); a short causal convolution over time on
every channel of q, k and v right after the projection (``conv_taps``; the last ``taps - 1`` projected values of a
sequence are then part of its state, beside its keys and values); and a position encoding with float tables, over
neighbouring pairs (``PairRotaryPositions``) or over halves (``HalfRotaryPositions``; this one also after the per-head
norms, in float); a sink of a fixed score instead of a learned one (``sink_value``: 0 puts ``1`` beside the sum of
the exponentials); chunks instead of a window (``chunk``: a row sees the earlier keys of its own run of so many
positions, runs counted from position 0); a learned bias by distance added to the scaled score (``distance_bias =
(rows, far)``, tensor ``rel [rows, heads]``: distances below ``rows / 2`` have a row each, the others share the upper
half on a logarithmic scale that reaches the last row at ``far``); one output gate per head instead of one per
feature (``output_gate="head"``); and values that lean on those of an earlier layer (``value_mix = (name, first)``:
the first layer of that name leaves its values of the step's rows in the step context, every later one takes ``(1 -
l) v + l v_first`` with its own learned ``l``, tensor ``vmix``, before anything is cached). Any of these takes the
step down ``_forward_general``.

``pad_pages``: in bfloat16, heads whose keys and values differ in width (or whose width is no multiple of 16) keep
pages of one width for both, the next multiple of 16 that holds either, with zeros behind a head's own features: the
matrix-core kernels, which take one width, then serve them (zeros add nothing to a score, and the outputs behind
``value_dim`` are never read). Off by default; without it such heads take the float kernel.

The part knows nothing of the model around it: sizes and constants are constructor arguments, the
position encoding is looked up by name in the step context, and its storage is the cache line it
is handed.
"""

from __future__ import annotations

import math

import torch

from ..cache.spec import KVNeed
from ..cache.store import KVLine
from ..csrc import ops
from ..limits import MATRIX_CORE_HEAD_STEP, MAX_HEAD_DIM
from ..weights.spec import VECTOR
from . import register_part
from .base import Mixer, Partials, StepContext, matrix
from .conv import conv_need, short_conv
from .linear import linear
from .rope import HalfRotaryPositions, PairRotaryPositions, RotaryPositions

_RESIDENT_WORKGROUPS = 512     # of the split kernel: two per compute unit (its registers allow no more)
_MAX_SPLITS = 32
_QKV_PARTIAL_ROWS = 256         # decoding steps of up to so many rows take the projection as partial sums over K
_PROMPT_PARTIAL_ROWS = 256      # and so do prompt steps of at most so many rows


def add_bias(delta, bias: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``delta + bias`` per row in ``dtype``; ``delta`` is a tensor or ``Partials`` (added up on the way in)."""
    data = delta.data if isinstance(delta, Partials) else delta
    out = torch.empty(data.shape[-2:], dtype=dtype, device=data.device)
    ops.stream_norm(None, (delta.data, delta.count) if isinstance(delta, Partials) else delta, None, None, bias, None, 0.0,
                    None, out, dtype, plain_read=True)
    return out


def distance_row(n: int, rows: int, far: int) -> int:
    """The row of a bias table that distance ``n`` reads: its own below half the table, then
    ``half + floor(log(n / half) / log(far / half) * (rows - half))``, at most the last."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


class GQAAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qk_norm_eps: float | None = None, positions: str | None = None, rotary_dim: int | None = None,
                 window: int | None = None, scale: float | None = None, value_dim: int | None = None,
                 softcap: float | None = None, sink: bool = False, output_gate: bool | str = False,
                 float_weights: bool = False, bias: bool = False, conv_taps: int | None = None,
                 sink_value: float | None = None, chunk: int | None = None,
                 distance_bias: tuple[int, int] | None = None, value_mix: tuple[str, bool] | None = None,
                 pad_pages: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot share {num_kv_heads} kv heads evenly")
        if not 0 < head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head_dim must lie in 1..{MAX_HEAD_DIM}, got {head_dim}")
        self.hidden, self.n_heads, self.n_kv, self.head_dim = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.qk_norm_eps = qk_norm_eps
        self.positions = positions
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim) if positions else 0
        if self.rotary_dim % 2 or self.rotary_dim > head_dim:
            raise ValueError(f"the rotated width must be even and at most head_dim ({head_dim}), got {self.rotary_dim}")
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # model.py:65
        self.value_dim = int(value_dim) if value_dim else self.head_dim
        if not 0 < self.value_dim <= MAX_HEAD_DIM:
            raise ValueError(f"value_dim must lie in 1..{MAX_HEAD_DIM}, got {value_dim}")
        self.softcap = float(softcap) if softcap else 0.0
        if output_gate not in (False, True, "head"):
            raise ValueError(f"output_gate is False, True (a gate per feature) or 'head', got {output_gate!r}")
        self.has_sink, self.output_gate, self.float_weights = bool(sink), bool(output_gate), bool(float_weights)
        self.head_gate = output_gate == "head"
        self.sink_value = None if sink_value is None else float(sink_value)
        if self.has_sink and self.sink_value is not None:
            raise ValueError("a sink is learned (sink) or fixed (sink_value), not both")
        self.chunk = int(chunk) if chunk else None
        if self.chunk and self.window:
            raise ValueError("a mixer has a window or chunks, not both")
        self.distance_bias = (int(distance_bias[0]), int(distance_bias[1])) if distance_bias else None
        if self.distance_bias and not (self.distance_bias[0] == -1 or 2 <= self.distance_bias[0] < 2 * self.distance_bias[1]):
            raise ValueError(f"a bias by distance needs at least 2 rows (-1: as many as the checkpoint holds) and a far "
                             f"distance beyond half of them, got {self.distance_bias}")
        self.value_mix = (str(value_mix[0]), bool(value_mix[1])) if value_mix else None
        self.pad_pages = bool(pad_pages)
        if self.pad_pages and positions:
            raise ValueError("pages of one padded width go with mixers that do not rotate")
        self.q_dim, self.kv_dim = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        self.v_dim, self.o_dim = self.n_kv * self.value_dim, self.n_heads * self.value_dim
        self.has_bias, self.conv_taps = bool(bias), int(conv_taps) if conv_taps else 0
        if self.conv_taps > ops.CONV_MAX_TAPS:
            raise ValueError(f"the convolution takes at most {ops.CONV_MAX_TAPS} taps, got {conv_taps}")
        self.g_dim = (self.n_heads if self.head_gate else self.o_dim) if self.output_gate else 0
        self.extended = bool(self.value_dim != self.head_dim or self.softcap or self.has_sink or self.output_gate or
                             self.float_weights or self.has_bias or self.conv_taps or self.sink_value is not None or
                             self.chunk or self.distance_bias or self.value_mix)
        self.conv_channels = self.q_dim + self.kv_dim + self.v_dim
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = self.sink = None
        self.in_bias = self.o_bias = self.conv_w = self.conv_wt = self.rel = self.vmix = self.w_o_padded = None

    def tensor_specs(self):
        specs = {"q_proj": matrix((self.q_dim, self.hidden)), "k_proj": matrix((self.kv_dim, self.hidden)),
                 "v_proj": matrix((self.v_dim, self.hidden)), "o_proj": matrix((self.hidden, self.o_dim))}
        if self.has_sink:
            specs["sink"] = ((self.n_heads,), VECTOR, "normal")
        if self.output_gate:
            specs["g_proj"] = matrix((self.g_dim, self.hidden))
        if self.distance_bias:
            specs["rel"] = ((self.distance_bias[0], self.n_heads), VECTOR, "normal")
        if self.value_mix:
            specs["vmix"] = ((), VECTOR, "normal")
        if self.qk_norm_eps is not None:
            specs["q_norm"] = ((self.head_dim,), VECTOR, "ones")
            specs["k_norm"] = ((self.head_dim,), VECTOR, "ones")
        if self.has_bias:
            specs.update({"q_bias": ((self.q_dim,), VECTOR, "normal"), "k_bias": ((self.kv_dim,), VECTOR, "normal"),
                          "v_bias": ((self.v_dim,), VECTOR, "normal"), "o_bias": ((self.hidden,), VECTOR, "normal")})
        if self.conv_taps:
            specs.update({"q_conv": matrix((self.q_dim, self.conv_taps)), "k_conv": matrix((self.kv_dim, self.conv_taps)),
                          "v_conv": matrix((self.v_dim, self.conv_taps))})
        return specs

    def load(self, tensors):
        fused = [tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]] + ([tensors["g_proj"]] if self.output_gate else [])
        self.w_qkv = torch.cat(fused, dim=0).contiguous()
        if self.has_sink:
            self.sink = tensors["sink"].float().contiguous()
        elif self.sink_value is not None:
            self.sink = torch.full((self.n_heads,), self.sink_value, dtype=torch.float32, device=self.w_qkv.device)
        if self.distance_bias:
            # a row per distance 0..far, so that the kernels look a bias up without logarithms
            rows, far = tensors["rel"].shape[0], self.distance_bias[1]
            if not 2 <= rows < 2 * far:
                raise ValueError(f"a bias table of {rows} rows does not go with a far distance of {far}")
            reach = self.chunk or self.window                      # no row looks further back than that
            last = min(far, reach - 1) if reach else far
            index = torch.tensor([distance_row(n, rows, far) for n in range(last + 1)], device=self.w_qkv.device)
            self.rel = tensors["rel"].float()[index].contiguous()
        if self.value_mix:
            self.vmix = tensors["vmix"].float().reshape(1).contiguous()
        self.w_o = tensors["o_proj"]
        wide = self.page_dim()
        if wide and not self.output_gate:
            # nothing packs the heads' outputs between attention and the projection: the projection skips the padding
            padded = torch.zeros((self.hidden, self.n_heads, wide), dtype=self.w_o.dtype, device=self.w_o.device)
            padded[:, :, :self.value_dim] = self.w_o.view(self.hidden, self.n_heads, self.value_dim)
            self.w_o_padded = padded.view(self.hidden, self.n_heads * wide).contiguous()
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = tensors["q_norm"], tensors["k_norm"]
            if self.q_norm.dtype != self.k_norm.dtype or self.extended:   # one kernel argument says how both are stored
                self.q_norm, self.k_norm = self.q_norm.float().contiguous(), self.k_norm.float().contiguous()
        if self.has_bias:
            self.in_bias = torch.cat([tensors[n].float() for n in ("q_bias", "k_bias", "v_bias")]).contiguous()
            self.o_bias = tensors["o_bias"].float().contiguous()
        if self.conv_taps:
            self.conv_w = torch.cat([tensors[n].float() for n in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        elif self.has_bias:                   # the biases ride on a convolution of one tap
            self.conv_w = torch.ones((self.conv_channels, 1), dtype=torch.float32, device=self.in_bias.device)
        if self.conv_w is not None:
            self.conv_wt = self.conv_w.t().contiguous()                  # tap by tap, for 8 channels a thread

    def page_dim(self) -> int:
        """The one width of keys' and values' pages where ``pad_pages`` applies (bfloat16, widths that differ or are
        no multiple of the matrix cores' step, and the padded width within what the kernels take); else 0."""
        D, Dv, step = self.head_dim, self.value_dim, MATRIX_CORE_HEAD_STEP
        if not self.pad_pages or self.compute_dtype != torch.bfloat16 or (D == Dv and D % step == 0):
            return 0
        wide = -(-max(D, Dv) // step) * step
        return wide if wide <= MAX_HEAD_DIM else 0

    def cache_need(self):
        # a row of a chunked mixer never looks further back than a chunk: the pages behind that are given back
        wide = self.page_dim()
        kv = KVNeed(self.n_kv, wide or self.head_dim, self.window or self.chunk,
                    self.value_dim if self.value_dim != self.head_dim and not wide else None)
        if self.conv_taps > 1:
            return {"kv": kv, "tail": conv_need(self.conv_taps, self.conv_channels)}
        return kv

    def kernel_modules(self, dtype):
        return ("gemm", "rope_kv", "attn_rows") + (("attn_mfma",) if dtype == torch.bfloat16 else ()) + \
            (("activation",) if self.output_gate or self.value_mix else ()) + (("latent",) if self.head_gate else ()) + \
            (("conv", "norm") if self.conv_taps or self.has_bias else ())

    def _forward_general(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        """Every option, in float arithmetic on the kernel that takes one (row, head) a workgroup. Returns the output
        projection's result without its bias."""
        rows, H, G, D, Dv = h.shape[0], self.n_heads, self.n_kv, self.head_dim, self.value_dim
        tail = line["tail"] if isinstance(line, dict) and "tail" in line else None
        line = line["kv"] if isinstance(line, dict) else line
        cos = sin = table = None
        rot = 0
        if self.positions:
            table = ctx.positions[self.positions]
            if not isinstance(table, (PairRotaryPositions, HalfRotaryPositions)):
                raise NotImplementedError("the options of this attention go with a position encoding that has float tables")
            if ctx.max_kv_len > table.n_positions:
                raise ValueError(f"position tables cover {table.n_positions} positions, the step reaches {ctx.max_kv_len}")
            cos, sin, rot = table.cos, table.sin, table.dims
            if rot > D:
                raise ValueError(f"the position encoding rotates {rot} features, a head has {D}")
        proj = linear(h, self.w_qkv)                                    # q | k | v | gate
        src = proj
        if self.conv_w is not None:
            # biases and the short convolution: q | k | v as one run of channels, each with its own history
            src = short_conv(proj, 0, self.conv_channels, self.conv_w, ctx, tail, writes_cache, in_bias=self.in_bias,
                             weight_t=self.conv_wt)
        if self.value_mix:
            name, first = self.value_mix
            v_cols = src[:, self.q_dim + self.kv_dim:self.q_dim + self.kv_dim + self.v_dim]
            if first:
                ctx.shared["values:" + name] = v_cols
            else:
                earlier = ctx.shared.get("values:" + name)
                if earlier is None or earlier.shape != v_cols.shape:
                    raise ValueError(f"values {name!r}: no earlier layer of this step has left values of this shape")
                ops.blend_columns(v_cols, earlier, self.vmix)
        wide = self.page_dim()
        q = torch.zeros((rows, H, wide), dtype=h.dtype, device=h.device) if wide else \
            torch.empty((rows, H, D), dtype=h.dtype, device=h.device)
        if isinstance(table, PairRotaryPositions):
            if self.qk_norm_eps is not None:
                raise NotImplementedError("per-head q/k norms do not go with the rotation over neighbouring pairs")
            ops.rope_pairs_kv(src, 0, self.q_dim, self.q_dim + self.kv_dim, cos, sin, rot, ctx.row_slot, ctx.row_pos, q,
                              line.k, line.v, line.page_table, writes_cache, H, G, D, Dv)
        else:
            ops.norm_rope_half_kv(src, 0, self.q_dim, self.q_dim + self.kv_dim, self.q_norm, self.k_norm,
                                  self.qk_norm_eps or 0.0, cos, sin, rot, ctx.row_slot, ctx.row_pos, q, line.k, line.v,
                                  line.page_table, writes_cache, H, G, D, Dv, page_dim=wide)
        # bfloat16 on the matrix cores where they take the sizes (keys and values of one width, a multiple of 16, as
        # they are or padded); float32, and the other sizes, on the kernel that takes one (row, head) a workgroup
        matrix_cores = h.dtype == torch.bfloat16 and (wide or (D == Dv and D % MATRIX_CORE_HEAD_STEP == 0))
        if wide:
            D = Dv = wide                        # what the attention kernels see; o_dim keeps the values' own width
        window = self.window or 0
        if matrix_cores and ctx.max_q_len == 1:
            out = torch.empty((rows, H, Dv), dtype=h.dtype, device=h.device)
            splits = self.decode_splits(ctx.n_seqs, ctx.max_kv_len)
            part_o = torch.empty((ctx.n_seqs, H, splits, D), dtype=torch.float32, device=h.device)
            part_ml = torch.empty((ctx.n_seqs, H, splits, 2), dtype=torch.float32, device=h.device)
            ops.attn_split_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, ctx.kv_len, ctx.n_seqs,
                                part_o, part_ml, splits, out, H, G, D, self.scale, window, softcap=self.softcap,
                                sink=self.sink, chunk=self.chunk or 0, rel=self.rel)
        elif matrix_cores:
            # the tiled kernel never visits the rows of sequences that sit out; they must hold something finite
            out = ctx.kept_zeros((rows, H, Dv), h.dtype) if ctx.some_sit_out() else \
                torch.empty((rows, H, Dv), dtype=h.dtype, device=h.device)
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu, ctx.seq_start,
                                 ctx.n_seqs, max_tiles, out, H, G, D, self.scale, window, softcap=self.softcap,
                                 sink=self.sink, chunk=self.chunk or 0, rel=self.rel)
        else:
            out = torch.empty((rows, H, Dv), dtype=h.dtype, device=h.device)
            ops.attn_rows(q, line.k, line.v, line.page_table, ctx.row_slot, ctx.row_pos, out, H, G, D, self.scale,
                          window, v_dim=Dv, softcap=self.softcap, sink=self.sink, exact_p=self.float_weights,
                          chunk=self.chunk or 0, rel=self.rel)
        if self.output_gate:
            gated = torch.empty((rows, self.o_dim), dtype=h.dtype, device=h.device)
            g_col = self.q_dim + self.kv_dim + self.v_dim
            if self.head_gate or wide:           # this kernel also packs heads that are padded
                ops.head_gate(out, proj, g_col, gated, H, self.value_dim, per_element=not self.head_gate)
                out = gated
            else:
                out = ops.sigmoid_gate(out.view(rows, self.o_dim), proj[:, g_col:g_col + self.o_dim], gated)
            return linear(out, self.w_o, allow_partials=True)
        if wide:
            return linear(out.view(rows, H * wide), self.w_o_padded, allow_partials=True)
        return linear(out.view(rows, self.o_dim), self.w_o, allow_partials=True)

    def forward_split(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        if self.has_bias:
            return self._forward_general(h, ctx, line, writes_cache), self.o_bias
        return self.forward(h, ctx, line, writes_cache), None

    def forward(self, h: torch.Tensor, ctx: StepContext, line: KVLine, writes_cache: bool):
        if self.extended or (self.positions and not isinstance(ctx.positions[self.positions], RotaryPositions)):
            out = self._forward_general(h, ctx, line, writes_cache)
            return add_bias(out, self.o_bias, h.dtype) if self.has_bias else out
        rows = h.shape[0]
        # bfloat16 on the matrix cores where they take the head size; float32 and the other head sizes on the plain kernel
        matrix_cores = h.dtype == torch.bfloat16 and self.head_dim % MATRIX_CORE_HEAD_STEP == 0
        decoding = matrix_cores and ctx.max_q_len == 1
        fused_decoding = decoding and self.n_heads // self.n_kv <= 16
        # The kernel that norms, rotates, appends and attends in one adds up partial sums of the projection on its way
        # in, so K may be split over workgroups. Measured on Qwen3-4B's sizes, a decoding step with the split against
        # without: 2.980 against 3.008 ms at 8 sequences, 4.63 against 4.74 at 32, 6.75 against 6.86 at 64, 8.92 against
        # 9.04 at 96 and, since the product whose waves own rows of x, 5.89 against 5.97 at 192.
        cos = sin = None
        if self.positions:
            table = ctx.positions[self.positions]
            cos, sin = table.cos, table.sin
            if ctx.max_kv_len > table.n_positions:
                raise ValueError(f"position tables cover {table.n_positions} positions, the step reaches {ctx.max_kv_len}")
        # So does the kernel that takes a short prompt's keys and values to the cache (and its queries out): up to 256
        # rows the split product is ahead of the vendor library's (Qwen3-4B's q/k/v: 11.7 against 15.2 us at 64 rows,
        # 17.9 against 31.0 at 256).
        prompt_parts = matrix_cores and not decoding and writes_cache and cos is not None and \
            rows <= _PROMPT_PARTIAL_ROWS and \
            ops.rows_to_cache_takes(rows, self.head_dim, self.rotary_dim, True)
        if prompt_parts:
            qkv = linear(h, self.w_qkv, allow_partials=True)
        else:
            qkv = linear(h, self.w_qkv, allow_partials=fused_decoding, partial_rows=_QKV_PARTIAL_ROWS)
        window = self.window or 0
        # The tiled prompt kernels never visit the rows of sequences that sit out, and the projection after them reads
        # every row: where the step may hold such sequences the output lives in a tensor that started as zeros, so
        # that those rows hold zeros or an earlier layer's or step's output, never what memory happened to hold.
        if ctx.max_q_len > 1 and ctx.some_sit_out():
            out = ctx.kept_zeros((rows, self.n_heads, self.head_dim), h.dtype)
        else:
            out = torch.empty((rows, self.n_heads, self.head_dim), dtype=h.dtype, device=h.device)
        if decoding:
            splits = self.decode_splits(ctx.n_seqs, ctx.max_kv_len)
            part_o = torch.empty((ctx.n_seqs, self.n_heads, splits, self.head_dim), dtype=torch.float32, device=h.device)
            part_ml = torch.empty((ctx.n_seqs, self.n_heads, splits, 2), dtype=torch.float32, device=h.device)
        if fused_decoding:
            # one token per sequence: norm, rotation, append and attention in one kernel
            parts = qkv.count if isinstance(qkv, Partials) else 0
            ops.attn_decode_fused_bf16(qkv.data if parts else qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, self.rotary_dim,
                                       writes_cache, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows,
                                       ctx.kv_len, ctx.n_seqs, part_o, part_ml, splits, out, self.n_heads, self.n_kv,
                                       self.head_dim, self.scale, window, qkv_parts=parts)
            return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)
        if prompt_parts and isinstance(qkv, Partials):
            q = torch.empty((rows, self.n_heads, self.head_dim), dtype=h.dtype, device=h.device)
            ops.rows_to_cache_from_partials(qkv.data, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin,
                                            self.rotary_dim, ctx.row_slot, ctx.row_pos, q, line.k, line.v,
                                            line.page_table, self.n_heads, self.n_kv, self.head_dim)
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu,
                                 ctx.seq_start, ctx.n_seqs, max_tiles, out, self.n_heads, self.n_kv,
                                 self.head_dim, self.scale, window)
            return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)
        if matrix_cores and not decoding and cos is not None and \
                ops.attn_causal_takes_projection(self.head_dim, self.rotary_dim):
            # the prompt kernel norms and rotates the queries on their way in: only keys and values go to the cache here
            if writes_cache:
                ops.qk_norm_rope_kv(qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, self.rotary_dim,
                                    ctx.row_slot, ctx.row_pos, None, line.k, line.v, line.page_table, True,
                                    self.n_heads, self.n_kv, self.head_dim)
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_projected_bf16(qkv, self.q_norm, self.qk_norm_eps or 0.0, cos, sin, line.k, line.v,
                                           line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu, ctx.seq_start,
                                           ctx.n_seqs, max_tiles, out, self.n_heads, self.n_kv, self.head_dim,
                                           self.scale, window)
            return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)
        q = torch.empty((rows, self.n_heads, self.head_dim), dtype=h.dtype, device=h.device)
        ops.qk_norm_rope_kv(qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, self.rotary_dim,
                            ctx.row_slot, ctx.row_pos, q, line.k, line.v, line.page_table, writes_cache,
                            self.n_heads, self.n_kv, self.head_dim)
        if decoding:
            ops.attn_split_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, ctx.kv_len,
                                ctx.n_seqs, part_o, part_ml, splits, out, self.n_heads, self.n_kv, self.head_dim,
                                self.scale, window)
        elif matrix_cores:
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu,
                                 ctx.seq_start, ctx.n_seqs, max_tiles, out, self.n_heads, self.n_kv,
                                 self.head_dim, self.scale, window)
        else:
            ops.attn_rows(q, line.k, line.v, line.page_table, ctx.row_slot, ctx.row_pos, out, self.n_heads, self.n_kv,
                          self.head_dim, self.scale, window)
        return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)

    def flops(self, rows, spans):
        """The projections, and both attention products over the keys each row sees."""
        seen = 0
        for start, q in spans:
            first, last = start + 1, start + q                  # keys that the span's first and last row see
            if self.window:
                full = max(0, min(last, self.window) - first + 1)          # rows that still see every key
                seen += (2 * first + full - 1) * full // 2 + (q - full) * self.window
            elif self.chunk:
                seen += sum(p % self.chunk + 1 for p in range(start, start + q))
            else:
                seen += (first + last) * q // 2
        return super().flops(rows, spans) + 2.0 * (self.q_dim + self.o_dim) * seen

    def decode_splits(self, n_seqs: int, max_kv_len: int) -> int:
        """How many ways each sequence's keys are split: as many as run at the same time, and no more.

        Workgroups beyond what the chip holds at once start when the first ones end, which costs more than
        the longer walk of fewer, larger splits.
        """
        blocks = self.n_kv * ((self.n_heads // self.n_kv + 15) // 16)
        want = _RESIDENT_WORKGROUPS // (n_seqs * blocks)
        span = self.window or getattr(self, "chunk", None) or max_kv_len
        pages = max(1, (span + 63) // 64)
        return max(1, min(want, _MAX_SPLITS, pages))


register_part("gqa_attention", GQAAttention)
