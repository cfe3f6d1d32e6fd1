"""Python faces of the HIP kernels: argument checks, then one ctypes call each.

Every function checks on the host that the operands have the dtypes, shapes and
strides its kernel assumes, and raises rather than launch a kernel that would read
outside its operands. Kernels run on torch's current stream, so they can be
recorded into a graph like any other work on it. There is no CPU path: tensors
must live on the GPU, and a missing library is compiled or the call fails.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from . import build

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float
_SIGNATURES = {
    "batch": {"dryft_prepare_batch": [_P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P],
              "dryft_tile_prefix": [_P, _P, _I, _I, _P, _P]},
    "embed": {"dryft_embed_rows": [_P, _P, _P, _I, _I, _I, _I, _I, _P],
              "dryft_embed_scaled": [_P, _P, _P, _I, _I, _I, _F, _I, _P]},
    "norm": {"dryft_add_rmsnorm": [_P, _P, _I, _I, _L, _P, _I, _P, _P, _I, _I, _F, _I, _P],
             "dryft_add_rows": [_P, _P, _P, _L, _I, _P],
             "dryft_stream_norm": [_P, _I, _P, _I, _I, _L, _P, _I, _P, _P, _I, _P, _I, _P, _P, _I, _I, _F, _I, _I, _P],
             "dryft_rms_pair_mean": [_P, _I, _I, _L, _P, _P, _P, _I, _I, _L, _P, _P, _P, _I, _I, _F, _I, _P]},
    "activation": {"dryft_silu_mul": [_P, _P, _I, _I, _L, _I, _P],
                   "dryft_glu_clamped": [_P, _P, _I, _I, _L, _F, _F, _I, _P],
                   "dryft_sigmoid_gate": [_P, _L, _P, _L, _P, _I, _I, _I, _P],
                   "dryft_relu_squared": [_P, _L, _P, _I, _I, _I, _P],
                   "dryft_token_gate": [_P, _L, _P, _P, _L, _I, _I, _P, _I, _I, _I, _P],
                   "dryft_blend_columns": [_P, _L, _P, _L, _P, _I, _I, _I, _P]},
    "mlstm": {"dryft_mlstm_steps": [_P, _L, _I, _I, _I, _P, _P, _P, _F, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _F,
                                    _I, _I, _P],
              "dryft_mlstm_chunks_takes": [_I, _I, _I, _I, _I, _L],
              "dryft_mlstm_chunks": [_P, _L, _I, _I, _I, _P, _P, _P, _F, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _F,
                                     _I, _I, _P, _I, _P, _P],
              "dryft_mlstm_out": [_P, _P, _L, _I, _P, _P, _P, _I, _I, _I, _F, _I, _P]},
    "rglru": {"dryft_rglru_gates": [_P, _L, _I, _P, _P, _P, _I, _P, _P, _P, _P, _P, _F, _P, _P, _P, _P, _P, _P, _I, _I,
                                    _I, _I, _P],
              "dryft_rglru_tile_rows": [],
              "dryft_rglru_scan_tiles": [_P, _P, _P, _L, _I, _I, _P, _P, _I, _P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I,
                                         _I, _P],
              "dryft_rglru_scan": [_P, _P, _L, _I, _I, _P, _P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _P]},
    "rope_kv": {"dryft_qk_norm_rope_kv": [_P, _L, _P, _P, _I, _I, _F, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I,
                                          _I, _I, _I, _I, _I, _P],
                "dryft_rope_pairs_kv": [_P, _L, _I, _I, _I, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I,
                                        _I, _I, _P],
                "dryft_norm_rope_half_kv": [_P, _L, _I, _I, _I, _P, _P, _F, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I,
                                            _I, _I, _I, _I, _I, _I, _P],
                "dryft_rows_to_cache_takes": [_I, _I, _I, _I],
                "dryft_rows_to_cache_parts": [_P, _I, _L, _P, _P, _I, _I, _F, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I,
                                              _I, _I, _I, _P]},
    "attn_rows": {"dryft_attn_rows": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _F, _P, _I, _I, _P, _I, _I, _P]},
    "attn_mfma": {"dryft_attn_causal_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _P, _I, _I, _I, _F, _I, _I, _F, _P,
                                             _I, _P, _I, _P],
                  "dryft_attn_causal_takes_projection": [_I, _I],
                  "dryft_attn_causal_projected_bf16": [_P, _L, _P, _I, _I, _F, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I,
                                                       _I, _P, _I, _I, _I, _F, _I, _I, _P],
                  "dryft_attn_split_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _P, _P, _I, _P, _I, _I, _I, _F, _I,
                                            _F, _P, _I, _P, _I, _P],
                  "dryft_attn_decode_fused_bf16": [_P, _L, _I, _L, _P, _P, _I, _I, _F, _P, _P, _I, _I, _P, _P, _P, _I, _P, _P,
                                                   _P, _I, _P, _P, _I, _P, _I, _I, _I, _F, _I, _P]},
    "gemm": {"dryft_gemm_tiled": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_stream_bf16": [_P, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_stream_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_wide_bf16": [_P, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_panel_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_panel_glu_clamped_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _F, _F, _P],
             "dryft_gemm_panel_waves": [_I],
             "dryft_gemm_tall_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_tall_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_tall_tiles": [_I],
             "dryft_gemm_mid_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_block_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_block_f32": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_rows_f32": [_P, _L, _P, _P, _I, _I, _I, _P],
             "dryft_gemm_wide_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_sum_partials": [_P, _P, _L, _I, _I, _P]},
    "hyper": {"dryft_hyper_norm": [_P, _I, _I, _P, _I, _I, _L, _P, _P, _P, _P, _P, _P, _I, _I, _I, _F, _I, _P]},
    "wkv": {"dryft_wkv_blend": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
            "dryft_wkv_decay": [_P, _P, _P, _P, _I, _I, _I, _I, _P],
            "dryft_wkv_steps": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _P, _I, _I, _P, _P, _I,
                                _P],
            "dryft_wkv_out": [_P, _P, _P, _P, _I, _I, _I, _F, _L, _I, _P]},
    "latent": {"dryft_rms_segments": [_P, _L, _I, _P, _P, _I, _P, _P, _I, _F, _I, _I, _P],
               "dryft_latent_rope_kv": [_P, _P, _P, _L, _I, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I,
                                        _I, _I, _I, _I, _P],
               "dryft_head_gate": [_P, _P, _L, _I, _P, _I, _I, _I, _I, _I, _I, _P]},
    "moe": {"dryft_moe_route": [_P, _L, _P, _I, _I, _I, _I, _F, _P, _P, _I, _I, _I, _I, _P],
            "dryft_moe_plan": [_P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _P],
            "dryft_moe_product": [_P, _L, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _F, _F, _I, _I, _I, _P],
            "dryft_moe_table_route": [_P, _P, _P, _P, _I, _I, _I, _I, _P],
            "dryft_moe_combine": [_P, _P, _P, _P, _P, _L, _I, _P, _I, _I, _I, _I, _P]},
    "conv": {"dryft_conv_max_taps": [],
             "dryft_causal_conv": [_P, _L, _I, _P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
             "dryft_conv_tail": [_P, _L, _I, _P, _I, _P, _P, _P, _P, _I, _I, _I, _P]},
    "ssm": {"dryft_ssm_max_state": [],
            "dryft_ssm_scan": [_P, _L, _I, _I, _I, _P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I,
                               _I, _P, _P, _I, _P],
            "dryft_gate_part_norm": [_P, _P, _L, _I, _P, _P, _P, _I, _I, _I, _F, _I, _P]},
    "delta": {"dryft_delta_max_dim": [],
              "dryft_delta_steps": [_P, _L, _I, _I, _I, _P, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I,
                                    _F, _F, _I, _P, _I, _I, _P, _P, _I, _P]},
    "sampling": {"dryft_argmax_rows": [_P, _I, _I, _L, _P, _I, _P, _P, _P],
                 "dryft_sample_rows": [_P, _I, _I, _L, _F, _P, _P, _I, _P, _P, _P]},
}
_functions: dict[str, object] = {}


class KernelError(RuntimeError):
    pass


def _fn(module: str, name: str):
    f = _functions.get(name)
    if f is None:
        lib = build.load(module)
        f = getattr(lib, name)
        f.argtypes = _SIGNATURES[module][name]
        f.restype = c_int
        _functions[name] = f
    return f


def preload(modules) -> None:
    build.ensure(list(modules))


# the current stream's handle without building a stream object per launch (hundreds of launches a step)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(rc: int, what: str) -> None:
    if rc == -1:
        raise KernelError(f"{what}: the kernel refuses these sizes")
    if rc != 0:
        raise KernelError(f"{what}: launch failed with HIP error {rc}")


def _gpu(t: torch.Tensor, name: str, dtype=None) -> None:
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise KernelError(f"{name}: must be a GPU tensor (there is no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")


def _float_flag(t: torch.Tensor, name: str) -> int:
    if t.dtype not in (torch.float32, torch.bfloat16):
        raise KernelError(f"{name}: expected float32 or bfloat16, got {t.dtype}")
    return 1 if t.dtype == torch.float32 else 0


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ------------------------------------------------------------------------------------------- batch
def prepare_batch(seq_slot, q_len, lengths, n_seqs: int, n_rows: int, cu_rows, kv_len, seq_start,
                  row_seq, row_slot, row_pos) -> None:
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("q_len", q_len, n_seqs), ("cu_rows", cu_rows, n_seqs + 1),
                       ("kv_len", kv_len, n_seqs), ("seq_start", seq_start, n_seqs),
                       ("row_seq", row_seq, n_rows), ("row_slot", row_slot, n_rows), ("row_pos", row_pos, n_rows),
                       ("lengths", lengths, 1)):
        _gpu(t, name, torch.int32)
        if not (t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"{name}: needs {n} contiguous entries, has {t.numel()}")
    _check(_fn("batch", "dryft_prepare_batch")(
        _ptr(seq_slot), _ptr(q_len), _ptr(lengths), n_seqs, n_rows, _ptr(cu_rows), _ptr(kv_len),
        _ptr(seq_start), _ptr(row_seq), _ptr(row_slot), _ptr(row_pos), _stream()), "prepare_batch")


def tile_prefix(seq_slot, q_len, n_seqs: int, tile_rows: int, tile_cu) -> None:
    """``tile_cu[s]``: how many tiles of ``tile_rows`` rows the sequences before ``s`` fill with their rows of this
    step (a sequence that sits out, slot -1, fills none); ``tile_cu[n_seqs]``: the step's tiles."""
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("q_len", q_len, n_seqs), ("tile_cu", tile_cu, n_seqs + 1)):
        _gpu(t, name, torch.int32)
        if not (t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"{name}: needs {n} contiguous entries, has {t.numel()}")
    if tile_rows <= 0:
        raise KernelError(f"tile_prefix: tiles of {tile_rows} rows")
    _check(_fn("batch", "dryft_tile_prefix")(_ptr(seq_slot), _ptr(q_len), n_seqs, int(tile_rows), _ptr(tile_cu),
                                             _stream()), "tile_prefix")


# ------------------------------------------------------------------------------------------- embed
def embed_rows(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[r] = table[tokens[r]]`` for a table ``[vocab, hidden]``; for several tables ``[tables, vocab, hidden]`` the same
    rows of each, ``out[t, r] = table[t, tokens[r]]``."""
    _gpu(tokens, "tokens", torch.int32)
    _gpu(table, "table")
    _gpu(out, "out", table.dtype)
    n = tokens.numel()
    tables = table.shape[0] if table.dim() == 3 else 1
    vocab, hidden = table.shape[-2:]
    if not (table.dim() in (2, 3) and table.is_contiguous() and out.is_contiguous() and tokens.is_contiguous()):
        raise KernelError("embed_rows: contiguous operands, the table [vocab, hidden] or [tables, vocab, hidden]")
    want = (n, hidden) if table.dim() == 2 else (tables, n, hidden)
    if not (out.shape == want):
        raise KernelError(f"embed_rows: out is {tuple(out.shape)}, expected {want}")
    _check(_fn("embed", "dryft_embed_rows")(_ptr(tokens), _ptr(table), _ptr(out), n, hidden, vocab, tables,
                                            _float_flag(table, "table"), _stream()), "embed_rows")
    return out


# -------------------------------------------------------------------------------------------- norm
def add_rmsnorm(res: torch.Tensor, delta, weight: torch.Tensor, eps: float, res_out, y: torch.Tensor,
                n_partials: int = 1) -> None:
    """``res_out = res + delta`` (when ``delta`` is given) and ``y = rmsnorm(res_out) * weight``.

    ``delta`` is ``[rows, width]`` in the dtype of ``res``, or ``[n_partials, rows, width]`` float32
    partial sums. Without ``delta`` nothing is added and ``res_out`` is ignored.
    """
    _gpu(res, "res")
    rows, width = res.shape
    is_f32 = _float_flag(res, "res")
    _gpu(weight, "weight")
    w_f32 = _float_flag(weight, "weight")
    if not (weight.shape == (width,) and weight.is_contiguous()):
        raise KernelError(f"add_rmsnorm: weight must be [{width}]")
    _gpu(y, "y", res.dtype)
    if not (res.is_contiguous() and y.is_contiguous() and y.shape == res.shape):
        raise KernelError("add_rmsnorm: res and y contiguous, same shape")
    kind, stride = 0, 0
    if delta is not None:
        _gpu(delta, "delta")
        _gpu(res_out, "res_out", res.dtype)
        if not (res_out.shape == res.shape and res_out.is_contiguous()):
            raise KernelError("add_rmsnorm: res_out like res")
        if not (delta.is_contiguous()):
            raise KernelError("add_rmsnorm: delta contiguous")
        if delta.dim() == 3:
            if not (delta.dtype == torch.float32 and delta.shape[1:] == res.shape and delta.shape[0] >= n_partials):
                raise KernelError("add_rmsnorm: partial sums must be float32 [n, rows, width]")
            kind, stride = 2, rows * width
        else:
            if not (delta.dtype == res.dtype and delta.shape == res.shape):
                raise KernelError("add_rmsnorm: delta like res")
            kind, n_partials, stride = 1, 1, rows * width
    else:
        n_partials = 0
    _check(_fn("norm", "dryft_add_rmsnorm")(_ptr(res), _ptr(delta), kind, n_partials, stride, _ptr(weight), w_f32,
                                            _ptr(res_out), _ptr(y), rows, width, float(eps), is_f32, _stream()),
           "add_rmsnorm")


def add_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(a, "a")
    _gpu(b, "b", a.dtype)
    _gpu(out, "out", a.dtype)
    if not (a.shape == b.shape == out.shape and a.is_contiguous() and b.is_contiguous() and out.is_contiguous()):
        raise KernelError("add_rows: contiguous operands of one shape")
    _check(_fn("norm", "dryft_add_rows")(_ptr(a), _ptr(b), _ptr(out), a.numel(), _float_flag(a, "a"), _stream()),
           "add_rows")
    return out


def stream_norm(x, delta, post_weight, extra, vec, weight, eps: float, x_out, y, act: torch.dtype,
                post_centred: bool = False, centred: bool = False, plain_read: bool = False) -> None:
    """The norms of a float32 residual stream in one launch, per row (``post_centred`` / ``centred``: the norm of
    ``d`` / of ``x_out`` takes the mean off first and divides by the standard deviation, a layer norm without bias;
    ``plain_read``: ``y`` is ``x_out`` itself in the activation dtype, no weight):
    ``d = delta`` (a tensor in the activation dtype, or ``[n, rows, width]`` float32 partial sums as ``(data, n)``);
    ``x_out = x + rmsnorm(d) * post_weight + extra + vec`` (each term optional; without ``post_weight`` ``d`` is added
    as it is); ``y = rmsnorm(x_out) * weight`` in the activation dtype (optional). ``x`` is float32, or in the
    activation dtype ``act`` (a stream that starts), or None; ``x_out`` is float32 (may be ``x`` itself) or None."""
    ref = y if y is not None else (x_out if x_out is not None else x)
    rows, width = ref.shape
    x_kind = 0
    if x is not None:
        _gpu(x, "x")
        if not (x.shape == (rows, width) and x.is_contiguous()):
            raise KernelError("stream_norm: x must be contiguous [rows, width]")
        x_kind = 1 if (x.dtype == act and x is not x_out) else 2
    n_partials, kind, stride = 0, 0, 0
    if delta is not None:
        data, n_partials = delta if isinstance(delta, tuple) else (delta, 1)
        _gpu(data, "delta")
        if isinstance(delta, tuple):
            if not (data.dtype == torch.float32 and data.dim() == 3 and data.shape[1:] == (rows, width) and
                    data.is_contiguous() and data.shape[0] >= n_partials >= 1):
                raise KernelError("stream_norm: partial sums must be contiguous float32 [n, rows, width]")
            kind, stride = 2, rows * width
        else:
            if not (data.shape == (rows, width) and data.is_contiguous()):
                raise KernelError("stream_norm: delta must be contiguous [rows, width]")
            kind = 1
        delta = data
    for name, t in (("post_weight", post_weight), ("vec", vec), ("weight", weight)):
        if t is not None:
            _gpu(t, name)
            _float_flag(t, name)
            if not (t.shape == (width,) and t.is_contiguous()):
                raise KernelError(f"stream_norm: {name} must be [{width}]")
    is_f32 = 1 if act == torch.float32 else 0
    if kind == 1 and delta.dtype != act or x_kind == 2 and x.dtype != torch.float32:
        raise KernelError("stream_norm: delta must be in the activation dtype, the stream in it or in float32")
    if extra is not None:
        _gpu(extra, "extra", act)
        if not (extra.shape == (rows, width) and extra.is_contiguous()):
            raise KernelError("stream_norm: extra must be contiguous [rows, width]")
    if x_out is not None:
        _gpu(x_out, "x_out", torch.float32)
        if not (x_out.shape == (rows, width) and x_out.is_contiguous()):
            raise KernelError("stream_norm: x_out must be contiguous float32 [rows, width]")
    if y is not None:
        _gpu(y, "y", act)
        if not (y.is_contiguous() and (weight is not None or plain_read)):
            raise KernelError("stream_norm: y contiguous, and a weight for it")
    flag = lambda t: 0 if t is None else _float_flag(t, "vector")      # noqa: E731
    _check(_fn("norm", "dryft_stream_norm")(
        _ptr(x), x_kind, _ptr(delta), kind, n_partials, stride, _ptr(post_weight), flag(post_weight), _ptr(extra),
        _ptr(vec), flag(vec), _ptr(weight), flag(weight), _ptr(x_out), _ptr(y), rows, width, float(eps), is_f32,
        (1 if post_centred else 0) | (2 if centred else 0) | (4 if plain_read else 0), _stream()), "stream_norm")


# -------------------------------------------------------------------------------------- activation
def glu_clamped(gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """``out = g * sigmoid(alpha * g) * (u + 1)`` with ``g = min(gate_up[:, :I], limit)`` and
    ``u = clamp(gate_up[:, I:], -limit, limit)``."""
    _gpu(gate_up, "gate_up")
    _gpu(out, "out", gate_up.dtype)
    rows, two = gate_up.shape
    inter = two // 2
    if not (two == 2 * inter and gate_up.stride(1) == 1 and out.shape == (rows, inter) and out.is_contiguous()):
        raise KernelError("glu_clamped: gate_up [rows, 2I] with unit column stride, out contiguous [rows, I]")
    _check(_fn("activation", "dryft_glu_clamped")(_ptr(gate_up), _ptr(out), rows, inter, gate_up.stride(0), float(limit),
                                                  float(alpha), _float_flag(gate_up, "gate_up"), _stream()),
           "glu_clamped")
    return out


def sigmoid_gate(a: torch.Tensor, gate: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out = a * sigmoid(gate)``; ``a`` and ``gate`` are ``[rows, width]`` and may be column runs of wider tensors."""
    _gpu(a, "a")
    _gpu(gate, "gate", a.dtype)
    _gpu(out, "out", a.dtype)
    rows, width = a.shape
    if not (gate.shape == a.shape and a.stride(1) == 1 and gate.stride(1) == 1 and out.shape == a.shape and
            out.is_contiguous()):
        raise KernelError("sigmoid_gate: a and gate [rows, width] with unit column stride, out contiguous")
    _check(_fn("activation", "dryft_sigmoid_gate")(_ptr(a), a.stride(0), _ptr(gate), gate.stride(0), _ptr(out), rows,
                                                   width, _float_flag(a, "a"), _stream()), "sigmoid_gate")
    return out


def relu_squared(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out = max(x, 0)^2``; ``x`` is ``[rows, width]`` and may be a column run of a wider tensor."""
    _gpu(x, "x")
    _gpu(out, "out", x.dtype)
    rows, width = x.shape
    if not (x.stride(1) == 1 and out.shape == x.shape and out.is_contiguous()):
        raise KernelError("relu_squared: x [rows, width] with unit column stride, out contiguous")
    _check(_fn("activation", "dryft_relu_squared")(_ptr(x), x.stride(0), _ptr(out), rows, width, _float_flag(x, "x"),
                                                   _stream()), "relu_squared")
    return out


def token_gate(gate: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor, col: int, out: torch.Tensor) -> torch.Tensor:
    """``out[r] = gelu_tanh(gate[r]) * table[tokens[r], col : col + width]``: a gate on the numbers a token id brings."""
    _gpu(gate, "gate")
    _gpu(tokens, "tokens", torch.int32)
    _gpu(table, "table", gate.dtype)
    _gpu(out, "out", gate.dtype)
    rows, width = gate.shape
    if not (gate.stride(1) == 1 and out.shape == gate.shape and out.is_contiguous() and tokens.numel() >= rows and
            tokens.is_contiguous()):
        raise KernelError("token_gate: gate [rows, width] with unit column stride, out contiguous, a token id a row")
    if not (table.dim() == 2 and table.stride(1) == 1 and 0 <= col and col + width <= table.shape[1]):
        raise KernelError("token_gate: the run of columns lies outside the table")
    _check(_fn("activation", "dryft_token_gate")(_ptr(gate), gate.stride(0), _ptr(tokens), _ptr(table), table.stride(0),
                                                 int(col), table.shape[0], _ptr(out), rows, width,
                                                 _float_flag(gate, "gate"), _stream()), "token_gate")
    return out


def blend_columns(a: torch.Tensor, b: torch.Tensor, lam: torch.Tensor) -> torch.Tensor:
    """``a <- (1 - lam) a + lam b`` in place; ``a`` and ``b`` are ``[rows, width]`` column runs of wider tensors,
    ``lam`` one float32 on the device."""
    _gpu(a, "a")
    _gpu(b, "b", a.dtype)
    _gpu(lam, "lam", torch.float32)
    if not (a.dim() == 2 and a.shape == b.shape and a.stride(1) == 1 and b.stride(1) == 1 and lam.numel() == 1):
        raise KernelError("blend_columns: a and b [rows, width] with unit column stride, lam one number")
    _check(_fn("activation", "dryft_blend_columns")(_ptr(a), a.stride(0), _ptr(b), b.stride(0), _ptr(lam), a.shape[0],
                                                    a.shape[1], _float_flag(a, "a"), _stream()), "blend_columns")
    return a


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(gate_up, "gate_up")
    _gpu(out, "out", gate_up.dtype)
    rows, two_i = gate_up.shape
    if not (two_i % 2 == 0 and out.shape == (rows, two_i // 2)):
        raise KernelError("silu_mul: out must be [rows, width / 2]")
    if not (gate_up.stride(1) == 1 and out.is_contiguous()):
        raise KernelError("silu_mul: unit stride along the width")
    _check(_fn("activation", "dryft_silu_mul")(_ptr(gate_up), _ptr(out), rows, two_i // 2, gate_up.stride(0),
                                               _float_flag(gate_up, "gate_up"), _stream()), "silu_mul")
    return out


# ----------------------------------------------------------------------------------------- rope_kv
def qk_norm_rope_kv(qkv: torch.Tensor, q_weight, k_weight, eps: float, cos, sin, rot: int, row_slot, row_pos,
                    q_out, k_pages, v_pages, page_table, write_kv: bool, n_heads: int, n_kv: int,
                    head_dim: int) -> None:
    """Per-head norm and rotation of a step's query and key heads, and the append of keys and values to the cache.
    ``q_out`` None: only keys and values are handled (the attention kernel takes the queries from ``qkv`` itself)."""
    _gpu(qkv, "qkv")
    is_f32 = _float_flag(qkv, "qkv")
    rows = qkv.shape[0]
    need_cols = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    if not (qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= need_cols):
        raise KernelError(f"qk_norm_rope_kv: qkv needs {need_cols} columns, has {tuple(qkv.shape)}")
    has_norm = q_weight is not None
    w_f32 = 0
    if has_norm:
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            _gpu(w, name)
            if not (w.shape == (head_dim,) and w.is_contiguous()):
                raise KernelError(f"{name}: must be [{head_dim}]")
        if not (q_weight.dtype == k_weight.dtype):
            raise KernelError("q_weight and k_weight must share a dtype")
        w_f32 = _float_flag(q_weight, "q_weight")
    if rot:
        if not (rot % 2 == 0 and rot <= head_dim):
            raise KernelError(f"rotary width {rot} must be even and at most {head_dim}")
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, qkv.dtype)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be [positions, {rot // 2}]")
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows and t.is_contiguous()):
            raise KernelError(f"{name}: needs {rows} entries")
    if q_out is not None:
        _gpu(q_out, "q_out", qkv.dtype)
        if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * head_dim):
            raise KernelError("q_out: must be [rows, heads, head_dim]")
    else:
        if not (write_kv):
            raise KernelError("qk_norm_rope_kv: nothing to do without q_out and without a cache to write")
    max_pages = 0
    if write_kv:
        _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, qkv.dtype)
        max_pages = page_table.shape[1]
    _check(_fn("rope_kv", "dryft_qk_norm_rope_kv")(
        _ptr(qkv), qkv.stride(0), _ptr(q_weight), _ptr(k_weight), w_f32, int(has_norm), float(eps), _ptr(cos),
        _ptr(sin), int(rot), _ptr(row_slot), _ptr(row_pos), _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
        _ptr(page_table), max_pages, int(write_kv), rows, n_heads, n_kv, head_dim, is_f32, _stream()),
        "qk_norm_rope_kv")


def rows_to_cache_takes(n_rows: int, head_dim: int, rot: int, write_kv: bool) -> bool:
    """Can ``rows_to_cache_from_partials`` take a step of so many rows, heads of this size rotated over ``rot``
    features?"""
    return bool(_fn("rope_kv", "dryft_rows_to_cache_takes")(int(n_rows), int(head_dim), int(rot), int(write_kv)))


def rows_to_cache_from_partials(parts: torch.Tensor, q_weight, k_weight, eps: float, cos, sin, rot: int, row_slot,
                                row_pos, q_out, k_pages, v_pages, page_table, n_heads: int, n_kv: int,
                                head_dim: int) -> None:
    """``qk_norm_rope_kv`` for a bfloat16 step whose projection was left as float partial sums ``parts`` [count, rows,
    columns]: each value is the sum of its parts rounded to bfloat16, then normed, rotated and written as there (queries
    to ``q_out``, or nowhere if it is None; keys and values to the cache)."""
    _gpu(parts, "parts", torch.float32)
    if not (parts.dim() == 3 and parts.is_contiguous()):
        raise KernelError("rows_to_cache_from_partials: parts must be [count, rows, columns], contiguous")
    count, rows, cols = parts.shape
    if not (cols >= (n_heads + 2 * n_kv) * head_dim and cols % 8 == 0):
        raise KernelError(f"rows_to_cache_from_partials: parts need {(n_heads + 2 * n_kv) * head_dim} columns, a multiple "
                          f"of 8; have {cols}")
    if not rows_to_cache_takes(rows, head_dim, rot, True):
        raise KernelError(f"rows_to_cache_from_partials: takes a full rotation and head sizes 32, 64, 128, 256; got head "
                          f"size {head_dim}, rotation over {rot}")
    has_norm = q_weight is not None
    w_f32 = 0
    if has_norm:
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            _gpu(w, name)
            if not (w.shape == (head_dim,) and w.is_contiguous()):
                raise KernelError(f"{name}: must be [{head_dim}]")
        if not (q_weight.dtype == k_weight.dtype):
            raise KernelError("q_weight and k_weight must share a dtype")
        w_f32 = _float_flag(q_weight, "q_weight")
    for name, t in (("cos", cos), ("sin", sin)):
        _gpu(t, name, torch.bfloat16)
        if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
            raise KernelError(f"{name}: must be [positions, {rot // 2}]")
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows and t.is_contiguous()):
            raise KernelError(f"{name}: needs {rows} entries")
    if q_out is not None:
        _gpu(q_out, "q_out", torch.bfloat16)
        if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * head_dim):
            raise KernelError("q_out: must be [rows, heads, head_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    _check(_fn("rope_kv", "dryft_rows_to_cache_parts")(
        _ptr(parts), int(count), cols, _ptr(q_weight), _ptr(k_weight), w_f32, int(has_norm), float(eps), _ptr(cos),
        _ptr(sin), int(rot), _ptr(row_slot), _ptr(row_pos), _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
        _ptr(page_table), page_table.shape[1], rows, n_heads, n_kv, head_dim, _stream()), "rows_to_cache_parts")


def _check_pages(k_pages, v_pages, page_table, n_kv: int, head_dim: int, dtype, v_dim: int | None = None) -> None:
    for name, t, d in (("k_pages", k_pages, head_dim), ("v_pages", v_pages, head_dim if v_dim is None else v_dim)):
        _gpu(t, name, dtype)
        if not (t.dim() == 4 and t.shape[1] == n_kv and t.shape[2] * t.shape[3] == 64 * d and t.is_contiguous()):
            raise KernelError(f"{name}: must be contiguous [pages, {n_kv}, 64, {d}], got {tuple(t.shape)}")
    if k_pages.shape[0] != v_pages.shape[0]:
        raise KernelError("k_pages and v_pages: different numbers of pages")
    _gpu(page_table, "page_table", torch.int32)
    if not (page_table.dim() == 2 and page_table.is_contiguous()):
        raise KernelError("page_table: must be contiguous [slots, pages]")


# --------------------------------------------------------------------------------------- attention
def attn_rows(q, k_pages, v_pages, page_table, row_slot, row_pos, out, n_heads: int, n_kv: int, head_dim: int,
              scale: float, window: int, *, v_dim: int | None = None, softcap: float = 0.0, sink=None,
              exact_p: bool = False, chunk: int = 0, rel=None) -> None:
    """``v_dim``: the values' width where it differs from the keys'; ``softcap`` > 0: scores become
    ``cap * tanh(s / cap)``; ``sink``: float32 ``[heads]`` whose exp() joins each head's denominator; ``exact_p``:
    the probabilities weigh the values unrounded; ``chunk`` > 0: a row sees the keys of its own run of so many
    positions instead of a window; ``rel``: float32 ``[distances, heads]``, a bias by distance added to the scaled
    score (the last row serves every larger distance)."""
    _gpu(q, "q")
    is_f32 = _float_flag(q, "q")
    v_dim = head_dim if v_dim is None else int(v_dim)
    rows = q.numel() // (n_heads * head_dim)
    if not (q.is_contiguous() and q.numel() == rows * n_heads * head_dim):
        raise KernelError("attn_rows: q must be [rows, heads, head_dim]")
    _gpu(out, "out", q.dtype)
    if not (out.is_contiguous() and out.numel() == rows * n_heads * v_dim):
        raise KernelError("attn_rows: out must be [rows, heads, v_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, q.dtype, v_dim)
    if sink is not None:
        _gpu(sink, "sink", torch.float32)
        if not (sink.is_contiguous() and sink.numel() == n_heads):
            raise KernelError(f"sink: needs {n_heads} entries")
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows):
            raise KernelError(f"{name}: needs {rows} entries")
    if not (n_heads <= 65535):
        raise KernelError("attn_rows: too many heads")
    _check_rel(rel, n_heads)
    _check(_fn("attn_rows", "dryft_attn_rows")(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(row_slot), _ptr(row_pos),
        _ptr(out), rows, n_heads, n_kv, head_dim, v_dim, float(scale), int(window), float(softcap), _ptr(sink),
        int(bool(exact_p)), int(chunk), _ptr(rel), rel.shape[0] if rel is not None else 0, is_f32, _stream()),
        "attn_rows")


def _check_rel(rel, n_heads: int) -> None:
    if rel is not None:
        _gpu(rel, "rel", torch.float32)
        if not (rel.dim() == 2 and rel.shape[1] == n_heads and rel.shape[0] >= 1 and rel.is_contiguous()):
            raise KernelError(f"rel: needs contiguous float32 [distances, {n_heads}]")


def _check_sink(sink, n_heads: int) -> None:
    if sink is not None:
        _gpu(sink, "sink", torch.float32)
        if not (sink.is_contiguous() and sink.numel() == n_heads):
            raise KernelError(f"sink: needs {n_heads} contiguous float32 entries")


ATTN_ROW_TILE = 64      # rows of a sequence that one workgroup of the prompt-attention kernels takes (``tile_cu``)


def attn_causal_bf16(q, k_pages, v_pages, page_table, seq_slot, cu_rows, tile_cu, seq_start, n_seqs: int,
                     max_tiles: int, out, n_heads: int, n_kv: int, head_dim: int, scale: float, window: int,
                     mode: int = 0, softcap: float = 0.0, sink=None, chunk: int = 0, rel=None) -> None:
    """Causal attention of steps with many rows per sequence. ``mode``: 0 lets the library choose how much a wave
    takes; 1 = one head and 16 rows, 2 = two heads of a kv group, 3 = one head and 32 rows. At head size 128, 1 and
    3 bring the pages straight into LDS; 5 and 7 are 1 and 3 with the pages staged through registers, as at every
    other head size. ``softcap`` > 0 caps the scores, ``sink`` (float32 ``[heads]``) joins each head's denominator;
    ``chunk`` > 0: a row sees the earlier keys of its own run of so many positions (no window then); ``rel``: float32
    ``[distances, heads]``, a bias by distance added to the scaled score (the last row for every larger distance)."""
    _check_sink(sink, n_heads)
    _check_rel(rel, n_heads)
    _gpu(q, "q", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    if not (q.is_contiguous() and out.is_contiguous() and out.numel() == q.numel()):
        raise KernelError("attn_causal: q and out contiguous")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1),
                       ("tile_cu", tile_cu, n_seqs + 1), ("seq_start", seq_start, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    if not (n_heads <= 65535):
        raise KernelError("attn_causal: too many heads")
    _check(_fn("attn_mfma", "dryft_attn_causal_bf16")(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot), _ptr(cu_rows),
        _ptr(tile_cu), _ptr(seq_start), n_seqs, max_tiles, _ptr(out), n_heads, n_kv, head_dim, float(scale),
        int(window), int(mode), float(softcap), _ptr(sink), int(chunk), _ptr(rel),
        rel.shape[0] if rel is not None else 0, _stream()), "attn_causal_bf16")


def attn_causal_takes_projection(head_dim: int, rot: int) -> bool:
    """Can ``attn_causal_projected_bf16`` run heads of this size, rotated over ``rot`` features?"""
    return bool(_fn("attn_mfma", "dryft_attn_causal_takes_projection")(int(head_dim), int(rot)))


def attn_causal_projected_bf16(qkv, q_weight, eps: float, cos, sin, k_pages, v_pages, page_table, seq_slot, cu_rows,
                               tile_cu, seq_start, n_seqs: int, max_tiles: int, out, n_heads: int, n_kv: int,
                               head_dim: int, scale: float, window: int, mode: int = 0) -> None:
    """``attn_causal_bf16`` with the queries taken from the fused projection ``qkv`` [rows, >= n_heads * head_dim]
    (query heads first): their per-head norm (``q_weight`` or None) and rotation happen inside the kernel, so they
    are neither written out nor read back. Keys and values must be in the cache already."""
    _gpu(qkv, "qkv", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    rows = qkv.shape[0]
    if not (qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= n_heads * head_dim and qkv.stride(0) % 8 == 0):
        raise KernelError(
            "attn_causal_projected: qkv must be [rows, >= heads * head_dim] with rows 16 bytes apart or a multiple"
        )
    if not (out.is_contiguous() and out.numel() == rows * n_heads * head_dim):
        raise KernelError("attn_causal_projected: out [rows, heads, head_dim]")
    if not (attn_causal_takes_projection(head_dim, 2 * cos.shape[1] if cos is not None else 0)):
        raise KernelError("attn_causal_projected: the kernel refuses these sizes")
    w_f32 = 0
    if q_weight is not None:
        _gpu(q_weight, "q_weight")
        if not (q_weight.shape == (head_dim,) and q_weight.is_contiguous()):
            raise KernelError(f"q_weight: must be [{head_dim}]")
        w_f32 = _float_flag(q_weight, "q_weight")
    for name, t in (("cos", cos), ("sin", sin)):
        _gpu(t, name, torch.bfloat16)
        if not (t.dim() == 2 and t.shape[1] == head_dim // 2 and t.is_contiguous()):
            raise KernelError(f"{name}: must be [positions, {head_dim // 2}]")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1),
                       ("tile_cu", tile_cu, n_seqs + 1), ("seq_start", seq_start, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    if not (n_heads <= 65535):
        raise KernelError("attn_causal: too many heads")
    _check(_fn("attn_mfma", "dryft_attn_causal_projected_bf16")(
        _ptr(qkv), qkv.stride(0), _ptr(q_weight), w_f32, int(q_weight is not None), float(eps), _ptr(cos), _ptr(sin),
        _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot), _ptr(cu_rows), _ptr(tile_cu),
        _ptr(seq_start), n_seqs, max_tiles, _ptr(out), n_heads, n_kv, head_dim, float(scale), int(window), int(mode),
        _stream()), "attn_causal_projected_bf16")


def attn_split_bf16(q, k_pages, v_pages, page_table, seq_slot, cu_rows, kv_len, n_seqs: int, part_o, part_ml,
                    n_splits: int, out, n_heads: int, n_kv: int, head_dim: int, scale: float, window: int,
                    softcap: float = 0.0, sink=None, chunk: int = 0, rel=None) -> None:
    _check_sink(sink, n_heads)
    _check_rel(rel, n_heads)
    _gpu(q, "q", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    if not (q.is_contiguous() and out.is_contiguous() and out.numel() == q.numel()):
        raise KernelError("attn_split: q and out contiguous")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1), ("kv_len", kv_len, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    _gpu(part_o, "part_o", torch.float32)
    _gpu(part_ml, "part_ml", torch.float32)
    entries = n_seqs * n_heads * n_splits
    if part_o.numel() < entries * head_dim or part_ml.numel() < entries * 2:
        raise KernelError("attn_split: partial buffers too small")
    if not (n_splits <= 65535 and n_kv * ((n_heads // n_kv + 15) // 16) <= 65535):
        raise KernelError("attn_split: grid too large")
    _check(_fn("attn_mfma", "dryft_attn_split_bf16")(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot), _ptr(cu_rows),
        _ptr(kv_len), n_seqs, _ptr(part_o), _ptr(part_ml), n_splits, _ptr(out), n_heads, n_kv, head_dim, float(scale),
        int(window), float(softcap), _ptr(sink), int(chunk), _ptr(rel), rel.shape[0] if rel is not None else 0,
        _stream()), "attn_split_bf16")


def attn_decode_fused_bf16(qkv, q_weight, k_weight, eps: float, cos, sin, rot: int, write_kv: bool, k_pages, v_pages,
                           page_table, seq_slot, cu_rows, kv_len, n_seqs: int, part_o, part_ml, n_splits: int, out,
                           n_heads: int, n_kv: int, head_dim: int, scale: float, window: int, qkv_parts: int = 0) -> None:
    """One row per sequence: q/k norm, rotation, append to the cache and attention in one kernel (plus the combine).

    ``qkv`` is the fused projection's output ``[n_seqs rows, (heads + 2 kv heads) * head_dim]``; row ``i`` belongs to
    sequence ``i`` (``cu_rows[i] == i``). It may also be that product left as float32 partial sums over K,
    ``[parts, rows, width]`` (``qkv_parts`` of them): the kernel adds them up in order and rounds the sum to bfloat16
    as the product would have.
    """
    _gpu(out, "out", torch.bfloat16)
    need_cols = (n_heads + 2 * n_kv) * head_dim
    if qkv_parts:
        _gpu(qkv, "qkv", torch.float32)
        if not (qkv.dim() == 3 and qkv.is_contiguous() and qkv.shape[0] >= qkv_parts and qkv.shape[1] >= n_seqs
                and qkv.shape[2] >= need_cols):
            raise KernelError(f"attn_decode_fused: partial sums must be [>= {qkv_parts}, rows >= {n_seqs}, >= {need_cols}]")
        row_stride, part_stride = qkv.stride(1), qkv.stride(0)
    else:
        _gpu(qkv, "qkv", torch.bfloat16)
        if not (qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= need_cols and qkv.shape[0] >= n_seqs):
            raise KernelError(f"attn_decode_fused: qkv must be [rows >= {n_seqs}, >= {need_cols}]")
        row_stride, part_stride = qkv.stride(0), 0
    if not (out.is_contiguous() and out.numel() >= n_seqs * n_heads * head_dim):
        raise KernelError("attn_decode_fused: out too small")
    if not (n_heads // n_kv <= 16):
        raise KernelError("attn_decode_fused: at most 16 query heads per kv head")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    has_norm = q_weight is not None
    w_f32 = 0
    if has_norm:
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            _gpu(w, name)
            if not (w.shape == (head_dim,) and w.is_contiguous()):
                raise KernelError(f"{name}: must be [{head_dim}]")
        if not (q_weight.dtype == k_weight.dtype):
            raise KernelError("q_weight and k_weight must share a dtype")
        w_f32 = _float_flag(q_weight, "q_weight")
    if rot:
        if not (rot % 2 == 0 and rot <= head_dim):
            raise KernelError(f"rotary width {rot} must be even and at most {head_dim}")
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, torch.bfloat16)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be [positions, {rot // 2}]")
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1), ("kv_len", kv_len, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    _gpu(part_o, "part_o", torch.float32)
    _gpu(part_ml, "part_ml", torch.float32)
    entries = n_seqs * n_heads * n_splits
    if part_o.numel() < entries * head_dim or part_ml.numel() < entries * 2:
        raise KernelError("attn_decode_fused: partial buffers too small")
    _check(_fn("attn_mfma", "dryft_attn_decode_fused_bf16")(
        _ptr(qkv), row_stride, int(qkv_parts), part_stride, _ptr(q_weight), _ptr(k_weight), w_f32, int(has_norm),
        float(eps), _ptr(cos), _ptr(sin),
        int(rot), int(write_kv), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot),
        _ptr(cu_rows), _ptr(kv_len), n_seqs, _ptr(part_o), _ptr(part_ml), n_splits, _ptr(out), n_heads, n_kv, head_dim,
        float(scale), int(window), _stream()), "attn_decode_fused_bf16")


# -------------------------------------------------------------------------------------------- gemm
def gemm_tiled(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out = x @ w.T`` with float accumulation by plain multiply-adds (any sizes)."""
    _gpu(x, "x")
    _gpu(w, "w", x.dtype)
    is_f32 = _float_flag(x, "x")
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_tiled: x [M,K] row-major, w [N,K] contiguous")
    _gpu(out, "out")
    out_f32 = 1 if out.dtype == torch.float32 else 0
    if not (out.shape == (m, n) and out.is_contiguous() and (out.dtype == x.dtype or out_f32)):
        raise KernelError(f"gemm_tiled: out must be [{m},{n}] in the input dtype or float32")
    for m0 in range(0, m, 65535 * 64):                      # the row tiles ride on grid.y
        m1 = min(m, m0 + 65535 * 64)
        _check(_fn("gemm", "dryft_gemm_tiled")(_ptr(x[m0:m1]), x.stride(0), _ptr(w), _ptr(out[m0:m1]), m1 - m0, n, k,
                                               is_f32, out_f32, _stream()), "gemm_tiled")
    return out


def gemm_stream_bf16(x, w, out, partials=None, group_blocks: int = 2, splits: int = 1, depth: int = 2) -> None:
    """``x [M<=16, K] @ w[N, K].T`` by the kernel that reads whole cache lines and stages operands in LDS.

    ``group_blocks`` (1 or 2) is how many 64-value blocks of K a wave loads at a time and ``depth``
    (1 or 2) how many such groups it keeps in flight; with ``splits > 1`` the result is left as
    ``partials[splits, M, N]``.
    """
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_stream: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= 16 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_stream: needs M <= 16 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_stream: operands must be 16-byte aligned")
    if not (group_blocks in (1, 2) and depth in (1, 2) and 1 <= splits <= 64):
        raise KernelError("gemm_stream: group_blocks and depth in 1, 2 and splits in 1..64")
    out_f32 = 0
    if splits > 1:
        _gpu(partials, "partials", torch.float32)
        if not (partials.numel() >= splits * m * n and partials.is_contiguous()):
            raise KernelError("gemm_stream: partials too small")
    else:
        _gpu(out, "out")
        out_f32 = 1 if out.dtype == torch.float32 else 0
        if not (out.shape == (m, n) and out.is_contiguous() and out.dtype in (torch.float32, torch.bfloat16)):
            raise KernelError(f"gemm_stream: out must be contiguous [{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_stream_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), _ptr(partials), m, n, k,
                                                 int(group_blocks), int(depth), int(splits), out_f32, _stream()), "gemm_stream_bf16")


def gemm_stream_swiglu_bf16(x, w_gate_up, out, group_blocks: int = 2, depth: int = 1) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 16 rows, in one kernel."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_stream_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= 16 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_stream_swiglu: needs M <= 16 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_stream_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_stream_swiglu: out must be [{m},{two_n // 2}]")
    if not (group_blocks in (1, 2) and depth in (1, 2)):
        raise KernelError("gemm_stream_swiglu: group_blocks and depth in 1, 2")
    _check(_fn("gemm", "dryft_gemm_stream_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                        int(group_blocks), int(depth), _stream()), "gemm_stream_swiglu_bf16")
    return out


def gemm_wide_bf16(x, w, out, partials=None, group_blocks: int = 2, splits: int = 1, depth: int = 2) -> None:
    """``x [M<=64, K] @ w[N, K].T`` by the kernel whose workgroups share the rows of ``x`` in LDS.

    ``group_blocks`` (1 or 2) is how many 64-value blocks of K are staged at a time and ``depth`` (1 to 3)
    how many such groups a wave has in flight; with ``splits > 1`` the result is left as
    ``partials[splits, M, N]``.
    """
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_wide: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= 64 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_wide: needs M <= 64 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_wide: operands must be 16-byte aligned")
    if not (group_blocks in (1, 2) and depth in (1, 2, 3) and 1 <= splits <= 64):
        raise KernelError("gemm_wide: group_blocks in 1, 2, depth in 1..3 and splits in 1..64")
    out_f32 = 0
    if splits > 1:
        _gpu(partials, "partials", torch.float32)
        if not (partials.numel() >= splits * m * n and partials.is_contiguous()):
            raise KernelError("gemm_wide: partials too small")
    else:
        _gpu(out, "out")
        out_f32 = 1 if out.dtype == torch.float32 else 0
        if not (out.shape == (m, n) and out.is_contiguous() and out.dtype in (torch.float32, torch.bfloat16)):
            raise KernelError(f"gemm_wide: out must be contiguous [{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_wide_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), _ptr(partials), m, n, k,
                                               int(group_blocks), int(depth), int(splits), out_f32, _stream()), "gemm_wide_bf16")


PANEL_GROUP = 128     # values of K the panel kernel moves at a time; K must be a multiple of it
DIRECT_REACH = 1 << 32    # bytes: the kernels that bring operands straight into LDS address them by 32-bit offsets


def gemm_panel_waves(n_outputs: int) -> int:
    """Waves per workgroup (8 outputs each) that the panel kernel chooses for this many outputs."""
    return int(_fn("gemm", "dryft_gemm_panel_waves")(int(n_outputs)))


def gemm_panel_swiglu_bf16(x, w_gate_up, out, waves: int = 0, clamped: tuple[float, float] | None = None) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 64 rows, by the kernel whose operands go
    from memory straight into LDS. K must be a multiple of 128. ``waves`` (4 to 8, 8 outputs each) per workgroup;
    0 lets the library choose. ``clamped = (limit, alpha)``: the clamped gated unit in the epilogue instead,
    ``g * sigmoid(alpha * g) * (u + 1)`` with ``g = min(x @ Wg.T, limit)`` and ``u = clamp(x @ Wu.T, -limit, limit)``."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_panel_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= 64 and k % PANEL_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_panel_swiglu: needs M <= 64 and K % {PANEL_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_panel_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_panel_swiglu: out must be [{m},{two_n // 2}]")
    if not (waves == 0 or 4 <= waves <= 8):
        raise KernelError("gemm_panel_swiglu: waves 4 to 8, or 0")
    if clamped is not None:
        limit, alpha = clamped
        if not limit > 0:
            raise KernelError(f"gemm_panel_swiglu: the clamp's limit must be positive, got {limit}")
        _check(_fn("gemm", "dryft_gemm_panel_glu_clamped_bf16")(
            _ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k, int(waves), float(limit), float(alpha),
            _stream()), "gemm_panel_glu_clamped_bf16")
        return out
    _check(_fn("gemm", "dryft_gemm_panel_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                       int(waves), _stream()), "gemm_panel_swiglu_bf16")
    return out


TALL_ROWS = 256     # the most rows gemm_tall_swiglu takes
TALL_GROUP = 64     # values of K it moves at a time; K must be a multiple of it


def gemm_tall_swiglu_bf16(x, w_gate_up, out, tiles: int = 0) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 256 rows, by the kernel whose waves each own
    rows of x and multiply them with all of the workgroup's rows of W (operands straight into LDS). K must be a multiple
    of 64. ``tiles`` (4 to 8, 8 outputs each) per workgroup; 0 lets the library choose."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_tall_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= TALL_ROWS and k % TALL_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_tall_swiglu: needs M <= {TALL_ROWS} and K % {TALL_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_tall_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_tall_swiglu: out must be [{m},{two_n // 2}]")
    if not (tiles == 0 or 4 <= tiles <= 8):
        raise KernelError("gemm_tall_swiglu: tiles 4 to 8, or 0")
    _check(_fn("gemm", "dryft_gemm_tall_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                      int(tiles), _stream()), "gemm_tall_swiglu_bf16")
    return out


def gemm_tall_bf16(x, w, partials, splits: int, tiles: int) -> torch.Tensor:
    """Float partial sums ``partials[s] = x @ w.T`` over the s-th run of K, at most 256 rows, by the kernel whose waves
    each own rows of x (see ``gemm_tall_swiglu_bf16``); a workgroup owns ``16 * tiles`` outputs (tiles 4 to 8). K must
    be a multiple of 64 and ``splits`` a count ``gemm_mid_splits`` gives."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    _gpu(partials, "partials", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_tall: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= TALL_ROWS and k % TALL_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_tall: needs M <= {TALL_ROWS} and K % {TALL_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and partials.data_ptr() % 16 == 0):
        raise KernelError("gemm_tall: operands must be 16-byte aligned")
    if not (partials.shape == (splits, m, n) and partials.is_contiguous()):
        raise KernelError(f"gemm_tall: partials must be [{splits},{m},{n}]")
    if not 4 <= tiles <= 8:
        raise KernelError("gemm_tall: tiles 4 to 8")
    if gemm_mid_splits(k, splits) != splits:
        raise KernelError(f"gemm_tall: {splits} runs of K={k} would leave one empty")
    _check(_fn("gemm", "dryft_gemm_tall_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(partials), m, n, k, int(splits),
                                               int(tiles), _stream()), "gemm_tall_bf16")
    return partials


MID_ROWS = 256      # the most rows gemm_mid takes
MID_GROUP = 64      # values of K it walks at a time; K must be a multiple, and the splits are runs of such groups


def gemm_mid_splits(k: int, splits: int) -> int:
    """The number of splits closest below ``splits`` that cuts ``k`` into runs of groups none of which is empty."""
    groups = k // MID_GROUP
    splits = max(1, min(splits, groups))
    while splits > 1 and -(-groups // -(-groups // splits)) != splits:
        splits -= 1
    return splits


def gemm_mid_bf16(x, w, partials, splits: int) -> torch.Tensor:
    """Float partial sums ``partials[splits, M, N]`` of ``x @ w.T`` over ``splits`` runs of K, for 1 to 256 rows, by the
    kernel whose operands go from memory straight into LDS. K must be a multiple of 64 and ``splits`` one that
    ``gemm_mid_splits`` returns."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    _gpu(partials, "partials", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_mid: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= MID_ROWS and k % MID_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_mid: needs M <= {MID_ROWS} and K % {MID_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and partials.data_ptr() % 16 == 0):
        raise KernelError("gemm_mid: operands must be 16-byte aligned")
    if not (splits >= 1 and gemm_mid_splits(k, splits) == splits):
        raise KernelError(f"gemm_mid: {splits} splits would leave a run of K = {k} empty")
    if not (partials.shape == (splits, m, n) and partials.is_contiguous()):
        raise KernelError(f"gemm_mid: partials must be [{splits},{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_mid_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(partials), m, n, k, int(splits),
                                              _stream()), "gemm_mid_bf16")
    return partials


def gemm_wide_swiglu_bf16(x, w_gate_up, out, group_blocks: int = 2, depth: int = 1) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 64 rows, in one kernel."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_wide_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= 64 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_wide_swiglu: needs M <= 64 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_wide_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_wide_swiglu: out must be [{m},{two_n // 2}]")
    if not (group_blocks in (1, 2) and depth in (1, 2, 3)):
        raise KernelError("gemm_wide_swiglu: group_blocks in 1, 2 and depth in 1..3")
    _check(_fn("gemm", "dryft_gemm_wide_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                      int(group_blocks), int(depth), _stream()), "gemm_wide_swiglu_bf16")
    return out


def gemm_block_bf16(x, w, out, swiglu: bool = False, shape: int | None = None) -> torch.Tensor:
    """``x [M, K] @ w[N, K].T`` for any number of rows, by the kernel that owns blocks of 128 rows by 128 outputs;
    ``out`` bfloat16 or float32. With ``swiglu``, ``w = [Wg; Wu]`` of ``2N`` rows and
    ``out = silu(x @ Wg.T) * (x @ Wu.T)`` in bfloat16. ``shape``: 0 = blocks of 128 x 128, 1 = 256 x 256; by default
    the large blocks where there are enough of them to give every compute unit one."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    _gpu(out, "out")
    m, k = x.shape
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    if not (w.dim() == 2 and w.shape[1] == k and w.is_contiguous() and x.stride(1) == 1) or (swiglu and w.shape[0] % 2):
        raise KernelError("gemm_block: x [M,K] row-major, w [N,K] (or [2N,K]) contiguous")
    if not (k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_block: needs K % 8 == 0, got K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_block: operands must be 16-byte aligned")
    out_dtypes = (torch.bfloat16,) if swiglu else (torch.float32, torch.bfloat16)
    if not (out.shape == (m, n) and out.is_contiguous() and out.dtype in out_dtypes):
        raise KernelError(f"gemm_block: out must be contiguous [{m},{n}]")
    if shape is None:
        shape = 1 if -(-m // 256) * -(-(2 * n if swiglu else n) // 256) >= 256 else 0
    if not (shape in (0, 1)):
        raise KernelError("gemm_block: shape 0 or 1")
    _check(_fn("gemm", "dryft_gemm_block_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, 1 if swiglu else 0,
                                                1 if out.dtype == torch.float32 else 0, int(shape), _stream()), "gemm_block_bf16")
    return out


def gemm_block_f32(x, w, out, shape: int | None = None) -> torch.Tensor:
    """``x [M, K] @ w[N, K].T`` on float32 values with the matrix cores' full-precision instruction
    (``v_mfma_f32_16x16x4_f32``); ``K`` a multiple of 4, operands 16-byte aligned."""
    _gpu(x, "x", torch.float32)
    _gpu(w, "w", torch.float32)
    _gpu(out, "out", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_block_f32: x [M,K] row-major, w [N,K] contiguous")
    if not (k % 4 == 0 and x.stride(0) % 4 == 0):
        raise KernelError(f"gemm_block_f32: needs K % 4 == 0, got K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_block_f32: operands must be 16-byte aligned")
    if not (out.shape == (m, n) and out.is_contiguous()):
        raise KernelError(f"gemm_block_f32: out must be contiguous [{m},{n}]")
    if shape is None:
        shape = 1 if -(-m // 256) * -(-n // 256) >= 256 else 0
    if not (shape in (0, 1)):
        raise KernelError("gemm_block_f32: shape 0 or 1")
    _check(_fn("gemm", "dryft_gemm_block_f32")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, int(shape), _stream()),
           "gemm_block_f32")
    return out


def gemm_rows_f32(x, w, out) -> torch.Tensor:
    """``x [M<=16, K] @ w[N, K].T`` on float32 values by plain multiply-adds, every weight read once; ``K`` a
    multiple of 4 and ``w`` 16-byte aligned."""
    _gpu(x, "x", torch.float32)
    _gpu(w, "w", torch.float32)
    _gpu(out, "out", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_rows_f32: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= 16 and k % 4 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError(f"gemm_rows_f32: needs M <= 16, K % 4 == 0, aligned w; got M={m} K={k}")
    if not (out.shape == (m, n) and out.is_contiguous()):
        raise KernelError(f"gemm_rows_f32: out must be contiguous [{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_rows_f32")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, _stream()), "gemm_rows_f32")
    return out


def sum_partials(partials: torch.Tensor, out: torch.Tensor, splits: int) -> torch.Tensor:
    _gpu(partials, "partials", torch.float32)
    _gpu(out, "out")
    if not (out.is_contiguous() and partials.is_contiguous() and partials.numel() >= splits * out.numel()):
        raise KernelError("sum_partials: partials must hold splits * out.numel() values")
    if not (out.dtype in (torch.float32, torch.bfloat16)):
        raise KernelError("sum_partials: out must be float32 or bfloat16")
    _check(_fn("gemm", "dryft_sum_partials")(_ptr(partials), _ptr(out), out.numel(), splits,
                                             1 if out.dtype == torch.float32 else 0, _stream()), "sum_partials")
    return out


# ---------------------------------------------------------------------------------------- sampling
def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(logits, "logits", torch.float32)
    _gpu(out, "out", torch.int32)
    rows, vocab = logits.shape
    if not (logits.stride(1) == 1 and out.numel() >= rows and out.is_contiguous()):
        raise KernelError("argmax_rows: bad operands")
    chunks = 1 if vocab < 8192 else min(64, vocab // 2048)
    scratch_v = scratch_i = None
    if chunks > 1:
        scratch_v = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
        scratch_i = torch.empty(rows * chunks, dtype=torch.int32, device=logits.device)
    _check(_fn("sampling", "dryft_argmax_rows")(_ptr(logits), rows, vocab, logits.stride(0), _ptr(out), chunks,
                                                _ptr(scratch_v), _ptr(scratch_i), _stream()), "argmax_rows")
    return out


def sample_rows(logits: torch.Tensor, temperature: float, uniforms: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(logits, "logits", torch.float32)
    _gpu(uniforms, "uniforms", torch.float32)
    _gpu(out, "out", torch.int32)
    rows, vocab = logits.shape
    if not (temperature > 0):
        raise KernelError("sample_rows: temperature must be positive (use argmax_rows for greedy)")
    if not (logits.stride(1) == 1 and out.numel() >= rows and uniforms.numel() >= rows):
        raise KernelError("sample_rows: bad operands")
    chunks = 1 if vocab < 8192 else min(64, vocab // 2048)
    chunk_max = chunk_sum = None
    if chunks > 1:
        chunk_max = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
        chunk_sum = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
    _check(_fn("sampling", "dryft_sample_rows")(_ptr(logits), rows, vocab, logits.stride(0), float(temperature),
                                                _ptr(uniforms), _ptr(out), chunks, _ptr(chunk_max), _ptr(chunk_sum),
                                                _stream()), "sample_rows")
    return out


# --------------------------------------------------------------------------------- rotary over neighbouring pairs
def rope_pairs_kv(proj, q_col: int, k_col: int, v_col: int, cos, sin, rot: int, row_slot, row_pos, q_out, k_pages,
                  v_pages, page_table, write_kv: bool, n_heads: int, n_kv: int, head_dim: int, v_dim: int) -> None:
    """Rotates the q and k heads of a fused projection pair by pair ``(2i, 2i + 1)`` over their first ``rot`` features
    with float32 tables ``[positions, rot / 2]``, writes the queries to ``q_out [rows, heads, head_dim]`` and, when
    ``write_kv``, the keys and the (unrotated) values of width ``v_dim`` to their pages."""
    _gpu(proj, "proj")
    is_f32 = _float_flag(proj, "proj")
    rows = proj.shape[0]
    if not (proj.dim() == 2 and proj.stride(1) == 1):
        raise KernelError("rope_pairs_kv: proj must be [rows, columns] with unit column stride")
    ends = (q_col + n_heads * head_dim, k_col + n_kv * head_dim, v_col + n_kv * v_dim)
    if min(q_col, k_col, v_col) < 0 or max(ends) > proj.shape[1]:
        raise KernelError("rope_pairs_kv: q, k or v lie outside the projection's columns")
    if rot % 2 or not 0 <= rot <= head_dim:
        raise KernelError(f"rope_pairs_kv: the rotated width must be even and at most {head_dim}, got {rot}")
    if rot:
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, torch.float32)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be contiguous float32 [positions, {rot // 2}]")
    _gpu(q_out, "q_out", proj.dtype)
    if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * head_dim):
        raise KernelError("rope_pairs_kv: q_out must be [rows, heads, head_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, proj.dtype, v_dim)
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows):
            raise KernelError(f"{name}: needs {rows} entries")
    _check(_fn("rope_kv", "dryft_rope_pairs_kv")(
        _ptr(proj), proj.stride(0), q_col, k_col, v_col, _ptr(cos), _ptr(sin), rot, _ptr(row_slot), _ptr(row_pos),
        _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], int(bool(write_kv)), rows,
        n_heads, n_kv, head_dim, v_dim, is_f32, _stream()), "rope_pairs_kv")


# ------------------------------------------------------------------------------------------ recurrent mixers
def _f32_vector(t, name: str, n: int) -> None:
    _gpu(t, name, torch.float32)
    if not (t.is_contiguous() and t.numel() == n):
        raise KernelError(f"{name}: needs {n} contiguous float32 entries, has {tuple(t.shape)}")


def _seq_facts(seq_slot, cu_rows, q_len, n_seqs: int) -> None:
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1), ("q_len", q_len, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"{name}: needs {n} contiguous entries")


MLSTM_MAX_DIM = 256
MLSTM_COLUMNS = 64       # value columns a workgroup of either kernel owns
MLSTM_CHUNK = 64         # tokens the chunked kernel takes at a time; segments are multiples of it


def mlstm_chunks_takes(proj, q_col: int, k_col: int, v_col: int, dim: int, v_dim: int) -> bool:
    """Does the chunked matrix-core form of ``mlstm_steps`` take this projection? (bfloat16, 16-byte pieces.)"""
    return proj.dtype == torch.bfloat16 and proj.data_ptr() % 16 == 0 and bool(
        _fn("mlstm", "dryft_mlstm_chunks_takes")(dim, v_dim, q_col, k_col, v_col, proj.stride(0)))


def mlstm_steps(proj, q_col: int, k_col: int, v_col: int, gates, bias_i, bias_f, cap: float, seq_slot, cu_rows, q_len,
                n_seqs: int, state_s, state_n, state_m, o_raw, n_heads: int, dim: int, v_dim: int, q_scale: float,
                write_state: bool, chunked: bool = False, segments: tuple | None = None) -> None:
    """The matrix-memory recurrence over each sequence's rows of the step, in order; ``o_raw`` (float32
    ``[rows, heads, v_dim]``) receives each token's read-out divided by its normaliser. ``gates`` are the float32
    projections ``[rows, 2 * heads]`` (input gates, then forget gates) before bias, cap and log-sigmoid. The states
    ``[slots, heads, dim, v_dim]``, ``[slots, heads, runs, dim]`` and ``[slots, heads, runs]`` are float32, the
    normaliser and the maximum once per run of ``MLSTM_COLUMNS`` value columns (each workgroup keeps its own)."""
    _gpu(proj, "proj")
    is_f32 = _float_flag(proj, "proj")
    rows = proj.shape[0]
    if not (proj.dim() == 2 and proj.stride(1) == 1):
        raise KernelError("mlstm_steps: proj must be [rows, columns] with unit column stride")
    if min(q_col, k_col, v_col) < 0 or max(q_col + n_heads * dim, k_col + n_heads * dim,
                                           v_col + n_heads * v_dim) > proj.shape[1]:
        raise KernelError("mlstm_steps: q, k or v lie outside the projection's columns")
    if not 0 < dim <= MLSTM_MAX_DIM:
        raise KernelError(f"mlstm_steps: key width must lie in 1..{MLSTM_MAX_DIM}, got {dim}")
    _gpu(gates, "gates", torch.float32)
    if not (gates.shape == (rows, 2 * n_heads) and gates.is_contiguous()):
        raise KernelError(f"mlstm_steps: gates must be contiguous float32 [{rows}, {2 * n_heads}]")
    _f32_vector(bias_i, "bias_i", n_heads)
    _f32_vector(bias_f, "bias_f", n_heads)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    slots = state_m.shape[0]
    runs = -(-v_dim // MLSTM_COLUMNS)
    for name, t, shape in (("state_s", state_s, (slots, n_heads, dim, v_dim)),
                           ("state_n", state_n, (slots, n_heads, runs, dim)), ("state_m", state_m, (slots, n_heads, runs))):
        _gpu(t, name, torch.float32)
        if not (tuple(t.shape) == shape and t.is_contiguous()):
            raise KernelError(f"{name}: must be contiguous float32 {shape}, got {tuple(t.shape)}")
    _gpu(o_raw, "o_raw", torch.float32)
    if not (o_raw.is_contiguous() and o_raw.numel() == rows * n_heads * v_dim):
        raise KernelError("mlstm_steps: o_raw must be float32 [rows, heads, v_dim]")
    if chunked:
        # the same recurrence a chunk of 64 tokens at a time on the matrix cores (steps of many rows, bfloat16)
        if not mlstm_chunks_takes(proj, q_col, k_col, v_col, dim, v_dim):
            raise KernelError("mlstm_steps: the chunked kernel does not take these sizes")
        # ``segments`` = (rows a segment, tile_cu, bound on the segments): long sequences cut into segments that run
        # side by side, in two launches with summaries of the segments in between
        seg_rows, tile_cu, max_tiles, scratch = 0, None, 0, None
        if segments is not None:
            seg_rows, tile_cu, max_tiles = segments
            if seg_rows <= 0 or seg_rows % MLSTM_CHUNK or max_tiles <= 0:
                raise KernelError(f"mlstm_steps: segments of {seg_rows} rows, at most {max_tiles} of them")
            _gpu(tile_cu, "tile_cu", torch.int32)
            if not (tile_cu.is_contiguous() and tile_cu.numel() >= n_seqs + 1):
                raise KernelError(f"tile_cu: needs {n_seqs + 1} contiguous entries")
            scratch = torch.empty(max_tiles * n_heads * (dim * v_dim + 2 * dim + 3), dtype=torch.float32,
                                  device=proj.device)
        _check(_fn("mlstm", "dryft_mlstm_chunks")(
            _ptr(proj), proj.stride(0), q_col, k_col, v_col, _ptr(gates), _ptr(bias_i), _ptr(bias_f), float(cap),
            _ptr(seq_slot), _ptr(cu_rows), _ptr(q_len), n_seqs, _ptr(state_s), _ptr(state_n), _ptr(state_m),
            _ptr(o_raw), n_heads, dim, v_dim, float(q_scale), int(bool(write_state)), seg_rows, _ptr(tile_cu),
            max_tiles, _ptr(scratch), _stream()), "mlstm_chunks")
        return
    _check(_fn("mlstm", "dryft_mlstm_steps")(
        _ptr(proj), proj.stride(0), q_col, k_col, v_col, _ptr(gates), _ptr(bias_i), _ptr(bias_f), float(cap),
        _ptr(seq_slot), _ptr(cu_rows), _ptr(q_len), n_seqs, _ptr(state_s), _ptr(state_n), _ptr(state_m), _ptr(o_raw),
        n_heads, dim, v_dim, float(q_scale), int(bool(write_state)), is_f32, _stream()), "mlstm_steps")


def mlstm_out(o_raw, proj, g_col: int, weight, row_slot, out, n_heads: int, v_dim: int, eps: float) -> None:
    """``out = o_raw / rms_per_head(o_raw) * weight * sigmoid(proj[:, g_col:...])`` in the activation dtype."""
    _gpu(proj, "proj")
    rows = proj.shape[0]
    _gpu(o_raw, "o_raw", torch.float32)
    _gpu(out, "out", proj.dtype)
    if not (o_raw.is_contiguous() and o_raw.numel() == rows * n_heads * v_dim and out.is_contiguous() and
            out.numel() == o_raw.numel()):
        raise KernelError("mlstm_out: o_raw and out must hold [rows, heads, v_dim]")
    if not (proj.stride(1) == 1 and 0 <= g_col and g_col + n_heads * v_dim <= proj.shape[1]):
        raise KernelError("mlstm_out: the gate lies outside the projection's columns")
    _f32_vector(weight, "weight", n_heads * v_dim)
    _gpu(row_slot, "row_slot", torch.int32)
    _check(_fn("mlstm", "dryft_mlstm_out")(_ptr(o_raw), _ptr(proj), proj.stride(0), g_col, _ptr(weight), _ptr(row_slot),
                                           _ptr(out), rows, n_heads, v_dim, float(eps),
                                           _float_flag(proj, "proj"), _stream()), "mlstm_out")


RGLRU_MAX_TAPS = 16


def rglru_gates(proj, x_col: int, x_bias, conv_w, conv_b, taps: int, gate_a, gate_a_bias, gate_i, gate_i_bias, lam,
                decay_scale: float, row_slot, row_seq, row_pos, seq_start, tail, coef, width: int, blocks: int) -> None:
    """Per row and channel the recurrence's two coefficients, ``coef[row, 0] = a`` and
    ``coef[row, 1] = sqrt(1 - a^2) * i * u``, from the convolution of the recurrent branch (columns ``x_col..`` of
    ``proj`` plus ``x_bias``; inputs before the step come from ``tail [slots, taps - 1, width]``) and the
    block-diagonal gates ``gate_a``, ``gate_i`` ``[blocks, width / blocks, width / blocks]``."""
    _gpu(proj, "proj")
    is_f32 = _float_flag(proj, "proj")
    rows = proj.shape[0]
    if not (proj.dim() == 2 and proj.stride(1) == 1 and 0 <= x_col and x_col + width <= proj.shape[1]):
        raise KernelError("rglru_gates: the branch lies outside the projection's columns")
    if blocks <= 0 or width % blocks or not 1 <= taps <= RGLRU_MAX_TAPS:
        raise KernelError(f"rglru_gates: {width} channels in {blocks} blocks, {taps} taps")
    bs = width // blocks
    for name, t in (("gate_a", gate_a), ("gate_i", gate_i)):
        _gpu(t, name, proj.dtype)
        if not (tuple(t.shape) == (blocks, bs, bs) and t.is_contiguous()):
            raise KernelError(f"{name}: must be contiguous [{blocks}, {bs}, {bs}]")
    for name, t in (("x_bias", x_bias), ("conv_b", conv_b), ("gate_a_bias", gate_a_bias), ("gate_i_bias", gate_i_bias),
                    ("lam", lam)):
        _f32_vector(t, name, width)
    _f32_vector(conv_w, "conv_w", width * taps)
    if taps > 1:
        _gpu(tail, "tail", torch.float32)
        if not (tail.dim() == 3 and tuple(tail.shape[1:]) == (taps - 1, width) and tail.is_contiguous()):
            raise KernelError(f"tail: must be contiguous float32 [slots, {taps - 1}, {width}]")
    for name, t in (("row_slot", row_slot), ("row_seq", row_seq), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows):
            raise KernelError(f"{name}: needs {rows} entries")
    _gpu(seq_start, "seq_start", torch.int32)
    _gpu(coef, "coef", torch.float32)
    if not (tuple(coef.shape) == (rows, 2, width) and coef.is_contiguous()):
        raise KernelError(f"coef: must be contiguous float32 [{rows}, 2, {width}]")
    _check(_fn("rglru", "dryft_rglru_gates")(
        _ptr(proj), proj.stride(0), x_col, _ptr(x_bias), _ptr(conv_w), _ptr(conv_b), taps, _ptr(gate_a),
        _ptr(gate_a_bias), _ptr(gate_i), _ptr(gate_i_bias), _ptr(lam), float(decay_scale), _ptr(row_slot), _ptr(row_seq),
        _ptr(row_pos), _ptr(seq_start), _ptr(tail) if taps > 1 else 0, _ptr(coef), rows, width, blocks, is_f32,
        _stream()), "rglru_gates")


def rglru_scan(coef, proj, x_col: int, y_col: int, x_bias, y_bias, taps: int, seq_slot, cu_rows, q_len, row_slot,
               n_seqs: int, state, tail, out, width: int, write_state: bool) -> None:
    """Walks each sequence's rows in order: ``S = a S + b``, ``out = S * gelu_tanh(y + y_bias)``; leaves ``S`` in
    ``state [slots, width]`` and the sequence's last ``taps - 1`` inputs in ``tail``."""
    _gpu(proj, "proj")
    rows = proj.shape[0]
    _gpu(coef, "coef", torch.float32)
    if not (tuple(coef.shape) == (rows, 2, width) and coef.is_contiguous()):
        raise KernelError(f"coef: must be contiguous float32 [{rows}, 2, {width}]")
    if not (proj.stride(1) == 1 and min(x_col, y_col) >= 0 and max(x_col, y_col) + width <= proj.shape[1]):
        raise KernelError("rglru_scan: a branch lies outside the projection's columns")
    _f32_vector(x_bias, "x_bias", width)
    _f32_vector(y_bias, "y_bias", width)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    _gpu(row_slot, "row_slot", torch.int32)
    _gpu(state, "state", torch.float32)
    if not (state.dim() == 2 and state.shape[1] == width and state.is_contiguous()):
        raise KernelError(f"state: must be contiguous float32 [slots, {width}]")
    if taps > 1:
        _gpu(tail, "tail", torch.float32)
        if not (tuple(tail.shape) == (state.shape[0], taps - 1, width) and tail.is_contiguous()):
            raise KernelError(f"tail: must be contiguous float32 [slots, {taps - 1}, {width}]")
    _gpu(out, "out", proj.dtype)
    if not (tuple(out.shape) == (rows, width) and out.is_contiguous()):
        raise KernelError(f"out: must be contiguous [{rows}, {width}]")
    _check(_fn("rglru", "dryft_rglru_scan")(
        _ptr(coef), _ptr(proj), proj.stride(0), x_col, y_col, _ptr(x_bias), _ptr(y_bias), taps, _ptr(seq_slot),
        _ptr(cu_rows), _ptr(q_len), _ptr(row_slot), n_seqs, _ptr(state), _ptr(tail) if taps > 1 else 0, _ptr(out), rows,
        width, int(bool(write_state)), _float_flag(proj, "proj"), _stream()), "rglru_scan")


RGLRU_TILE = 64         # tokens of a sequence that one workgroup of the tiled walk takes (``ctx.tiles``)


def rglru_scan_tiles(coef, proj, x_col: int, y_col: int, x_bias, y_bias, taps: int, seq_slot, cu_rows, q_len, tile_cu,
                     max_tiles: int, n_seqs: int, state, tail, out, width: int, write_state: bool) -> None:
    """``rglru_scan`` for steps of many rows per sequence: the walk cut into tiles of ``RGLRU_TILE`` tokens (their
    prefix sums per sequence in ``tile_cu``, at most ``max_tiles`` in all) that run side by side. ``out``'s rows of
    sequences that sit out are not written."""
    if _fn("rglru", "dryft_rglru_tile_rows")() != RGLRU_TILE:
        raise KernelError("rglru_scan_tiles: the library was built for another tile")
    _gpu(proj, "proj")
    rows = proj.shape[0]
    _gpu(coef, "coef", torch.float32)
    if not (tuple(coef.shape) == (rows, 2, width) and coef.is_contiguous()):
        raise KernelError(f"coef: must be contiguous float32 [{rows}, 2, {width}]")
    if not (proj.stride(1) == 1 and min(x_col, y_col) >= 0 and max(x_col, y_col) + width <= proj.shape[1]):
        raise KernelError("rglru_scan_tiles: a branch lies outside the projection's columns")
    _f32_vector(x_bias, "x_bias", width)
    _f32_vector(y_bias, "y_bias", width)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    _gpu(tile_cu, "tile_cu", torch.int32)
    if not (tile_cu.is_contiguous() and tile_cu.numel() >= n_seqs + 1):
        raise KernelError(f"tile_cu: needs {n_seqs + 1} contiguous entries")
    _gpu(state, "state", torch.float32)
    if not (state.dim() == 2 and state.shape[1] == width and state.is_contiguous()):
        raise KernelError(f"state: must be contiguous float32 [slots, {width}]")
    if taps > 1:
        _gpu(tail, "tail", torch.float32)
        if not (tuple(tail.shape) == (state.shape[0], taps - 1, width) and tail.is_contiguous()):
            raise KernelError(f"tail: must be contiguous float32 [slots, {taps - 1}, {width}]")
    _gpu(out, "out", proj.dtype)
    if not (tuple(out.shape) == (rows, width) and out.is_contiguous()):
        raise KernelError(f"out: must be contiguous [{rows}, {width}]")
    ends = torch.empty((max(1, max_tiles), 2, width), dtype=torch.float32, device=proj.device)
    _check(_fn("rglru", "dryft_rglru_scan_tiles")(
        _ptr(coef), _ptr(ends), _ptr(proj), proj.stride(0), x_col, y_col, _ptr(x_bias), _ptr(y_bias), taps,
        _ptr(seq_slot), _ptr(cu_rows), _ptr(q_len), _ptr(tile_cu), n_seqs, max_tiles, _ptr(state),
        _ptr(tail) if taps > 1 else 0, _ptr(out), width, int(bool(write_state)), _float_flag(proj, "proj"), _stream()),
        "rglru_scan_tiles")


# ------------------------------------------------------------------------------------------ several copies of a stream
HYPER_MAX_STREAMS = 8


def hyper_norm(x, n: int, delta, mix, write, read, weight, eps: float, x_out, y, *, normed: bool, act=None) -> None:
    """One launch for a residual stream of ``n`` copies: ``x'_t = sum_s mix[s, t] x_s + write[t] * delta`` (skipped
    without ``delta``), written to ``x_out [n, rows, width]`` (float32, may be ``x``; None: not kept);
    ``u = sum_t read[t] x'_t`` (``read`` None: the plain sum); ``y = rmsnorm(u) * weight`` in the activation dtype
    when ``normed``, else ``y = u`` in float32. ``x`` is the copies in float32 or one ``[rows, width]`` tensor in the
    activation dtype that every copy equals; ``delta`` a tensor in the activation dtype or ``(partials, count)``
    (partial sums are rounded to the activation dtype once added up, as the product itself would have stored them;
    ``act`` names that dtype where no operand shows it)."""
    _gpu(x, "x")
    rows, width = x.shape[-2:]
    copies = x.dim() == 3
    if copies:
        if not (x.dtype == torch.float32 and x.shape[0] == n and x.is_contiguous()):
            raise KernelError(f"hyper_norm: the copies must be contiguous float32 [{n}, rows, width]")
    elif not (x.dim() == 2 and x.is_contiguous()):
        raise KernelError("hyper_norm: a stream that starts must be contiguous [rows, width]")
    if not 1 <= n <= HYPER_MAX_STREAMS:
        raise KernelError(f"hyper_norm: 1..{HYPER_MAX_STREAMS} copies, got {n}")
    if act is None:
        act = y.dtype if (y is not None and normed) else (x.dtype if not copies else None)
    kind, n_partials, stride = 0, 0, 0
    if delta is not None:
        data, n_partials = delta if isinstance(delta, tuple) else (delta, 1)
        _gpu(data, "delta")
        if isinstance(delta, tuple):
            if not (data.dtype == torch.float32 and data.dim() == 3 and data.shape[1:] == (rows, width) and
                    data.is_contiguous() and data.shape[0] >= n_partials >= 1):
                raise KernelError("hyper_norm: partial sums must be contiguous float32 [n, rows, width]")
            kind, stride = 2, rows * width
        else:
            if not (data.shape == (rows, width) and data.is_contiguous()):
                raise KernelError("hyper_norm: delta must be contiguous [rows, width]")
            if act is None:
                act = data.dtype
            if data.dtype != act:
                raise KernelError("hyper_norm: delta must be in the activation dtype")
            kind = 1
        delta = data
        _f32_vector(mix, "mix", n * n)
        _f32_vector(write, "write", n)
    if act is None:
        act = torch.float32
    if not copies and x.dtype != act:
        raise KernelError("hyper_norm: a stream that starts must be in the activation dtype")
    if read is not None:
        _f32_vector(read, "read", n)
    if x_out is not None:
        _gpu(x_out, "x_out", torch.float32)
        if not (x_out.shape == (n, rows, width) and x_out.is_contiguous()):
            raise KernelError("hyper_norm: x_out must be contiguous float32 [n, rows, width]")
    if y is not None:
        _gpu(y, "y", act if normed else torch.float32)
        if not (y.shape == (rows, width) and y.is_contiguous()):
            raise KernelError("hyper_norm: y must be contiguous [rows, width]")
        if normed:
            _f32_vector(weight, "weight", width)
    _check(_fn("hyper", "dryft_hyper_norm")(
        _ptr(x), int(copies), n, _ptr(delta), kind, n_partials, stride, _ptr(mix), _ptr(write), _ptr(read), _ptr(weight),
        _ptr(x_out), _ptr(y), int(bool(normed)), rows, width, float(eps), 1 if act == torch.float32 else 0, _stream()),
        "hyper_norm")


# ------------------------------------------------------------------------------------------ wkv
WKV_MAX_DIM = 256


def wkv_blend(h, previous, mu, row_slot, row_seq, row_pos, seq_start, out) -> None:
    """``out[b] = h + (h' - h) * mu[b]`` for the five blends, ``h'`` the row before of the same sequence
    (``previous[slot]`` for a sequence's first row of the step)."""
    _gpu(h, "h")
    rows, width = h.shape
    _gpu(out, "out", h.dtype)
    _gpu(previous, "previous", torch.float32)
    if not (h.is_contiguous() and out.shape == (5, rows, width) and out.is_contiguous()):
        raise KernelError("wkv_blend: h contiguous [rows, width], out contiguous [5, rows, width]")
    if not (previous.dim() == 2 and previous.shape[1] == width and previous.is_contiguous()):
        raise KernelError("wkv_blend: previous must be contiguous float32 [slots, width]")
    _f32_vector(mu, "mu", 5 * width)
    for name, t in (("row_slot", row_slot), ("row_seq", row_seq), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if t.numel() < rows:
            raise KernelError(f"{name}: needs {rows} entries")
    _gpu(seq_start, "seq_start", torch.int32)
    _check(_fn("wkv", "dryft_wkv_blend")(_ptr(h), _ptr(previous), _ptr(mu), _ptr(row_slot), _ptr(row_seq), _ptr(row_pos),
                                         _ptr(seq_start), _ptr(out), rows, width, _float_flag(h, "h"), _stream()),
           "wkv_blend")


def wkv_decay(low, up, bias, decay) -> None:
    """``decay = exp(-exp(tanh(low) @ up.T + bias))``: ``low`` float32 ``[rows, rank]``, ``up`` ``[n, rank]``."""
    _gpu(low, "low", torch.float32)
    _gpu(up, "up")
    rows, rank = low.shape
    n = up.shape[0]
    if not (low.is_contiguous() and up.is_contiguous() and up.shape == (n, rank)):
        raise KernelError(f"wkv_decay: low contiguous [rows, {rank}], up contiguous [n, {rank}], got {tuple(up.shape)}")
    _f32_vector(bias, "bias", n)
    _gpu(decay, "decay", torch.float32)
    if not (decay.shape == (rows, n) and decay.is_contiguous()):
        raise KernelError("wkv_decay: decay must be contiguous float32 [rows, n]")
    _check(_fn("wkv", "dryft_wkv_decay")(_ptr(low), _ptr(up), _ptr(bias), _ptr(decay), rows, n, rank,
                                         _float_flag(up, "up"), _stream()), "wkv_decay")


WKV_GROUP = 16          # tokens the recurrence's kernel takes at a time; segments are multiples of it


def wkv_steps(r, k, v, decay, bonus, seq_slot, cu_rows, q_len, n_seqs: int, state, o_raw, h, previous, n_heads: int,
              dim: int, write_state: bool, segments=None) -> None:
    """The recurrence over every sequence's rows in order, from ``state[slot]`` (float32 ``[slots, heads, dim, dim]``)
    to the raw read-outs ``o_raw`` (float32 ``[rows, heads * dim]``); ``decay`` is float32, ``r``, ``k`` and ``v`` in the
    activation dtype. When ``write_state`` the state is written back and ``previous[slot]`` receives the sequence's
    last row of ``h``. ``segments = (rows per segment, prefix sums of segments over the sequences, their bound)``: long
    sequences run as segments side by side, in three launches (every segment's summary from a zero state, the state
    that enters each, every segment's outputs); the rows of sequences that sit out are then not written."""
    _gpu(v, "v")
    rows = v.shape[0]
    inner = n_heads * dim
    for name, t in (("r", r), ("k", k), ("v", v)):
        _gpu(t, name, v.dtype)
        if not (t.shape == (rows, inner) and t.is_contiguous()):
            raise KernelError(f"wkv_steps: {name} must be contiguous [rows, {inner}]")
    for name, t in (("decay", decay), ("o_raw", o_raw)):
        _gpu(t, name, torch.float32)
        if not (t.shape == (rows, inner) and t.is_contiguous()):
            raise KernelError(f"wkv_steps: {name} must be contiguous float32 [rows, {inner}]")
    _f32_vector(bonus, "bonus", inner)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    _gpu(state, "state", torch.float32)
    if not (state.dim() == 4 and state.shape[1:] == (n_heads, dim, dim) and state.is_contiguous()):
        raise KernelError(f"wkv_steps: state must be contiguous float32 [slots, {n_heads}, {dim}, {dim}]")
    _gpu(h, "h", v.dtype)
    _gpu(previous, "previous", torch.float32)
    if not (h.dim() == 2 and h.shape[0] == rows and h.is_contiguous() and previous.dim() == 2 and
            previous.shape == (state.shape[0], h.shape[1]) and previous.is_contiguous()):
        raise KernelError("wkv_steps: h contiguous [rows, width], previous contiguous float32 [slots, width]")
    if not 0 < dim <= WKV_MAX_DIM:
        raise KernelError(f"wkv_steps: dim must lie in 1..{WKV_MAX_DIM}")
    seg_cu = seg_state = seg_decay = None
    seg_rows = max_segs = 0
    if segments is not None:
        seg_rows, seg_cu, max_segs = segments
        _gpu(seg_cu, "segment prefix sums", torch.int32)
        if not (seg_cu.numel() >= n_seqs + 1 and seg_rows > 0 and seg_rows % WKV_GROUP == 0 and write_state):
            raise KernelError(f"wkv_steps: segments of a multiple of {WKV_GROUP} rows, prefix sums for every sequence, "
                              "and a state that is written back")
        if max_segs <= 0:
            return
        seg_state = torch.empty((max_segs, n_heads, dim, dim), dtype=torch.float32, device=v.device)
        seg_decay = torch.empty((max_segs, n_heads, dim), dtype=torch.float32, device=v.device)
    _check(_fn("wkv", "dryft_wkv_steps")(
        _ptr(r), _ptr(k), _ptr(v), _ptr(decay), _ptr(bonus), _ptr(seq_slot), _ptr(cu_rows), _ptr(q_len), n_seqs,
        _ptr(state), _ptr(o_raw), _ptr(h), _ptr(previous), h.shape[1], n_heads, dim, int(bool(write_state)),
        _ptr(seg_cu), max_segs, seg_rows, _ptr(seg_state), _ptr(seg_decay), _float_flag(v, "v"), _stream()), "wkv_steps")


def wkv_out(o_raw, gate, weight, out, n_heads: int, dim: int, eps: float) -> None:
    """``out = o_raw / rms_per_head(o_raw) * weight * silu(gate)`` in the activation dtype; ``gate`` may be a run of
    columns of a wider tensor."""
    _gpu(gate, "gate")
    rows = gate.shape[0]
    inner = n_heads * dim
    _gpu(o_raw, "o_raw", torch.float32)
    _gpu(out, "out", gate.dtype)
    for name, t in (("o_raw", o_raw), ("out", out)):
        if not (t.shape == (rows, inner) and t.is_contiguous()):
            raise KernelError(f"wkv_out: {name} must be contiguous [rows, {inner}]")
    if not (gate.shape == (rows, inner) and gate.stride(1) == 1):
        raise KernelError(f"wkv_out: gate must be [rows, {inner}] with unit column stride")
    _f32_vector(weight, "weight", inner)
    _check(_fn("wkv", "dryft_wkv_out")(_ptr(o_raw), _ptr(gate), _ptr(weight), _ptr(out), rows, n_heads, dim, float(eps),
                                       gate.stride(0), _float_flag(gate, "gate"), _stream()), "wkv_out")


# ------------------------------------------------------------------------------------------ latent attention
def rms_segments(src, col: int, w_a, out_a, n_a: int, w_b, out_b, eps: float) -> None:
    """``out_a = rmsnorm(src[:, col : col + n_a]) * w_a`` and, when ``out_b`` is given, the same for the columns
    after them with ``w_b``; float statistics, plain float32 weights."""
    _gpu(src, "src")
    rows = src.shape[0]
    n_b = out_b.shape[1] if out_b is not None else 0
    if not (src.dim() == 2 and src.stride(1) == 1 and 0 <= col and col + n_a + n_b <= src.shape[1]):
        raise KernelError("rms_segments: the runs of columns lie outside src")
    for name, t, n, w in (("out_a", out_a, n_a, w_a), ("out_b", out_b, n_b, w_b)):
        if t is None:
            continue
        _gpu(t, name, src.dtype)
        if not (t.shape == (rows, n) and t.is_contiguous()):
            raise KernelError(f"rms_segments: {name} must be contiguous [rows, {n}]")
        _f32_vector(w, name + "'s weight", n)
    _check(_fn("latent", "dryft_rms_segments")(_ptr(src), src.stride(0), col, _ptr(w_a), _ptr(out_a), n_a, _ptr(w_b),
                                               _ptr(out_b), n_b, float(eps), rows, _float_flag(src, "src"), _stream()),
           "rms_segments")


def latent_rope_kv(q_raw, kv, down, krot_col: int, cos, sin, rot: int, row_slot, row_pos, q_out, k_pages, v_pages,
                   page_table, write_kv: bool, n_heads: int, plain: int, rot_dim: int, v_dim: int, page_dv: int,
                   pairs: bool = False) -> None:
    """Queries ``[plain | rotated]`` per head from ``q_raw``; keys ``[that head's plain part of kv | the one rotated
    part at column krot_col of down]``; values from ``kv`` after the keys. The rotated parts' first ``rot`` features
    turn, feature ``i`` with ``i + rot/2`` (with ``pairs``: feature ``2i`` with ``2i + 1``), with float32 tables; keys
    and values go to their pages (values ``page_dv`` wide, of which ``v_dim`` are written)."""
    _gpu(q_raw, "q_raw")
    is_f32 = _float_flag(q_raw, "q_raw")
    rows, key_dim = q_raw.shape[0], plain + rot_dim
    if not (q_raw.shape == (rows, n_heads * key_dim) and q_raw.is_contiguous()):
        raise KernelError(f"latent_rope_kv: q_raw must be contiguous [rows, {n_heads * key_dim}]")
    _gpu(kv, "kv", q_raw.dtype)
    if not (kv.shape == (rows, n_heads * (plain + v_dim)) and kv.is_contiguous()):
        raise KernelError(f"latent_rope_kv: kv must be contiguous [rows, {n_heads * (plain + v_dim)}]")
    _gpu(down, "down", q_raw.dtype)
    if not (down.dim() == 2 and down.shape[0] == rows and down.stride(1) == 1 and 0 <= krot_col and
            krot_col + rot_dim <= down.shape[1]):
        raise KernelError("latent_rope_kv: the rotated key part lies outside down's columns")
    if rot % 2 or not 0 <= rot <= rot_dim:
        raise KernelError(f"latent_rope_kv: the rotated width must be even and at most {rot_dim}, got {rot}")
    if rot:
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, torch.float32)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be contiguous float32 [positions, {rot // 2}]")
    _gpu(q_out, "q_out", q_raw.dtype)
    if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * key_dim):
        raise KernelError("latent_rope_kv: q_out must be [rows, heads, key_dim]")
    if not v_dim <= page_dv:
        raise KernelError("latent_rope_kv: the values' pages are narrower than the values")
    _check_pages(k_pages, v_pages, page_table, n_heads, key_dim, q_raw.dtype, page_dv)
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows):
            raise KernelError(f"{name}: needs {rows} entries")
    _check(_fn("latent", "dryft_latent_rope_kv")(
        _ptr(q_raw), _ptr(kv), _ptr(down), down.stride(0), krot_col, _ptr(cos), _ptr(sin), rot, _ptr(row_slot),
        _ptr(row_pos), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1],
        int(bool(write_kv)), rows, n_heads, plain, rot_dim, v_dim, page_dv, int(bool(pairs)), is_f32, _stream()),
        "latent_rope_kv")


def head_gate(attn, down, g_col: int, out, n_heads: int, v_dim: int, per_element: bool = False) -> None:
    """``out[row, head, :] = attn[row, head, :v_dim] * sigmoid(down[row, g_col + head])``; ``attn``'s heads may be
    wider than ``v_dim``, ``out`` is packed ``[rows, heads * v_dim]``. With ``per_element`` every output has a gate
    of its own, ``down[row, g_col + head * v_dim + j]``."""
    _gpu(attn, "attn")
    rows = down.shape[0]
    _gpu(down, "down", attn.dtype)
    _gpu(out, "out", attn.dtype)
    in_dim = attn.numel() // max(1, rows * n_heads)
    if not (attn.is_contiguous() and attn.numel() == rows * n_heads * in_dim and in_dim >= v_dim):
        raise KernelError("head_gate: attn must be contiguous [rows, heads, >= v_dim]")
    if not (out.shape == (rows, n_heads * v_dim) and out.is_contiguous()):
        raise KernelError("head_gate: out must be contiguous [rows, heads * v_dim]")
    if not (down.stride(1) == 1 and 0 <= g_col and g_col + n_heads * (v_dim if per_element else 1) <= down.shape[1]):
        raise KernelError("head_gate: the gates lie outside down's columns")
    _check(_fn("latent", "dryft_head_gate")(_ptr(attn), _ptr(down), down.stride(0), g_col, _ptr(out), rows, n_heads,
                                            in_dim, v_dim, int(bool(per_element)), _float_flag(attn, "attn"), _stream()),
           "head_gate")


# ------------------------------------------------------------------------------------------ routed experts
MOE_MAX_EXPERTS = 512
MOE_TILE = 64


def moe_route(logits, correction, n_experts: int, groups: int, keep: int, scale: float, chosen, weights, *,
              softmax: bool = False, group_best: bool = False, renorm: bool = True) -> None:
    """Per row of float32 ``logits`` (their first ``n_experts`` columns): the ``top`` experts by ``sigmoid + correction``
    among the ``keep`` best of ``groups`` groups (a group's score: its two largest such scores), and their weights
    ``sigmoid / (sum of the chosen sigmoids + 1e-20) * scale``. ``chosen`` int32 and ``weights`` float32 ``[rows, top]``.
    ``softmax``: scores are the softmax over all experts instead; ``correction`` None: none; ``group_best``: a group
    scores as its best expert; ``renorm`` off: the weights are the scores times ``scale`` as they are."""
    _gpu(logits, "logits", torch.float32)
    rows, top = chosen.shape
    if not (logits.dim() == 2 and logits.shape[0] == rows and logits.stride(1) == 1 and logits.shape[1] >= n_experts):
        raise KernelError("moe_route: logits must be float32 [rows, >= experts] with unit column stride")
    if correction is not None:
        _f32_vector(correction, "correction", n_experts)
    _gpu(chosen, "chosen", torch.int32)
    _gpu(weights, "weights", torch.float32)
    if not (chosen.is_contiguous() and weights.shape == (rows, top) and weights.is_contiguous()):
        raise KernelError("moe_route: chosen and weights must be contiguous [rows, top]")
    if not (1 <= top <= n_experts <= MOE_MAX_EXPERTS and 1 <= keep <= groups <= 64 and n_experts % groups == 0 and
            keep * (n_experts // groups) >= top):
        raise KernelError("moe_route: sizes the router does not take")
    _check(_fn("moe", "dryft_moe_route")(_ptr(logits), logits.stride(0), _ptr(correction), n_experts, groups, keep, top,
                                         float(scale), _ptr(chosen), _ptr(weights), rows, int(bool(softmax)),
                                         int(bool(group_best)), int(bool(renorm)), _stream()), "moe_route")


class MoePlan:
    """Where each (row, expert) pair of a step sits once the pairs are sorted by expert, and the tiles of the sorted
    run, all on the device. ``most_places``: what the host knows no expert's run to exceed (a row chooses an expert
    once, so the step's rows)."""

    def __init__(self, n_pairs: int, n_experts: int, device, most_places: int | None = None):
        self.n_pairs = n_pairs
        self.most_places = n_pairs if most_places is None else int(most_places)
        self.max_tiles = n_pairs // MOE_TILE + min(n_experts, n_pairs)
        i32 = dict(dtype=torch.int32, device=device)
        self.sorted_pair = torch.empty(n_pairs, **i32)
        self.place_of = torch.empty(n_pairs, **i32)
        self.tiles = torch.empty((3, self.max_tiles), **i32)        # expert | first place | places
        self.n_tiles = torch.empty(1, **i32)


def moe_plan(chosen, n_experts: int) -> MoePlan:
    _gpu(chosen, "chosen", torch.int32)
    if not chosen.is_contiguous():
        raise KernelError("moe_plan: chosen must be contiguous")
    plan = MoePlan(chosen.numel(), n_experts, chosen.device, most_places=chosen.shape[0] if chosen.dim() == 2 else None)
    _check(_fn("moe", "dryft_moe_plan")(_ptr(chosen), plan.n_pairs, n_experts, _ptr(plan.sorted_pair), _ptr(plan.place_of),
                                        _ptr(plan.tiles[0]), _ptr(plan.tiles[1]), _ptr(plan.tiles[2]), _ptr(plan.n_tiles),
                                        plan.max_tiles, _stream()), "moe_plan")
    return plan


def moe_table_route(tokens, table, n_experts: int, chosen, weights) -> None:
    """A router that is a table: row ``r`` goes to the experts ``table[tokens[r]]`` (int32 ``[vocab, top]``), each with
    weight ``1 / top``. ``chosen`` int32 and ``weights`` float32 ``[rows, top]``."""
    _gpu(tokens, "tokens", torch.int32)
    _gpu(table, "table", torch.int32)
    _gpu(chosen, "chosen", torch.int32)
    _gpu(weights, "weights", torch.float32)
    rows, top = chosen.shape
    if not (tokens.is_contiguous() and tokens.numel() == rows and table.dim() == 2 and table.shape[1] == top and
            table.is_contiguous() and chosen.is_contiguous() and weights.shape == (rows, top) and weights.is_contiguous()):
        raise KernelError("moe_table_route: tokens [rows], table [vocab, top], chosen and weights [rows, top], contiguous")
    _check(_fn("moe", "dryft_moe_table_route")(_ptr(tokens), _ptr(table), _ptr(chosen), _ptr(weights), rows, top,
                                               table.shape[0], n_experts, _stream()), "moe_table_route")


def moe_products(a, w, plan: MoePlan, out, top: int, glu: tuple | None = None, act: str | None = None) -> None:
    """``out[place] = W_e a_row`` for every place of the plan, ``e`` the place's expert. ``top`` > 0: ``a`` is
    ``[rows, K]`` and a place's operand is row ``pair // top``; ``top`` == 0: ``a`` is ``[pairs, K]`` in place order.
    ``w`` is ``[experts, N, K]``; with ``glu = (limit, alpha)`` it holds gate rows then up rows (``N = 2 I``) and
    ``out [pairs, I]`` receives the clamped gated unit of the two, ``g sigmoid(alpha g) (u + 1)``; ``glu = (limit, alpha,
    offset)`` puts ``offset`` in the place of that 1 (``(inf, 1, 0)`` is ``silu(gate) * up``). ``out`` may be float32
    for a plain product. ``act="relu2"`` (no gate): ``out`` receives the square of relu of the product."""
    if act not in (None, "relu2") or (act and glu):
        raise KernelError("moe_products: act is None or 'relu2', and goes without a gate")
    _gpu(a, "a")
    _gpu(w, "w", a.dtype)
    _gpu(out, "out")
    k = a.shape[1]
    n_out = w.shape[1] // 2 if glu else w.shape[1]
    if not (a.dim() == 2 and a.stride(1) == 1 and w.dim() == 3 and w.shape[2] == k and w.is_contiguous()):
        raise KernelError("moe_products: a [rows, K] with unit column stride, w contiguous [experts, N, K]")
    if top == 0 and a.shape[0] != plan.n_pairs:
        raise KernelError("moe_products: an operand in place order needs a row per pair")
    if top > 0 and a.shape[0] * top != plan.n_pairs:
        raise KernelError("moe_products: the plan was made for another number of rows")
    if not (out.shape == (plan.n_pairs, n_out) and out.is_contiguous() and out.dtype in (a.dtype, torch.float32)):
        raise KernelError(f"moe_products: out must be contiguous [{plan.n_pairs}, {n_out}] in a's dtype or float32")
    if glu and out.dtype != a.dtype:
        raise KernelError("moe_products: the gated unit is stored in the activation dtype")
    limit, alpha, offset = (tuple(glu) + (1.0,))[:3] if glu else (0.0, 0.0, 0.0)
    _check(_fn("moe", "dryft_moe_product")(
        _ptr(a), a.stride(0), _ptr(w), _ptr(plan.sorted_pair), _ptr(plan.tiles[0]), _ptr(plan.tiles[1]),
        _ptr(plan.tiles[2]), _ptr(plan.n_tiles), plan.max_tiles, _ptr(out), 1 if out.dtype == torch.float32 else 0,
        int(top), n_out, k, 1 if glu else 0, float(limit), float(alpha), float(offset), 1 if act else 0, plan.most_places,
        _float_flag(a, "a"), _stream()),
        "moe_products")


def moe_combine(y, plan: MoePlan, weights, shared, logits, shared_col: int, out) -> None:
    """``out[row] = sum_k weights[row, k] * y[place of (row, k)] + sigmoid(logits[row, shared_col]) * shared[row]``
    (the last term only with ``shared``; without ``logits`` the shared expert's output is added as it is)."""
    _gpu(y, "y", torch.float32)
    rows, top = weights.shape
    width = y.shape[1]
    _gpu(weights, "weights", torch.float32)
    _gpu(out, "out")
    if not (y.shape == (rows * top, width) and y.is_contiguous() and weights.is_contiguous() and
            out.shape == (rows, width) and out.is_contiguous() and plan.n_pairs == rows * top):
        raise KernelError("moe_combine: y [pairs, width], weights [rows, top], out [rows, width], all contiguous")
    if shared is not None:
        _gpu(shared, "shared", out.dtype)
        if not (shared.shape == (rows, width) and shared.is_contiguous()):
            raise KernelError("moe_combine: shared [rows, width] contiguous")
    if shared is not None and logits is not None:
        _gpu(logits, "logits", torch.float32)
        if not (logits.stride(1) == 1 and 0 <= shared_col < logits.shape[1] and logits.shape[0] == rows):
            raise KernelError("moe_combine: the shared expert's logit must be a column of logits")
    _check(_fn("moe", "dryft_moe_combine")(_ptr(y), _ptr(plan.place_of), _ptr(weights), _ptr(shared), _ptr(logits),
                                           logits.stride(0) if (shared is not None and logits is not None) else 0, shared_col, _ptr(out), rows, top,
                                           width, _float_flag(out, "out"), _stream()), "moe_combine")


# ------------------------------------------------------------------------------- scaled embedding, pair of branches
def embed_scaled(tokens: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
    """``out[r] = table[tokens[r]] * scale`` as float32: the start of a float32 residual stream."""
    _gpu(tokens, "tokens", torch.int32)
    _gpu(table, "table")
    _gpu(out, "out", torch.float32)
    n = tokens.numel()
    if not (table.dim() == 2 and table.is_contiguous() and tokens.is_contiguous() and out.is_contiguous() and
            out.shape == (n, table.shape[1])):
        raise KernelError("embed_scaled: table [vocab, hidden], out float32 [rows, hidden], all contiguous")
    _check(_fn("embed", "dryft_embed_scaled")(_ptr(tokens), _ptr(table), _ptr(out), n, table.shape[1], table.shape[0],
                                              float(scale), _float_flag(table, "table"), _stream()), "embed_scaled")
    return out


def _branch(delta, rows: int, width: int, act: torch.dtype, what: str):
    """(pointer, kind, parts, stride) of a branch's output: a tensor ``[rows, width]`` in the activation dtype, or float32
    partial sums ``(data [n, rows, width], n)``."""
    if isinstance(delta, tuple):
        data, n = delta
        _gpu(data, what, torch.float32)
        if not (data.dim() == 3 and data.shape[1:] == (rows, width) and data.is_contiguous() and data.shape[0] >= n >= 1):
            raise KernelError(f"{what}: partial sums must be contiguous float32 [n, rows, width]")
        return data, 2, int(n), rows * width
    _gpu(delta, what, act)
    if not (delta.shape == (rows, width) and delta.is_contiguous()):
        raise KernelError(f"{what}: must be contiguous [rows, width] in the activation dtype")
    return delta, 1, 1, rows * width


def rms_pair_mean(a, a_bias, a_weight, b, b_bias, b_weight, eps: float, out: torch.Tensor, act: torch.dtype) -> torch.Tensor:
    """``out = (rmsnorm(a + a_bias) * a_weight + rmsnorm(b + b_bias) * b_weight) / 2`` per row, float32. ``a`` and ``b``
    are tensors in the activation dtype ``act`` or float32 partial sums ``(data, n)``; biases (optional) and weights
    are float32 vectors."""
    _gpu(out, "out", torch.float32)
    rows, width = out.shape
    if not out.is_contiguous():
        raise KernelError("rms_pair_mean: out must be contiguous")
    pa, ka, na, sa = _branch(a, rows, width, act, "a")
    pb, kb, nb, sb = _branch(b, rows, width, act, "b")
    for name, t in (("a_bias", a_bias), ("b_bias", b_bias)):
        if t is not None:
            _f32_vector(t, name, width)
    _f32_vector(a_weight, "a_weight", width)
    _f32_vector(b_weight, "b_weight", width)
    _check(_fn("norm", "dryft_rms_pair_mean")(_ptr(pa), ka, na, sa, _ptr(a_bias), _ptr(a_weight), _ptr(pb), kb, nb, sb,
                                              _ptr(b_bias), _ptr(b_weight), _ptr(out), rows, width, float(eps),
                                              1 if act == torch.float32 else 0, _stream()), "rms_pair_mean")
    return out


# --------------------------------------------------------------------------------------- short causal convolution
CONV_MAX_TAPS = 16


def _row_facts(rows: int, **tensors) -> None:
    for name, t in tensors.items():
        _gpu(t, name, torch.int32)
        if not (t.is_contiguous() and t.numel() >= rows):
            raise KernelError(f"{name}: needs {rows} contiguous entries")


def causal_conv(u, col: int, channels: int, in_bias, weight, out_bias, silu: bool, row_slot, row_seq, row_pos, seq_start,
                tail, out, weight_t=None) -> torch.Tensor:
    """``out[t, c] = act(sum_j weight[c, j] * v[t - taps + 1 + j, c] + out_bias[c])`` with ``v = u[:, col + c] + in_bias[c]``
    over each sequence's own rows, the ``taps - 1`` inputs before the step's first row from ``tail [slots, taps - 1,
    channels]`` (float32), zeros before the sequence's start. ``act`` is the identity or (``silu``) ``z sigmoid(z)``.
    Rows of sequences that sit out give zeros. The tail is not touched (``conv_tail`` moves it on). With ``weight_t``
    (the same weights as contiguous float32 ``[taps, channels]``) and rows that start at multiples of 8 channels a thread
    takes 8 channels at a time."""
    _gpu(u, "u")
    rows = u.shape[0]
    if not (u.dim() == 2 and u.stride(1) == 1 and 0 <= col and col + channels <= u.shape[1]):
        raise KernelError("causal_conv: u [rows, columns] with unit column stride that holds the channels")
    _gpu(weight, "weight", torch.float32)
    if not (weight.dim() == 2 and weight.shape[0] == channels and weight.is_contiguous() and
            1 <= weight.shape[1] <= CONV_MAX_TAPS):
        raise KernelError(f"causal_conv: weight must be contiguous float32 [channels, 1..{CONV_MAX_TAPS}]")
    taps = weight.shape[1]
    if weight_t is not None:
        _gpu(weight_t, "weight_t", torch.float32)
        if not (weight_t.shape == (taps, channels) and weight_t.is_contiguous()):
            raise KernelError(f"causal_conv: weight_t must be contiguous float32 [{taps}, {channels}]")
    for name, t in (("in_bias", in_bias), ("out_bias", out_bias)):
        if t is not None:
            _f32_vector(t, name, channels)
    _row_facts(rows, row_slot=row_slot, row_seq=row_seq, row_pos=row_pos)
    _gpu(seq_start, "seq_start", torch.int32)
    if taps > 1:
        _gpu(tail, "tail", torch.float32)
        if not (tail.dim() == 3 and tail.shape[1:] == (taps - 1, channels) and tail.is_contiguous()):
            raise KernelError(f"causal_conv: tail must be contiguous float32 [slots, {taps - 1}, {channels}]")
    _gpu(out, "out", u.dtype)
    if not (out.shape == (rows, channels) and out.is_contiguous()):
        raise KernelError("causal_conv: out must be contiguous [rows, channels]")
    _check(_fn("conv", "dryft_causal_conv")(_ptr(u), u.stride(0), col, _ptr(in_bias), _ptr(weight), _ptr(weight_t),
                                            _ptr(out_bias), taps,
                                            1 if silu else 0, _ptr(row_slot), _ptr(row_seq), _ptr(row_pos),
                                            _ptr(seq_start), _ptr(tail) if taps > 1 else 0, _ptr(out), rows, channels,
                                            _float_flag(u, "u"), _stream()), "causal_conv")
    return out


def conv_tail(u, col: int, channels: int, in_bias, taps: int, seq_slot, cu_rows, q_len, n_seqs: int, tail) -> None:
    """Moves each sequence's tail on past the step's rows: afterwards it holds the last ``taps - 1`` inputs
    ``u[:, col + c] + in_bias[c]`` of the sequence (older ones from the tail before where the step brought fewer)."""
    if taps <= 1:
        return
    _gpu(u, "u")
    if not (u.dim() == 2 and u.stride(1) == 1 and 0 <= col and col + channels <= u.shape[1]):
        raise KernelError("conv_tail: u [rows, columns] with unit column stride that holds the channels")
    if in_bias is not None:
        _f32_vector(in_bias, "in_bias", channels)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    _gpu(tail, "tail", torch.float32)
    if not (tail.dim() == 3 and tail.shape[1:] == (taps - 1, channels) and tail.is_contiguous() and taps <= CONV_MAX_TAPS):
        raise KernelError(f"conv_tail: tail must be contiguous float32 [slots, {taps - 1}, {channels}]")
    _check(_fn("conv", "dryft_conv_tail")(_ptr(u), u.stride(0), col, _ptr(in_bias), taps, _ptr(seq_slot), _ptr(cu_rows),
                                          _ptr(q_len), _ptr(tail), n_seqs, channels, _float_flag(u, "u"), _stream()),
           "conv_tail")


# ------------------------------------------------------------------------- norm per head, rotation over halves, append
def norm_rope_half_kv(src, q_col: int, k_col: int, v_col: int, q_weight, k_weight, eps: float, cos, sin, rot: int,
                      row_slot, row_pos, q_out, k_pages, v_pages, page_table, write_kv: bool, n_heads: int, n_kv: int,
                      head_dim: int, v_dim: int, page_dim: int = 0) -> None:
    """Every q and k head of ``src`` divided by its root mean square and multiplied by ``q_weight`` / ``k_weight``
    (float32 ``[head_dim]``; None: the head passes), then feature ``i`` of its first ``rot`` turned with feature
    ``i + rot / 2`` by float32 tables ``[positions, rot / 2]``; queries to ``q_out [rows, heads, head_dim]`` and, when
    ``write_kv``, keys and (untouched) values of width ``v_dim`` to their pages. ``page_dim`` > 0: pages and the rows of
    ``q_out`` are that wide for keys and values alike (at least as wide as either); what lies behind a head's own
    features is not written, so ``q_out`` and the pages must have started as zeros."""
    _gpu(src, "src")
    is_f32 = _float_flag(src, "src")
    rows = src.shape[0]
    if not (src.dim() == 2 and src.stride(1) == 1):
        raise KernelError("norm_rope_half_kv: src must be [rows, columns] with unit column stride")
    ends = (q_col + n_heads * head_dim, k_col + n_kv * head_dim, v_col + n_kv * v_dim)
    if min(q_col, k_col, v_col) < 0 or max(ends) > src.shape[1]:
        raise KernelError("norm_rope_half_kv: q, k or v lie outside the columns of src")
    if rot % 2 or not 0 <= rot <= head_dim or head_dim > 256:
        raise KernelError(f"norm_rope_half_kv: the rotated width must be even and at most {head_dim} <= 256, got {rot}")
    if rot:
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, torch.float32)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be contiguous float32 [positions, {rot // 2}]")
    for name, t in (("q_weight", q_weight), ("k_weight", k_weight)):
        if t is not None:
            _f32_vector(t, name, head_dim)
    _gpu(q_out, "q_out", src.dtype)
    page_dim = int(page_dim)
    if page_dim and page_dim < max(head_dim, v_dim):
        raise KernelError("norm_rope_half_kv: padded pages must be at least as wide as keys and values")
    if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * (page_dim or head_dim)):
        raise KernelError("norm_rope_half_kv: q_out must be [rows, heads, head_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv, page_dim or head_dim, src.dtype, page_dim or v_dim)
    _row_facts(rows, row_slot=row_slot, row_pos=row_pos)
    _check(_fn("rope_kv", "dryft_norm_rope_half_kv")(
        _ptr(src), src.stride(0), q_col, k_col, v_col, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos), _ptr(sin),
        rot, _ptr(row_slot), _ptr(row_pos), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _ptr(page_table),
        page_table.shape[1], int(bool(write_kv)), rows, n_heads, n_kv, head_dim, v_dim, page_dim, is_f32, _stream()),
        "norm_rope_half_kv")


# ------------------------------------------------------------------------------------------ state-space mixer
SSM_MAX_STATE = 256


def _segment_facts(who: str, segments, n_seqs: int, write_state: bool):
    """``(rows per segment, prefix sums, bound)`` of a walk cut into segments, checked; zeros and None for a whole walk."""
    if segments is None:
        return 0, None, 0
    seg_rows, seg_cu, max_segs = segments
    _gpu(seg_cu, "segment prefix sums", torch.int32)
    if not (seg_cu.numel() >= n_seqs + 1 and seg_rows > 0 and write_state):
        raise KernelError(f"{who}: segments of a positive number of rows, prefix sums for every sequence, and a state "
                          "that is written back")
    return int(seg_rows), seg_cu, int(max_segs)


def ssm_scan(xbc, x_col: int, b_col: int, c_col: int, dt_raw, dt_bias, a_log, d_skip, seq_slot, cu_rows, q_len,
             n_seqs: int, state, y, n_heads: int, head_dim: int, n_state: int, groups: int, write_state: bool,
             segments=None) -> None:
    """Per sequence and head, over the sequence's rows of the step in order, from ``state [slots, heads, n_state,
    head_dim]`` (float32): ``dt = softplus(dt_raw + dt_bias)``, ``S <- exp(-exp(a_log) dt) S + dt B x^T``,
    ``y = S^T C + d_skip x``. ``x [heads, head_dim]``, ``B`` and ``C [groups, n_state]`` are runs of columns of ``xbc``
    (activation dtype), ``dt_raw`` float32 ``[rows, >= heads]``, ``y`` float32 ``[rows, heads * head_dim]`` (rows of
    sequences that sit out are not written). ``segments = (rows per segment, prefix sums of segments over the
    sequences, their bound)``: long sequences run as segments side by side, in three launches (every segment's summary
    from a zero state, the state that enters each, every segment's read-outs)."""
    _gpu(xbc, "xbc")
    rows = xbc.shape[0]
    inner = n_heads * head_dim
    if not (xbc.dim() == 2 and xbc.stride(1) == 1 and min(x_col, b_col, c_col) >= 0 and
            max(x_col + inner, b_col + groups * n_state, c_col + groups * n_state) <= xbc.shape[1]):
        raise KernelError("ssm_scan: x, B or C lie outside the columns of xbc")
    _gpu(dt_raw, "dt_raw", torch.float32)
    if not (dt_raw.dim() == 2 and dt_raw.shape[0] == rows and dt_raw.stride(1) == 1 and dt_raw.shape[1] >= n_heads):
        raise KernelError("ssm_scan: dt_raw must be float32 [rows, >= heads] with unit column stride")
    for name, t in (("dt_bias", dt_bias), ("a_log", a_log), ("d_skip", d_skip)):
        _f32_vector(t, name, n_heads)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    _gpu(state, "state", torch.float32)
    if not (state.dim() == 4 and state.shape[1:] == (n_heads, n_state, head_dim) and state.is_contiguous()):
        raise KernelError(f"ssm_scan: state must be contiguous float32 [slots, {n_heads}, {n_state}, {head_dim}]")
    _gpu(y, "y", torch.float32)
    if not (y.shape == (rows, inner) and y.is_contiguous()):
        raise KernelError("ssm_scan: y must be contiguous float32 [rows, heads * head_dim]")
    if not (0 < n_state <= SSM_MAX_STATE and groups > 0 and n_heads % groups == 0):
        raise KernelError(f"ssm_scan: a state of 1..{SSM_MAX_STATE} rows, heads a multiple of groups")
    seg_rows, seg_cu, max_segs = _segment_facts("ssm_scan", segments, n_seqs, write_state)
    if segments is not None and max_segs <= 0:
        return
    seg_state = seg_decay = None
    if segments is not None:
        seg_state = torch.empty((max_segs, n_heads, n_state, head_dim), dtype=torch.float32, device=xbc.device)
        seg_decay = torch.empty((max_segs, n_heads), dtype=torch.float32, device=xbc.device)
    _check(_fn("ssm", "dryft_ssm_scan")(_ptr(xbc), xbc.stride(0), x_col, b_col, c_col, _ptr(dt_raw), dt_raw.stride(0),
                                        _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(seq_slot), _ptr(cu_rows),
                                        _ptr(q_len), _ptr(state), _ptr(y), n_seqs, n_heads, head_dim, n_state, groups,
                                        int(bool(write_state)), _ptr(seg_cu), max_segs, seg_rows, _ptr(seg_state),
                                        _ptr(seg_decay), _float_flag(xbc, "xbc"), _stream()), "ssm_scan")


def gate_part_norm(y, z, z_col: int, weight, row_slot, out, parts: int, eps: float) -> None:
    """``v = y * silu(z[:, z_col : z_col + inner])``, each of ``parts`` equal runs of ``v`` divided by its own root mean
    square, times ``weight``: the gate comes before the norm. ``y`` float32, ``z`` and ``out`` in the activation dtype."""
    _gpu(y, "y", torch.float32)
    rows, inner = y.shape
    _gpu(z, "z")
    _gpu(out, "out", z.dtype)
    if not (y.is_contiguous() and z.dim() == 2 and z.shape[0] == rows and z.stride(1) == 1 and 0 <= z_col and
            z_col + inner <= z.shape[1] and out.shape == (rows, inner) and out.is_contiguous()):
        raise KernelError("gate_part_norm: y and out contiguous [rows, inner], the gate a run of columns of z")
    if parts <= 0 or inner % parts:
        raise KernelError(f"gate_part_norm: {inner} values do not split into {parts} equal parts")
    _f32_vector(weight, "weight", inner)
    _row_facts(rows, row_slot=row_slot)
    _check(_fn("ssm", "dryft_gate_part_norm")(_ptr(y), _ptr(z), z.stride(0), z_col, _ptr(weight), _ptr(row_slot), _ptr(out),
                                              rows, inner, parts, float(eps), _float_flag(z, "z"), _stream()),
           "gate_part_norm")


# ------------------------------------------------------------------------------------------ gated delta rule
DELTA_MAX_DIM = 256


def delta_steps(qkv, q_col: int, k_col: int, v_col: int, gates, a_col: int, b_col: int, dt_bias, a_log, seq_slot, cu_rows,
                q_len, n_seqs: int, state, out, n_heads: int, n_groups: int, key_dim: int, value_dim: int, q_scale: float,
                unit_eps: float, write_state: bool, segments=None) -> None:
    """Per sequence and head, over the sequence's rows of the step in order, from ``state [slots, heads, key_dim,
    value_dim]`` (float32): ``S <- g S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q`` with
    ``g = exp(-exp(a_log) softplus(gates[:, a_col + h] + dt_bias))``, ``beta = sigmoid(gates[:, b_col + h])``, q and k
    (``n_groups`` of them, runs of columns of ``qkv``) made unit vectors with ``unit_eps`` under the root, q times
    ``q_scale``. ``out`` float32 ``[rows, heads * value_dim]`` (rows of sequences that sit out are not written).
    ``segments = (rows per segment, prefix sums of segments over the sequences, their bound)``: long sequences run as
    segments side by side, in three launches (every segment's summary, the state it reaches from zero and the map it
    applies to the state that enters it; the state that enters each; every segment's read-outs)."""
    _gpu(qkv, "qkv")
    rows = qkv.shape[0]
    if not (qkv.dim() == 2 and qkv.stride(1) == 1 and min(q_col, k_col, v_col) >= 0 and
            max(q_col + n_groups * key_dim, k_col + n_groups * key_dim, v_col + n_heads * value_dim) <= qkv.shape[1]):
        raise KernelError("delta_steps: q, k or v lie outside the columns of qkv")
    _gpu(gates, "gates", torch.float32)
    if not (gates.dim() == 2 and gates.shape[0] == rows and gates.stride(1) == 1 and min(a_col, b_col) >= 0 and
            max(a_col, b_col) + n_heads <= gates.shape[1]):
        raise KernelError("delta_steps: gates must be float32 [rows, columns] that hold a and b for every head")
    _f32_vector(dt_bias, "dt_bias", n_heads)
    _f32_vector(a_log, "a_log", n_heads)
    _seq_facts(seq_slot, cu_rows, q_len, n_seqs)
    _gpu(state, "state", torch.float32)
    if not (state.dim() == 4 and state.shape[1:] == (n_heads, key_dim, value_dim) and state.is_contiguous()):
        raise KernelError(f"delta_steps: state must be contiguous float32 [slots, {n_heads}, {key_dim}, {value_dim}]")
    _gpu(out, "out", torch.float32)
    if not (out.shape == (rows, n_heads * value_dim) and out.is_contiguous()):
        raise KernelError("delta_steps: out must be contiguous float32 [rows, heads * value_dim]")
    if not (0 < key_dim <= DELTA_MAX_DIM and n_groups > 0 and n_heads % n_groups == 0):
        raise KernelError(f"delta_steps: keys of 1..{DELTA_MAX_DIM} features, heads a multiple of the key heads")
    seg_rows, seg_cu, max_segs = _segment_facts("delta_steps", segments, n_seqs, write_state)
    if segments is not None and max_segs <= 0:
        return
    seg_state = seg_trans = None
    if segments is not None:
        seg_state = torch.empty((max_segs, n_heads, key_dim, value_dim), dtype=torch.float32, device=qkv.device)
        seg_trans = torch.empty((max_segs, n_heads, key_dim, key_dim), dtype=torch.float32, device=qkv.device)
    _check(_fn("delta", "dryft_delta_steps")(
        _ptr(qkv), qkv.stride(0), q_col, k_col, v_col, _ptr(gates), gates.stride(0), a_col, b_col, _ptr(dt_bias),
        _ptr(a_log), _ptr(seq_slot), _ptr(cu_rows), _ptr(q_len), _ptr(state), _ptr(out), n_seqs, n_heads, n_groups,
        key_dim, value_dim, float(q_scale), float(unit_eps), int(bool(write_state)), _ptr(seg_cu), max_segs, seg_rows,
        _ptr(seg_state), _ptr(seg_trans), _float_flag(qkv, "qkv"), _stream()), "delta_steps")
