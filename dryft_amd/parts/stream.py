"""A float32 residual stream with a norm on both sides of every branch.

``x <- x + norm_b(branch(norm_a(x)))``: the branch's output is normed before it is added, and the stream is
normed again for the next branch. The stream stays float32 whatever the activation dtype, so that the sum
over many layers (and over several passes through the same layers) is not rounded to 8 bits each time.
Every residual sum is folded into the norm that follows it: a block hands its last branch's output on
unadded (``Deferred``), and the next block's first kernel norms it, adds it, adds whatever else has come
due meanwhile, and norms the stream for its own first branch, in one launch.

``StreamRMSNorm``    the norm itself: ``x / sqrt(mean(x^2) + eps) * w`` in float, rounded once.
``StreamLayerNorm``  the same with the mean taken off first: ``(x - mean) / sqrt(var + eps) * w``, no bias.
``SandwichBlock``    mixer and feed-forward, each between two norms; ``SandwichMixerBlock`` has the mixer alone.
``PostNormBlock``    ``x <- x + norm(branch(x))``: the branches read the stream as it is, only their outputs are
                     normed; ``PostNormMixerBlock`` has the mixer alone.
``PreNormBlock``     ``x <- x + branch(norm(x))``: a norm in front of every branch and none behind it; optionally a
                     third sublayer (``TokenSide``) that reads the stream as it is.
``TokenSide``        what a token id brings to a layer: a few numbers from a table, gated by the stream, projected
                     to the width and rms-normed.
``PassEntry``        what a pass over a run of layers begins with: one learned vector per pass is added to the
                     stream, and from the second pass on the embedding's output once more.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from ..weights.spec import VECTOR
from . import register_block, register_part
from .base import Deferred, FeedForward, Mixer, Norm, Part, Partials, StepContext, StreamPart, matrix
from .linear import linear


class StreamRMSNorm(Norm):
    """``offset``: what the stored weight is counted from (1 for weights stored around zero); ``scale``: a factor on
    the whole weight (a head's factor on its logits rides here). A stream of several copies ``[copies, rows, width]``
    (``parts/hyper.py``) is normed as the sum of its copies."""

    centred = False           # does the norm take the mean off first (a layer norm without bias)?

    def __init__(self, size: int, eps: float, offset: float = 0.0, scale: float = 1.0):
        self.size, self.eps, self.offset, self.scale = int(size), float(eps), float(offset), float(scale)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {"weight": ((self.size,), VECTOR, "zeros" if self.offset == 1.0 else "ones")}

    def load(self, tensors):
        self.weight = ((tensors["weight"].float() + self.offset) * self.scale).contiguous()

    def kernel_modules(self, dtype):
        return ("norm",)

    def forward(self, x: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
        if x.dim() == 3:
            return self.add_forward(x, None, dtype)[1]
        y = torch.empty(x.shape, dtype=dtype or self.compute_dtype or x.dtype, device=x.device)
        ops.stream_norm(x, None, None, None, None, self.weight, self.eps, None, y, y.dtype, centred=self.centred)
        return y

    def add_forward(self, res: torch.Tensor, delta, dtype: torch.dtype | None = None, in_place: bool = True):
        """``(stream, norm(stream))`` after everything in ``delta`` (a ``Deferred``, a tensor, ``Partials`` or None)
        has been added to ``res``. The stream comes back as float32: ``res`` itself, updated, when it is float32 and
        ``in_place`` allows; the normed rows in ``dtype`` (default: the dtype the model computes in)."""
        pending = as_deferred(delta)
        act = dtype or self.compute_dtype or _activation_dtype(res, pending)
        if res.dim() == 3 or pending.route is not None:
            from .hyper import read_streams
            return read_streams(res, pending, None, self, act, keep=False)
        own = in_place and res.dtype == torch.float32 and res.is_contiguous()
        out = res if own else torch.empty(res.shape, dtype=torch.float32, device=res.device)
        y = torch.empty(res.shape, dtype=act, device=res.device)
        _launch(res, pending, self.weight, self.eps, out, y, act, centred=self.centred)
        return out, y


class StreamLayerNorm(StreamRMSNorm):
    """``(x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w`` in float, without a bias."""

    centred = True


def as_deferred(pending) -> Deferred:
    if pending is None:
        return Deferred()
    if isinstance(pending, Deferred):
        return pending
    return Deferred(delta=pending)


def _activation_dtype(x: torch.Tensor, pending: Deferred) -> torch.dtype:
    for t in (pending.delta, pending.rows):
        if isinstance(t, torch.Tensor):
            return t.dtype
    return x.dtype


def _launch(x, pending: Deferred, weight, eps, x_out, y, act, centred: bool = False, plain_read: bool = False) -> None:
    delta = pending.delta
    if isinstance(delta, Partials):
        delta = (delta.data, delta.count)
    post = pending.norm.weight if pending.norm is not None else None
    if pending.norm is not None and pending.norm.eps != eps:
        raise ValueError("the norms around one residual sum differ in eps; one launch takes one")
    ops.stream_norm(x, delta, post, pending.rows, pending.vector, weight, eps, x_out, y, act,
                    post_centred=bool(getattr(pending.norm, "centred", False)), centred=centred, plain_read=plain_read)


def read_plain(x: torch.Tensor, pending, act: torch.dtype):
    """``(stream, stream in act)`` after everything pending has entered the float32 stream ``x`` (updated in place):
    for sublayers that read the stream as it is. Nothing pending and a float32 reader: the stream itself, no launch."""
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("a stream that is read as it is must be contiguous float32")
    if pending is None and act == torch.float32:
        return x, x
    pending = as_deferred(pending)
    y = torch.empty(x.shape, dtype=act, device=x.device)
    eps = pending.norm.eps if pending.norm is not None else 0.0
    _launch(x, pending, None, eps, x if pending.delta is not None else None, y, act, plain_read=True)
    return x, y


def settle(x: torch.Tensor, pending, eps: float = 0.0) -> torch.Tensor:
    """The stream with everything pending added, as a new float32 tensor (for looking at it; the compute path never
    needs the stream without the norm that follows)."""
    pending = as_deferred(pending)
    if x.dim() == 3 or pending.route is not None:
        from .hyper import summed_streams
        return summed_streams(x, pending)
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    act = _activation_dtype(x, pending)
    _launch(x, pending, None, pending.norm.eps if pending.norm is not None else eps, out, None, act)
    return out


class SandwichBlock:
    roles = ("mixer_norm", "mixer", "mixer_post_norm", "ffn_norm", "ffn", "ffn_post_norm")

    def __init__(self, mixer_norm: Norm, mixer: Mixer, mixer_post_norm: Norm, ffn_norm: Norm | None = None,
                 ffn: FeedForward | None = None, ffn_post_norm: Norm | None = None):
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ffn_norm, self.ffn, self.ffn_post_norm = ffn_norm, ffn, ffn_post_norm

    def parts(self):
        return {role: getattr(self, role) for role in self.roles}

    def forward(self, x, pending, ctx: StepContext, line, writes_cache: bool):
        # the embedding's output starts the stream and is read again later: it is never updated in place
        x, h = self.mixer_norm.add_forward(x, pending, ctx.dtype, in_place=x is not ctx.embedded)
        pending = Deferred(delta=self.mixer.forward(h, ctx, line, writes_cache), norm=self.mixer_post_norm)
        if self.ffn is None:
            return x, pending
        x, h = self.ffn_norm.add_forward(x, pending, ctx.dtype)
        return x, Deferred(delta=self.ffn.forward(h, ctx), norm=self.ffn_post_norm)


class SandwichMixerBlock(SandwichBlock):
    roles = ("mixer_norm", "mixer", "mixer_post_norm")


class PostNormBlock:
    """``x <- x + norm_a(mixer(x))``, then ``x <- x + norm_b(ffn(x))``: no norm in front of a sublayer. The stream is
    float32 from the embedding on; as everywhere here a sublayer's output is handed on unadded and enters the stream
    in the launch that also hands the next reader its rows."""

    roles = ("mixer", "mixer_post_norm", "ffn", "ffn_post_norm")

    def __init__(self, mixer: Mixer, mixer_post_norm: Norm, ffn: FeedForward | None = None,
                 ffn_post_norm: Norm | None = None):
        self.mixer, self.mixer_post_norm, self.ffn, self.ffn_post_norm = mixer, mixer_post_norm, ffn, ffn_post_norm

    def parts(self):
        return {role: getattr(self, role) for role in self.roles}

    def forward(self, x, pending, ctx: StepContext, line, writes_cache: bool):
        x, h = read_plain(x, pending, ctx.dtype)
        pending = Deferred(delta=self.mixer.forward(h, ctx, line, writes_cache), norm=self.mixer_post_norm)
        if self.ffn is None:
            return x, pending
        x, h = read_plain(x, pending, ctx.dtype)
        return x, Deferred(delta=self.ffn.forward(h, ctx), norm=self.ffn_post_norm)


class PostNormMixerBlock(PostNormBlock):
    roles = ("mixer", "mixer_post_norm")


class TokenSide(Part):
    """A sublayer fed by the token id: ``e`` = columns ``[index * dim, (index + 1) * dim)`` of ``table[token]``,
    ``g = gelu_tanh(W_gate x) * e``, ``y = W_proj g``, and what enters the stream is ``y / sqrt(mean(y^2) + eps) * w``
    (an rms norm with a plain weight, whatever the model's own norm is). ``x`` is the stream as it is, not normed.
    ``forward`` hands the output on unadded, with its norm, as every sublayer of a float32 stream does. The table is
    one tensor for all layers (the plan gives every layer's part the same checkpoint name)."""

    def __init__(self, hidden_size: int, dim: int, index: int, count: int, vocab_size: int, eps: float):
        self.hidden, self.dim, self.index, self.count = int(hidden_size), int(dim), int(index), int(count)
        self.vocab = int(vocab_size)
        if not 0 <= self.index < self.count:
            raise ValueError(f"run {index} of the table's {count}")
        self.norm = StreamRMSNorm(hidden_size, eps)
        self.table = self.w_gate = self.w_proj = None

    def tensor_specs(self):
        return {"table": matrix((self.vocab, self.count * self.dim)), "gate": matrix((self.dim, self.hidden)),
                "proj": matrix((self.hidden, self.dim)), "norm": ((self.hidden,), VECTOR, "ones")}

    def load(self, tensors):
        self.table, self.w_gate, self.w_proj = tensors["table"], tensors["gate"], tensors["proj"]
        self.norm.compute_dtype = self.compute_dtype
        self.norm.load({"weight": tensors["norm"]})

    def kernel_modules(self, dtype):
        return ("gemm", "activation", "norm")

    def flops(self, rows, spans):
        return 4.0 * rows * self.dim * self.hidden

    def forward(self, x: torch.Tensor, ctx: StepContext) -> Deferred:
        gate = linear(x, self.w_gate)
        g = torch.empty_like(gate)
        ops.token_gate(gate, ctx.tokens, self.table, self.index * self.dim, g)
        return Deferred(delta=linear(g, self.w_proj, allow_partials=True), norm=self.norm)


class PreNormBlock:
    """``x <- x + mixer(norm_a(x))``, then ``x <- x + ffn(norm_b(x))``, then (with a ``side``) ``x <- x + side(x)``.
    The stream is float32 from the first sum on; a sublayer's output is handed on unadded and enters the stream in
    the launch that norms it for the next reader. A mixer's output bias rides along as the vector of that sum."""

    roles = ("mixer_norm", "mixer", "ffn_norm", "ffn")

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None = None, ffn: FeedForward | None = None,
                 side: TokenSide | None = None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.side = mixer_norm, mixer, ffn_norm, ffn, side

    def parts(self):
        return {role: getattr(self, role) for role in self.roles}

    def forward(self, x, pending, ctx: StepContext, line, writes_cache: bool):
        # the embedding's output starts the stream and other parts may read it again: never updated in place
        x, h = self.mixer_norm.add_forward(x, pending, ctx.dtype, in_place=x is not ctx.embedded)
        delta, bias = self.mixer.forward_split(h, ctx, line, writes_cache)
        pending = Deferred(delta=delta, vector=bias)
        if self.ffn is not None:
            x, h = self.ffn_norm.add_forward(x, pending, ctx.dtype)
            pending = Deferred(delta=self.ffn.forward(h, ctx))
        if self.side is not None:
            x, h = read_plain(x, pending, ctx.dtype)
            pending = self.side.forward(h, ctx)
        return x, pending


class PreNormMixerBlock(PreNormBlock):
    roles = ("mixer_norm", "mixer")


class PreNormSideBlock(PreNormBlock):
    roles = ("mixer_norm", "mixer", "ffn_norm", "ffn", "side")


class PreNormMixerSideBlock(PreNormBlock):
    roles = ("mixer_norm", "mixer", "side")


class PassEntry(StreamPart):
    """``steps [passes, width]``: pass ``t`` begins by adding ``steps[t]`` to every row of the stream, and every pass
    but the first (when ``readd_embedding``) by adding the embedding's output of the row once more."""

    def __init__(self, passes: int, size: int, readd_embedding: bool = True):
        self.passes, self.size, self.readd = int(passes), int(size), bool(readd_embedding)
        self.steps: torch.Tensor | None = None

    def tensor_specs(self):
        return {"steps": ((self.passes, self.size), VECTOR, "normal")}

    def load(self, tensors):
        self.steps = tensors["steps"].float().contiguous()

    def kernel_modules(self, dtype):
        return ("norm",)

    def reads_whole(self) -> bool:
        return False

    def enter(self, pending, index: int, ctx: StepContext) -> Deferred:
        if not 0 <= index < self.passes:
            raise ValueError(f"pass {index} of {self.passes}")
        pending = as_deferred(pending)
        if pending.rows is not None or pending.vector is not None:
            raise ValueError("two entries before one run")
        rows = ctx.embedded if self.readd and index > 0 else None
        return Deferred(pending.delta, pending.norm, rows, self.steps[index])


register_part("stream_rmsnorm", StreamRMSNorm)
register_part("stream_layernorm", StreamLayerNorm)
register_part("pass_entry", PassEntry)
register_part("token_side", TokenSide)
register_block("pre_norm", PreNormBlock)
register_block("pre_norm_mixer", PreNormMixerBlock)
register_block("pre_norm_side", PreNormSideBlock)
register_block("pre_norm_mixer_side", PreNormMixerSideBlock)
register_block("sandwich", SandwichBlock)
register_block("sandwich_mixer", SandwichMixerBlock)
register_block("post_norm", PostNormBlock)
register_block("post_norm_mixer", PostNormMixerBlock)
