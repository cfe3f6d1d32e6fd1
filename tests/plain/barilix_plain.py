"""A plain, slow Barilix: one function per mechanism, written from the design's equations.

Everything is computed token by token (or with a dense score matrix) in the dtype of the tensors it is handed,
float64 in the tests. Nothing here is shared with the library: no kernel, no part, no cache. A mixer's function
takes the inputs of one sequence ``[T, width]`` and, optionally, the state an earlier portion left, and returns
its outputs and the state after the last token.

Notation. ``rms(x) = x / sqrt(mean(x^2) + eps)``. Linear weights are ``[out, in]``. ``w`` is a dictionary of one
part's tensors by their short names (``"q"``, ``"q.conv"``, ``"left.o.b"``, ...), ``c`` the part's entry of the
configuration.
"""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, weight, eps):
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ------------------------------------------------------------------------------------------ short convolution
def short_conv(u, kernel, history=None, bias=None):
    """``u [T, C]``, ``kernel [C, taps]`` whose last column meets the current token. ``history [taps - 1, C]`` are the
    inputs before ``u`` (zeros at a sequence's start). Returns the outputs and the history after ``u``."""
    taps = kernel.shape[1]
    if history is None:
        history = u.new_zeros(taps - 1, u.shape[1])
    full = torch.cat([history, u], 0)
    T = u.shape[0]
    y = u.new_zeros(u.shape)
    for j in range(taps):
        y = y + full[j:j + T] * kernel[:, j]
    if bias is not None:
        y = y + bias
    return y, full[full.shape[0] - (taps - 1):]


# ------------------------------------------------------------------------------------------ rotation
def scaled_frequencies(dims, base, scaling, dtype=torch.float64):
    """``f_i = base^(-2i/dims)``; with ``scaling`` long wavelengths are stretched by ``factor``, short ones kept,
    and those between blended by where ``original / wavelength`` lies between ``low`` and ``high``."""
    f = base ** (-2 * torch.arange(dims // 2, dtype=dtype) / dims)
    if not scaling:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = []
    for fi in f.tolist():
        wave = 2 * math.pi / fi
        if wave < original / high:
            out.append(fi)
        elif wave > original / low:
            out.append(fi / factor)
        else:
            s = (original / wave - low) / (high - low)
            out.append((1 - s) * fi / factor + s * fi)
    return torch.tensor(out, dtype=dtype)


def rotate_half(x, pos, dims, f):
    """``x [T, heads, D]``: entry ``i`` of the first ``dims`` turns with entry ``i + dims/2`` by ``pos * f_i``."""
    if not dims:
        return x
    half = dims // 2
    a = (pos.to(x.dtype)[:, None] * f.to(x.dtype)[None, :])[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * a.cos() - v * a.sin(), v * a.cos() + u * a.sin(), x[..., dims:]], -1)


# ------------------------------------------------------------------------------------------ windowed attention
def conv_attention(h, w, c, eps, past=None):
    """Projections with biases, a short convolution on each of q, k, v, a norm per head on q and k, a partial
    rotation, softmax over the last ``mask.size`` keys. ``past``: ``(keys, values, conv histories of q, k, v)``."""
    T, H, G, D, Dv = h.shape[0], c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    keys, values, hist = (None, None, {n: None for n in "qkv"}) if past is None else past
    start = 0 if keys is None else keys.shape[0]
    pos = torch.arange(start, start + T)
    proj, new_hist = {}, {}
    for n in "qkv":
        u = h @ w[n].T + w[n + ".b"]
        proj[n], new_hist[n] = short_conv(u, w[n + ".conv"], hist[n])
    q = rms(proj["q"].view(T, H, D), eps) * w["q.norm"]
    k = rms(proj["k"].view(T, G, D), eps) * w["k.norm"]
    v = proj["v"].view(T, G, Dv)
    rot = c.get("rot")
    if rot and rot["dims"]:
        f = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_half(q, pos, rot["dims"], f), rotate_half(k, pos, rot["dims"], f)
    keys = k if keys is None else torch.cat([keys, k], 0)
    values = v if values is None else torch.cat([values, v], 0)
    window = c["mask"]["size"] if c.get("mask") else None
    out = h.new_zeros(T, H, Dv)
    for t in range(T):
        i = start + t
        lo = 0 if window is None else max(0, i - window + 1)
        for a in range(H):
            g = a // (H // G)
            s = (keys[lo:i + 1, g] @ q[t, a]) * c["scale"]
            p = torch.softmax(s, 0)
            out[t, a] = p @ values[lo:i + 1, g]
    y = out.reshape(T, H * Dv) @ w["o"].T + w["o.b"]
    return y, (keys, values, new_hist)


# ------------------------------------------------------------------------------------------ state-space mixer
def state_space(h, w, c, eps, past=None):
    """``[z | x | B | C | dt] = W_in h``; x, B, C through one convolution with bias and silu; per head
    ``S <- exp(-exp(A_log) dt) S + dt B x^T``, ``y = S^T C + D x``; gate, norm in equal parts, projection.
    ``past``: ``(S [heads, N, vdim], conv history)``."""
    T, H, P, N, G = h.shape[0], c["heads"], c["vdim"], c["state"], c["groups"]
    inner = H * P
    S, hist = (h.new_zeros(H, N, P), None) if past is None else (past[0].clone(), past[1])
    u = h @ w["in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc, hist = short_conv(xbc, w["conv"], hist, w["conv.b"])
    xbc = silu(xbc)
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w["dt_bias"])
    rate = torch.exp(w["A_log"])
    ys = []
    for t in range(T):
        y = h.new_zeros(H, P)
        for a in range(H):
            g = a // (H // G)
            S[a] = torch.exp(-rate[a] * dt[t, a]) * S[a] + dt[t, a] * torch.outer(B[t, g], x[t, a])
            y[a] = S[a].T @ C[t, g] + w["D"][a] * x[t, a]
        ys.append(y.reshape(inner))
    y = torch.stack(ys) * silu(z)
    parts = c["norm_groups"]
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T, (S, hist)


def parallel_mixer(h, w, c, eps, past=None):
    """Both mixers read ``h``; each output is rms-normed over the width with its weight; half their sum."""
    sub = lambda side: {k[len(side) + 1:]: v for k, v in w.items() if k.startswith(side + ".")}
    past = (None, None) if past is None else past
    left, pl = conv_attention(h, sub("left"), c["left"], eps, past[0])
    right, pr = state_space(h, sub("right"), c["right"], eps, past[1])
    return 0.5 * (rms(left, eps) * w["left.out"] + rms(right, eps) * w["right.out"]), (pl, pr)


# ------------------------------------------------------------------------------------------ gated delta rule
def delta_mixer(h, w, c, eps, past=None):
    """q, k (``kv_heads`` of them) and v through convolution and silu; q, k made unit vectors; per head
    ``S <- g S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``. ``past``: ``(S, histories)``."""
    T, H, G, D, P = h.shape[0], c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    S, hist = (h.new_zeros(H, D, P), {n: None for n in "qkv"}) if past is None else (past[0].clone(), past[1])
    proj, new_hist = {}, {}
    for n in "qkv":
        y, new_hist[n] = short_conv(h @ w[n].T, w[n + ".conv"], hist[n])
        proj[n] = silu(y)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q = unit(proj["q"].view(T, G, D)) * D ** -0.5
    k = unit(proj["k"].view(T, G, D))
    v = proj["v"].view(T, H, P)
    beta = torch.sigmoid(h @ w["b"].T)
    decay = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    gate = silu(h @ w["g"].T).view(T, H, P)
    out = h.new_zeros(T, H, P)
    for t in range(T):
        for a in range(H):
            g = a // (H // G)
            S[a] = decay[t, a] * S[a]
            u = beta[t, a] * (v[t, a] - S[a].T @ k[t, g])
            S[a] = S[a] + torch.outer(k[t, g], u)
            out[t, a] = S[a].T @ q[t, g]
    o = rms(out, eps) * w["norm"] * gate
    return o.reshape(T, H * P) @ w["o"].T, (S, new_hist)


# ------------------------------------------------------------------------------------------ feed-forwards
def gated_unit(h, w, prefix=""):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def table_experts(h, tokens, w, c):
    """Each token id's row of the table names its experts, all with weight ``1 / top``; a shared expert is added."""
    top = c["router"]["top"]
    out = h.new_zeros(h.shape)
    for t in range(h.shape[0]):
        for e in w["table"][int(tokens[t])].tolist():
            out[t] += gated_unit(h[t:t + 1], w, f"e{e}.")[0] / top
    if c.get("shared"):
        out = out + gated_unit(h, w, "shared.")
    return out


def feed_forward(h, tokens, w, c):
    return gated_unit(h, w) if c["kind"] == "dense" else table_experts(h, tokens, w, c)


# ------------------------------------------------------------------------------------------ the model
MIXERS = {"parallel": parallel_mixer, "delta": delta_mixer}


def part_tensors(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, past=None, taps=None):
    """One sequence's next ``tokens`` after whatever ``past`` holds (a list with one entry per layer, or None).
    Returns ``(logits [T, vocab], past)``; ``taps``, a list, receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = tensors["embed"][tokens] * cfg["embedding"]["scale"]
    past = [None] * len(cfg["layers"]) if past is None else list(past)
    for i, layer in enumerate(cfg["layers"]):
        y, past[i] = MIXERS[layer["type"]](x, part_tensors(tensors, f"l{i}.mix."), layer["mixer"], eps, past[i])
        x = x + layer_norm(y, tensors[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            y = feed_forward(x, tokens, part_tensors(tensors, f"l{i}.mlp."), layer["mlp"])
            x = x + layer_norm(y, tensors[f"l{i}.norm2"], eps)
        if taps is not None:
            taps.append(x.clone())
    return layer_norm(x, tensors["final.norm"], eps) @ tensors["head"].T, past
