"""A plain, slow Podenex: one function per mechanism, written from the design's equations.

Everything is computed with dense score matrices in the dtype of the tensors it is handed (float64 in the tests).
Nothing here is shared with the library: no kernel, no part, no cache. A mixer's function takes the inputs of one
sequence ``[T, width]`` and, optionally, what an earlier portion of the same sequence left (``past``), and returns its
outputs and what it leaves for the next portion.

Notation. ``rms(x) = x / sqrt(mean(x^2) + eps)``. Linear weights are ``[out, in]``. ``w`` is a dictionary of one
part's tensors by their short names (``"q"``, ``"q.conv"``, ``"o.b"``, ...), ``c`` the part's entry of the
configuration. Positions count from 0 in every sequence; a portion's first position is the length of its past.
"""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, weight, eps):
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------------------------ short convolution
def short_conv(u, kernel, history=None):
    """``u [T, C]``, ``kernel [C, taps]`` whose last column meets the current token; ``history [taps - 1, C]`` are the
    inputs before ``u`` (zeros at a sequence's start). Returns the outputs and the history after ``u``."""
    taps = kernel.shape[1]
    if history is None:
        history = u.new_zeros(taps - 1, u.shape[1])
    full = torch.cat([history, u], 0)
    T = u.shape[0]
    y = u.new_zeros(u.shape)
    for j in range(taps):
        y = y + full[j:j + T] * kernel[:, j]
    return y, full[full.shape[0] - (taps - 1):]


# ------------------------------------------------------------------------------------------ who sees whom
def window_mask(pos_q, pos_k, size):
    """Row i sees key j when ``0 <= i - j < size`` (every earlier key without a size)."""
    d = pos_q[:, None] - pos_k[None, :]
    return (d >= 0) & (d < size) if size else d >= 0


def chunk_mask(pos_q, pos_k, size):
    """Row i sees key j <= i of its own chunk: ``i // size == j // size``, chunks counted from position 0."""
    d = pos_q[:, None] - pos_k[None, :]
    return (d >= 0) & ((pos_q[:, None] // size) == (pos_k[None, :] // size))


# ------------------------------------------------------------------------------------------ distance bias
def distance_bucket(n: int, rows: int, far: int) -> int:
    """Distances below half the table have a row each; the rest share the other half on a logarithmic scale that
    reaches the last row at distance ``far``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def distance_bias(table, pos_q, pos_k, far):
    """``table [rows, heads]`` -> ``[heads, Tq, Tk]``; entries for keys ahead of the row are never looked at."""
    rows = table.shape[0]
    d = (pos_q[:, None] - pos_k[None, :]).clamp(min=0)
    idx = torch.tensor([[distance_bucket(int(n), rows, far) for n in row] for row in d.tolist()], dtype=torch.long)
    return table[idx].permute(2, 0, 1)


# ------------------------------------------------------------------------------------------ softmax, with a sink or not
def weigh(scores, mask, values, group, sink=False):
    """``scores [H, Tq, Tk]``, ``values [Tk, G, Dv]`` -> ``[Tq, H, Dv]``. With ``sink`` a key of score 0 that has no
    value joins the denominator: ``p_j = exp(s_j) / (1 + sum exp(s_j))``."""
    s = scores.masked_fill(~mask[None], -math.inf)
    m = s.amax(-1, keepdim=True)
    if sink:
        m = m.clamp(min=0.0)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink:
        den = den + torch.exp(-m)
    p = e / den
    v = values.repeat_interleave(group, dim=1)                     # query head h reads kv head h // group
    return torch.einsum("hqk,khd->qhd", p, v)


def mix_values(v, lam, v_first):
    """Values of a later layer lean on those the first such layer computed for the same token (a token's values
    taken as one vector over all its key/value heads)."""
    return (1 - lam) * v + lam * v_first.reshape(v.shape)


# ------------------------------------------------------------------------------------------ mixer 'attention'
def chunked_attention(h, w, c, past=None, v_first=None, first=False):
    """Short convolutions on q, k and v; no rotation; a learned bias by distance; chunks; a gate per head.
    Returns ``(output, past, values)``."""
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    T = h.shape[0]
    past = past or {}
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    hist = {}
    if c.get("conv"):
        q, hist["q"] = short_conv(q, w["q.conv"], past.get("hq"))
        k, hist["k"] = short_conv(k, w["k.conv"], past.get("hk"))
        v, hist["v"] = short_conv(v, w["v.conv"], past.get("hv"))
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, Dv)
    if c.get("v_mix") and not first:
        v = mix_values(v, w["vmix"], v_first)
    start = past["k"].shape[0] if "k" in past else 0
    if start:
        k, v_all = torch.cat([past["k"], k]), torch.cat([past["v"], v])
    else:
        v_all = v
    pos_q, pos_k = torch.arange(start, start + T), torch.arange(0, start + T)
    s = torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(H // G, dim=1)) * c["scale"]
    if "rel" in w:
        s = s + distance_bias(w["rel"], pos_q, pos_k, c["bias_max"])
    mask = chunk_mask(pos_q, pos_k, c["mask"]["size"]) if c.get("mask") else window_mask(pos_q, pos_k, None)
    o = weigh(s, mask, v_all, H // G)
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    out = o.reshape(T, H * Dv) @ w["o"].T
    return out, {"k": k, "v": v_all, "hq": hist.get("q"), "hk": hist.get("k"), "hv": hist.get("v")}, v


# ------------------------------------------------------------------------------------------ mixer 'attention_2'
def sink_attention(h, w, c, eps, past=None, v_first=None, first=False):
    """Biases on all four projections; a norm per head on q and k with one weight for all heads; no positions in
    the scores; a sliding window; a sink of score 0 in the denominator. Returns ``(output, past, values)``."""
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    T = h.shape[0]
    past = past or {}
    q = (h @ w["q"].T + w["q.b"]).view(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, D)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, Dv)
    q, k = rms(q, eps) * w["q.norm"], rms(k, eps) * w["k.norm"]
    if c.get("v_mix") and not first:
        v = mix_values(v, w["vmix"], v_first)
    start = past["k"].shape[0] if "k" in past else 0
    if start:
        k, v_all = torch.cat([past["k"], k]), torch.cat([past["v"], v])
    else:
        v_all = v
    pos_q, pos_k = torch.arange(start, start + T), torch.arange(0, start + T)
    s = torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(H // G, dim=1)) * c["scale"]
    mask = window_mask(pos_q, pos_k, c["mask"]["size"] if c.get("mask") else None)
    o = weigh(s, mask, v_all, H // G, sink=True)
    out = o.reshape(T, H * Dv) @ w["o"].T + w["o.b"]
    return out, {"k": k, "v": v_all}, v


# ------------------------------------------------------------------------------------------ rotation
def rotate_pairs(x, pos, dims, base):
    """``x [T, heads, D]``: entries ``2i`` and ``2i + 1`` of the first ``dims`` turn by ``pos * base^(-2i/dims)``."""
    if not dims:
        return x
    f = base ** (-2 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    a = (pos.to(torch.float64)[:, None] * f[None, :]).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a)], dim=-1)
    return torch.cat([turned.flatten(-2), x[..., dims:]], dim=-1)


# ------------------------------------------------------------------------------------------ mixer 'latent_attention'
def latent_attention(h, w, c, eps, past=None):
    """Queries and keys/values through normed latents; one rotated key part for all heads; a sliding window; the
    heads' outputs gated element by element. Keeps the latent and the rotated key part. Returns ``(output, past)``."""
    H, D, R, Dv, rank = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    T = h.shape[0]
    past = past or {}
    start = past["c"].shape[0] if "c" in past else 0
    pos_q = torch.arange(start, start + T)
    rot = c.get("rot") or {"dims": 0, "base": 1.0}
    q = ((rms(h @ w["dq"].T, eps) * w["dq.norm"]) @ w["uq"].T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], pos_q, rot["dims"], rot["base"])
    down = h @ w["dkv"].T
    lat = rms(down[:, :rank], eps) * w["dkv.norm"]
    k_rot = rotate_pairs(down[:, None, rank:], pos_q, rot["dims"], rot["base"])[:, 0]
    if start:
        lat, k_rot = torch.cat([past["c"], lat]), torch.cat([past["r"], k_rot])
    pos_k = torch.arange(0, start + T)
    k_plain = (lat @ w["uk"].T).view(-1, H, D)
    v = (lat @ w["uv"].T).view(-1, H, Dv)
    s = (torch.einsum("qhd,khd->hqk", q_plain, k_plain) + torch.einsum("qhd,kd->hqk", q_rot, k_rot)) * c["scale"]
    mask = window_mask(pos_q, pos_k, c["mask"]["size"] if c.get("mask") else None)
    o = weigh(s, mask, v, 1).reshape(T, H * Dv)
    o = o * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T, {"c": lat, "r": k_rot}


# ------------------------------------------------------------------------------------------ feed-forward
def squared_relu_unit(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def route(z, top, groups=None):
    """``z [T, E]`` -> ``(chosen [T, top], weights [T, top])``: softmax over all experts; a group of neighbours scores
    as its best expert, and only the best ``keep`` groups stay in; the weights are the scores as they are."""
    s = torch.softmax(z, dim=-1)
    pick = s.clone()
    E = z.shape[1]
    if groups and groups["keep"] < groups["count"]:
        size = E // groups["count"]
        best = s.view(-1, groups["count"], size).amax(-1)
        order = torch.sort(best, dim=-1, descending=True, stable=True).indices[:, :groups["keep"]]
        keep = torch.zeros_like(best, dtype=torch.bool).scatter_(1, order, True)
        pick = pick.masked_fill(~keep.repeat_interleave(size, dim=1), -1.0)
    chosen = torch.sort(pick, dim=-1, descending=True, stable=True).indices[:, :top]
    return chosen, s.gather(1, chosen)


def routed_experts(h, w, c):
    r = c["router"]
    chosen, weights = route((h @ w["router"].T).float().to(h.dtype), r["top"], r.get("groups"))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weights[t]):
            out[t] = out[t] + g * squared_relu_unit(h[t], w[f"e{e}.up"], w[f"e{e}.down"])
    if c.get("shared"):
        out = out + squared_relu_unit(h, w["shared.up"], w["shared.down"])
    return out


# ------------------------------------------------------------------------------------------ what a token brings to every layer
def token_side(x, tokens, table, w, layer, dim, eps):
    """The stream's own gate on a few numbers the token id brings for this layer, projected up and rms-normed."""
    e = table[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return rms(y, eps) * w["norm"]


# ------------------------------------------------------------------------------------------ the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, past=None):
    """One sequence's next ``tokens`` (a list) after ``past``. Returns ``(logits [T, vocab], the stream after every
    layer [layers, T, width], past)``."""
    eps = cfg["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    x = tensors["embed"][tok]
    past = past or [None] * len(cfg["layers"])
    new_past, after = [], []
    v_first, seen_mix = None, False
    side = cfg.get("token_side")
    for i, layer in enumerate(cfg["layers"]):
        p, c = f"l{i}.", layer["mixer"]
        w = sub(tensors, p + "mix.")
        h = layer_norm(x, tensors[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            y, state = latent_attention(h, w, c, eps, past[i])
        else:
            first = bool(c.get("v_mix")) and not seen_mix
            if layer["type"] == "attention":
                y, state, v = chunked_attention(h, w, c, past[i], v_first, first)
            else:
                y, state, v = sink_attention(h, w, c, eps, past[i], v_first, first)
            if first:
                v_first, seen_mix = v, True
        new_past.append(state)
        x = x + y
        if layer.get("mlp"):
            x = x + routed_experts(layer_norm(x, tensors[p + "norm2"], eps), sub(tensors, p + "mlp."), layer["mlp"])
        if side:
            x = x + token_side(x, tok, tensors["side.embed"], sub(tensors, p + "side."), i, side["dim"], eps)
        after.append(x)
    logits = layer_norm(x, tensors["final.norm"], eps) @ tensors["head"].T
    return logits, torch.stack(after), new_past
