"""Small Podenex configurations with weights of the tests' own making.

The weights are drawn here, not by the library: matrices ``N(0, 1 / in)`` so that activations stay of order one, norm
weights around one, convolution taps that keep a channel's size, bias tables of order one, blends of values between 0.2 and 0.8,
everything rounded to bfloat16 so that both precisions read the same numbers.
"""

from __future__ import annotations

import copy
import json
import os

import torch
from safetensors.torch import save_file


def chunked(heads, kv_heads, dim, vdim, conv=None, chunk=None, bias=None, v_mix=False, scale=None):
    """``bias = (rows of the table, distance at which it reaches its last row)``."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if conv:
        m["conv"] = conv
    if chunk:
        m["mask"] = {"size": chunk}
    if bias:
        m["bias_rows"], m["bias_max"] = bias
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def sinked(heads, kv_heads, dim, vdim, window=None, v_mix=False, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention_2", "mixer": m}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window=None, rot_dims=None, base=10000.0, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    return {"type": "latent_attention", "mixer": m}


def moe(experts, top, ff, groups=None, shared=None):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": groups[0], "keep": groups[1]} if groups else None},
            "shared": {"ff": shared} if shared else None}


def with_mlp(layer, mlp=None):
    layer = dict(layer)
    layer["mlp"] = mlp
    return layer


def config(width, vocab, layers, eps=1e-5, side=None):
    out = {"architecture": "Podenex", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [l if "mlp" in l else with_mlp(l) for l in layers]}
    if side:
        out["token_side"] = {"dim": side}
    return out


# A: all three mixers; heads of 32 with equal keys and values (the matrix cores' sizes) under a window shorter than a
# page; values wider than keys; a chunk shorter than a page with a bias table that saturates inside it; a window of a
# page and one token; a rotation over part of the rotated width; groups of experts; a layer without a feed-forward.
CASE_A = config(64, 200, [
    with_mlp(sinked(4, 2, 32, 32, window=20, v_mix=True), moe(8, 2, 32, groups=(4, 2), shared=40)),
    with_mlp(latent(2, 16, 16, 16, 24, 20, window=70, rot_dims=16, base=100.0), moe(6, 3, 24)),
    chunked(4, 2, 16, 32, conv=3, chunk=24, bias=(12, 18), v_mix=True),
    with_mlp(sinked(2, 1, 24, 64, window=65, v_mix=True), moe(8, 2, 32, groups=(2, 1), shared=16)),
    with_mlp(latent(3, 8, 16, 24, 16, 12, rot_dims=8), moe(4, 1, 16, shared=24))], side=8)
# B: sizes that are no multiples of 8; the first layer that shares values is a chunked one with a convolution of one
# tap (no history at all); no window, no chunk, no bias table, no token side; every expert chosen, and one expert.
CASE_B = config(72, 131, [
    with_mlp(chunked(3, 3, 20, 12, conv=1, v_mix=True), moe(4, 4, 20, groups=(2, 2))),
    with_mlp(sinked(6, 3, 10, 12, v_mix=True), moe(1, 1, 12, shared=20)),
    with_mlp(latent(3, 12, 6, 20, 10, 14, rot_dims=6, base=50.0), moe(5, 2, 12))], eps=1e-6)
# C: chunks of exactly a page and of a page and one token; a window of one token; a bias table whose logarithmic half
# has exact borders (distances 16, 32, 64 with 16 rows reaching 128); many experts in groups of which one is kept;
# layers that do not share values between layers that do; the rotated part wider than the plain one.
CASE_C = config(96, 300, [
    with_mlp(chunked(4, 2, 32, 32, conv=4, chunk=64, bias=(16, 128)), moe(16, 4, 16, groups=(4, 1), shared=24)),
    with_mlp(chunked(2, 1, 16, 48, conv=2, chunk=65, bias=(6, 200), v_mix=True), moe(16, 4, 16, groups=(4, 2))),
    sinked(8, 2, 16, 16, window=1),
    with_mlp(latent(4, 16, 48, 32, 40, 24, window=64, rot_dims=48, base=1e4), moe(3, 2, 40, shared=8)),
    with_mlp(sinked(3, 3, 32, 16, window=130, v_mix=True), moe(16, 2, 8, groups=(8, 3)))], side=16)
CASES = {"A": CASE_A, "B": CASE_B, "C": CASE_C}


def tensors_for(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """Every tensor the configuration names, as bfloat16-exact float32."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    out: dict[str, torch.Tensor] = {}

    def mat(name, o, i, gain=1.0):
        out[name] = gain * torch.randn(o, i, generator=g) / i ** 0.5

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * torch.randn(n, generator=g)

    def unit(p, ff):
        mat(p + "up", ff, W, 1.5); mat(p + "down", W, ff)

    out["embed"] = torch.randn(V, W, generator=g)
    mat("head", V, W, 2.0)
    vec("final.norm", W, 1.0)
    side = cfg.get("token_side")
    if side:
        out["side.embed"] = torch.randn(V, len(cfg["layers"]) * side["dim"], generator=g)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        vec(p + "norm1", W, 1.0)
        if layer["type"] == "latent_attention":
            H, D, R, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            mat(p + "mix.dq", m["q_rank"], W, 2.0); vec(p + "mix.dq.norm", m["q_rank"], 1.0, 0.3)
            mat(p + "mix.uq", H * (D + R), m["q_rank"], 1.4)
            mat(p + "mix.dkv", m["kv_rank"] + R, W, 2.0); vec(p + "mix.dkv.norm", m["kv_rank"], 1.0, 0.3)
            mat(p + "mix.uk", H * D, m["kv_rank"], 1.4); mat(p + "mix.uv", H * Dv, m["kv_rank"], 2.0)
            mat(p + "mix.g", H * Dv, W, 2.0); mat(p + "mix.o", W, H * Dv)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, width in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                mat(p + "mix." + n, width, W, 2.0 if n == "v" else 1.4)
                if layer["type"] == "attention_2":
                    vec(p + f"mix.{n}.b", width, 0.0, 0.5)
                elif m.get("conv"):
                    taps = m["conv"]
                    out[p + f"mix.{n}.conv"] = torch.randn(width, taps, generator=g) / taps ** 0.5 + (0.5 if taps == 1 else 0.0)
            mat(p + "mix.o", W, H * Dv)
            if layer["type"] == "attention_2":
                vec(p + "mix.q.norm", D, 1.0, 0.3); vec(p + "mix.k.norm", D, 1.0, 0.3); vec(p + "mix.o.b", W, 0.0, 0.3)
            else:
                mat(p + "mix.g", H, W, 2.0)
                if m.get("bias_max"):
                    out[p + "mix.rel"] = torch.randn(m["bias_rows"], H, generator=g)
            if m.get("v_mix"):
                out[p + "mix.vmix"] = 0.2 + 0.6 * torch.rand((), generator=g)
        mlp = layer["mlp"]
        if mlp is not None:
            vec(p + "norm2", W, 1.0)
            mat(p + "mlp.router", mlp["router"]["experts"], W, 3.0)
            for e in range(mlp["router"]["experts"]):
                unit(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp["shared"]:
                unit(p + "mlp.shared.", mlp["shared"]["ff"])
        if side:
            mat(p + "side.gate", side["dim"], W, 2.0); mat(p + "side.proj", W, side["dim"]); vec(p + "side.norm", W, 0.5, 0.2)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in out.items()}


def write_dir(path: str, cfg: dict, tensors: dict[str, torch.Tensor]) -> str:
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def double(tensors):
    return {k: v.double() for k, v in tensors.items()}


def variant(cfg: dict, **changes) -> dict:
    out = copy.deepcopy(cfg)
    out.update(changes)
    return out


def random_config(rng) -> dict:
    """A configuration drawn with ``rng`` (a ``random.Random``): sizes, head counts, the order of layers, which of them
    share values, where feed-forwards sit, windows, chunks, taps, tables, rotations, groups and the token side all vary."""
    width = rng.choice([64, 96, 128, 160, 192, 256])
    mix_width = rng.choice([16, 24, 48, 64])          # kv_heads * vdim of the layers that share values
    layers = []
    for _ in range(rng.randrange(2, 6)):
        kind = rng.choice(["attention", "attention_2", "latent_attention"])
        if kind == "latent_attention":
            dim, rot_dim = rng.choice([8, 16, 32, 40]), rng.choice([8, 16, 24, 64])
            layer = latent(rng.choice([1, 2, 3, 6]), dim, rot_dim, rng.choice([8, 16, 32, 72]), rng.choice([16, 40, 96]),
                           rng.choice([12, 32, 64]), window=rng.choice([None, 1, 17, 63, 64, 65, 128, 1000]),
                           rot_dims=rng.choice([None, 2, rot_dim // 2 // 2 * 2, rot_dim]), base=rng.choice([100.0, 1e4, 5e5]),
                           scale=rng.choice([None, 0.3, 0.05]))
        else:
            v_mix = rng.random() < 0.6
            kv = rng.choice([1, 2]) if v_mix else rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 32, 48, 64])
            vdim = mix_width // kv if v_mix else rng.choice([dim, dim, 8, 40])
            heads, size = kv * rng.choice([1, 2, 4]), rng.choice([None, 1, 2, 17, 63, 64, 65, 128, 1000])
            if kind == "attention":
                rows = rng.choice([2, 6, 16, 32])
                layer = chunked(heads, kv, dim, vdim, conv=rng.choice([None, 1, 2, 3, 4, 5]), chunk=size,
                                bias=rng.choice([None, (rows, rows // 2 + rng.choice([1, 7, 120, 512]))]), v_mix=v_mix,
                                scale=rng.choice([None, 0.3, 0.05]))
            else:
                layer = sinked(heads, kv, dim, vdim, window=size, v_mix=v_mix, scale=rng.choice([None, 0.3, 0.05]))
        mlp = None
        if rng.random() < 0.75:
            count = rng.choice([1, 2, 4])
            experts = count * rng.choice([1, 2, 3, 4])
            keep = rng.randrange(1, count + 1)
            top = rng.randrange(1, min(keep * (experts // count), 5) + 1)
            mlp = moe(experts, top, rng.choice([8, 24, 64, 100]), groups=rng.choice([None, (count, keep)]),
                      shared=rng.choice([None, 16, 72]))
            if mlp["router"]["groups"] is None:
                mlp["router"]["top"] = rng.randrange(1, min(experts, 5) + 1)
        layers.append(with_mlp(layer, mlp))
    return config(width, rng.randrange(100, 600), layers, eps=rng.choice([1e-6, 1e-5]), side=rng.choice([None, 4, 16]))
