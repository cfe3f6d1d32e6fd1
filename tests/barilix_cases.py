"""Small Barilix configurations with weights of the tests' own making.

The weights are drawn here, not by the library: matrices ``N(0, 1 / in)`` so that activations stay of order one, norm
weights around one, convolution taps of order one, decays spread between fast and slow, expert tables whose rows hold
different experts, everything rounded to bfloat16 so that both precisions read the same numbers.
"""

from __future__ import annotations

import copy
import json
import os

import torch
from safetensors.torch import save_file


def attention(heads, kv_heads, dim, vdim, conv, window=None, rot_dims=None, base=10000.0, scaling=None, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
            "mask": {"size": window} if window else None,
            "rot": {"dims": rot_dims, "base": base, "scaling": scaling} if rot_dims else None,
            "scale": scale if scale is not None else dim ** -0.5}


def state_space(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def parallel(left, right):
    return {"type": "parallel", "mixer": {"left": left, "right": right}}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared} if shared else None}


def with_mlp(layer, mlp=None):
    layer = dict(layer)
    layer["mlp"] = mlp
    return layer


def config(width, vocab, layers, eps=1e-5, scale=1.0):
    return {"architecture": "Barilix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": [l if "mlp" in l else with_mlp(l) for l in layers]}


STRETCH = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
# A: both kinds of layer; attention heads of 32 (the matrix cores' sizes) with a window shorter than a page, and heads
# whose values are wider than their keys with a window longer than one; frequencies of all three kinds (kept, stretched,
# blended); experts with and without a shared one; a layer without a feed-forward.
CASE_A = config(64, 200, [
    with_mlp(delta(4, 2, 16, 24, 3), dense(96)),
    with_mlp(parallel(attention(4, 2, 32, 32, 2, window=20, rot_dims=8, base=100.0, scaling=STRETCH),
                      state_space(4, 16, 24, 2, 4, 2)), moe(8, 3, 32, shared=40)),
    delta(2, 2, 8, 8, 4),
    with_mlp(parallel(attention(2, 1, 16, 24, 4, window=70, rot_dims=16), state_space(3, 8, 16, 1, 2, 1)), moe(6, 2, 24))],
    scale=3.0)
# B: sizes that are no multiples of 8; convolutions of one tap (no history at all); no window, no rotation; one expert
# chosen, and all of them; a state-space head wider than a run of value columns, with a state of 100 rows.
CASE_B = config(72, 131, [
    with_mlp(parallel(attention(3, 3, 20, 12, 1), state_space(2, 40, 8, 2, 1, 4)), dense(80)),
    with_mlp(delta(3, 1, 24, 40, 1), moe(5, 1, 20, shared=16)),
    with_mlp(parallel(attention(2, 2, 64, 64, 4, window=64, rot_dims=32, base=500.0,
                                scaling={"factor": 2.0, "low": 2.0, "high": 16.0, "original": 256}),
                      state_space(1, 72, 100, 1, 3, 1)), moe(4, 4, 12))], eps=1e-6, scale=0.7)
# C: delta-rule keys of 128 and values of 64; many small heads; a window of one page and one token, and a window of one
# token; a norm in as many parts as there are heads; many experts.
CASE_C = config(96, 300, [
    with_mlp(delta(6, 3, 128, 64, 4), moe(16, 4, 16, shared=24)),
    parallel(attention(8, 2, 16, 16, 3, window=65, rot_dims=16, base=1e4), state_space(8, 8, 64, 4, 4, 8)),
    with_mlp(parallel(attention(1, 1, 32, 32, 2, window=1, rot_dims=2), state_space(2, 32, 32, 2, 2, 2)), dense(48)),
    with_mlp(delta(1, 1, 40, 136, 2), dense(64))], scale=9.0)
CASES = {"A": CASE_A, "B": CASE_B, "C": CASE_C}


def tensors_for(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """Every tensor the configuration names, as bfloat16-exact float32 (the experts' tables as int32)."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    out: dict[str, torch.Tensor] = {}
    tables: dict[str, torch.Tensor] = {}

    def mat(name, o, i, gain=1.0):
        out[name] = gain * torch.randn(o, i, generator=g) / i ** 0.5

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * torch.randn(n, generator=g)

    def glu(p, ff):
        mat(p + "gate", ff, W, 1.5); mat(p + "up", ff, W, 1.5); mat(p + "down", W, ff)

    def taps(name, channels, n):
        out[name] = torch.randn(channels, n, generator=g) * (0.8 if n > 1 else 1.0) + (0.5 if n == 1 else 0.0)

    out["embed"] = torch.randn(V, W, generator=g) / cfg["embedding"]["scale"]
    mat("head", V, W, 2.0)
    vec("final.norm", W, 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        vec(p + "norm1", W, 1.0)
        if layer["type"] == "delta":
            H, G, D, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, width in (("q", G * D), ("k", G * D), ("v", H * P)):
                mat(p + "mix." + n, width, W, 2.0)
                taps(p + f"mix.{n}.conv", width, m["conv"])
            mat(p + "mix.g", H * P, W); mat(p + "mix.a", H, W); mat(p + "mix.b", H, W, 2.0)
            vec(p + "mix.dt_bias", H, -1.0, 1.0); vec(p + "mix.A_log", H, -0.5, 1.0)
            vec(p + "mix.norm", P, 1.0); mat(p + "mix.o", W, H * P)
        else:
            a, r = m["left"], m["right"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for n, width in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                mat(p + "mix.left." + n, width, W, 2.0)
                vec(p + f"mix.left.{n}.b", width, 0.0, 0.5)
                taps(p + f"mix.left.{n}.conv", width, a["conv"])
            vec(p + "mix.left.q.norm", D, 1.0, 0.3); vec(p + "mix.left.k.norm", D, 1.0, 0.3)
            mat(p + "mix.left.o", W, H * Dv); vec(p + "mix.left.o.b", W, 0.0, 0.3)
            inner, GN = r["heads"] * r["vdim"], r["groups"] * r["state"]
            mat(p + "mix.right.in", 2 * inner + 2 * GN + r["heads"], W, 1.5)
            taps(p + "mix.right.conv", inner + 2 * GN, r["conv"]); vec(p + "mix.right.conv.b", inner + 2 * GN, 0.0, 0.3)
            vec(p + "mix.right.dt_bias", r["heads"], -1.0, 1.0); vec(p + "mix.right.A_log", r["heads"], -0.5, 1.0)
            vec(p + "mix.right.D", r["heads"], 1.0, 0.5); vec(p + "mix.right.norm", inner, 1.0)
            mat(p + "mix.right.o", W, inner)
            vec(p + "mix.left.out", W, 1.0, 0.3); vec(p + "mix.right.out", W, 1.0, 0.3)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        vec(p + "norm2", W, 1.0)
        if mlp["kind"] == "dense":
            glu(p + "mlp.", mlp["ff"])
            continue
        E, top = mlp["router"]["experts"], mlp["router"]["top"]
        for e in range(E):
            glu(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
        tables[p + "mlp.table"] = torch.rand(V, E, generator=g).argsort(dim=1)[:, :top].to(torch.int32).contiguous()
        if mlp["shared"]:
            glu(p + "mlp.shared.", mlp["shared"]["ff"])
    out = {k: v.to(torch.bfloat16).to(torch.float32) for k, v in out.items()}
    out.update(tables)
    return out


def write_dir(path: str, cfg: dict, tensors: dict[str, torch.Tensor]) -> str:
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: (v if v.dtype == torch.int32 else v.to(torch.bfloat16)).contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
    return path


def double(tensors):
    return {k: (v.double() if v.dtype.is_floating_point else v) for k, v in tensors.items()}


def variant(cfg: dict, **changes) -> dict:
    out = copy.deepcopy(cfg)
    out.update(changes)
    return out


def random_config(rng) -> dict:
    """A configuration drawn with ``rng`` (a ``random.Random``): sizes, head counts, the order of layers, where
    feed-forwards sit and of which kind, windows, taps, rotations and their stretching all vary."""
    width = rng.choice([64, 96, 128, 160, 192, 256])
    layers = []
    for _ in range(rng.randrange(2, 6)):
        taps = rng.choice([1, 2, 3, 4, 5])
        if rng.random() < 0.5:
            kv = rng.choice([1, 2, 3])
            layer = delta(kv * rng.choice([1, 2, 4]), kv, rng.choice([8, 16, 24, 64, 96]), rng.choice([8, 16, 32, 48, 72]), taps)
        else:
            kv, dim = rng.choice([1, 2, 3]), rng.choice([8, 16, 32, 48, 64])
            rot = rng.choice([None, 2, dim // 2, dim])
            scaling = rng.choice([None, STRETCH, {"factor": 3.0, "low": 0.5, "high": 8.0, "original": 128}])
            left = attention(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([dim, dim, 8, 40]), taps,
                             window=rng.choice([None, 1, 2, 17, 63, 64, 65, 128, 1000]), rot_dims=rot,
                             base=rng.choice([100.0, 1e4, 5e5]), scaling=scaling, scale=rng.choice([None, 0.3, 0.05]))
            groups = rng.choice([1, 2, 3])
            heads, vdim = groups * rng.choice([1, 2, 3]), rng.choice([8, 16, 24, 64])
            right = state_space(heads, vdim, rng.choice([8, 16, 48, 128]), groups, rng.choice([1, 2, 3, 4]),
                                rng.choice([1, heads, groups]))
            layer = parallel(left, right)
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "dense":
            mlp = dense(rng.choice([48, 100, 256]))
        elif kind == "moe":
            experts = rng.choice([1, 2, 3, 7, 16])
            mlp = moe(experts, rng.randrange(1, min(experts, 5) + 1), rng.choice([8, 24, 64, 100]), shared=rng.choice([None, 16, 72]))
        else:
            mlp = None
        layers.append(with_mlp(layer, mlp))
    return config(width, rng.randrange(100, 600), layers, eps=rng.choice([1e-6, 1e-5]), scale=rng.choice([1.0, 4.0, 11.0]))
