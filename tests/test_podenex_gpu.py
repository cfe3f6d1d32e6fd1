"""Podenex on the GPU against the plain implementation (float64), in float32 and bfloat16: each new kernel and
mechanism alone, then whole models of three configurations through the step function (whole prompts, portions down
to two tokens, one token at a time, unequal batches, slots used again, long decoding), configurations drawn at random,
greedy generation through the entry point with captured steps, and the trace program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import collect_positions, trace_batches
from plain import podenex_plain as P
from podenex_cases import CASES, chunked, config, double, latent, moe, random_config, sinked, tensors_for, with_mlp, write_dir
from test_piralix_gpu import CUTS, MIXER_TOL, TOL, feed, rel_err, run_mixer

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
EPS = 1e-5
# rows of logits: in bfloat16 the worst of a thousand rows of these models lies at up to 10 times the median (0.012 to
# 0.015 of the logits' size: a layer here rounds more often than the other designs' do, after the convolution, the
# blend of values, both latents, the side input's gate), while a lost key, a window or chunk that is one off, a sink
# or a bias left out move rows by 0.1 to 1 (the tests that build such cases say so)
TOL = {"float32": TOL["float32"], "bfloat16": 0.15}
MORE_CUTS = CUTS + ([1, 2, 3, 4, 5, 6, 8],)


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_token_gate_squared_relu_and_blend(dtype):
    from dryft_amd.csrc import ops
    T = TORCH[dtype]
    g = torch.Generator().manual_seed(1)
    rows, dim, count, vocab = 9, 12, 3, 40
    gate = (2 * torch.randn(rows, dim + 5, generator=g)).to(T)
    table = torch.randn(vocab, count * dim, generator=g).to(T)
    tokens = torch.randint(0, vocab, (rows,), generator=g).to(torch.int32)
    out = torch.empty(rows, dim, dtype=T, device=DEV)
    ops.token_gate(gate.to(DEV)[:, 5:], tokens.to(DEV), table.to(DEV), 2 * dim, out)
    want = P.gelu_tanh(gate.double()[:, 5:]) * table.double()[tokens.long()][:, 2 * dim:3 * dim]
    assert rel_err(out, want) <= (1e-6 if dtype == "float32" else 6e-3)
    x = (3 * torch.randn(rows, 50, generator=g)).to(T)
    sq = torch.empty(rows, 50, dtype=T, device=DEV)
    ops.relu_squared(x.to(DEV), sq)
    assert rel_err(sq, torch.relu(x.double()) ** 2) <= (1e-6 if dtype == "float32" else 6e-3)
    a, b = torch.randn(rows, 70, generator=g).to(T), torch.randn(rows, 40, generator=g).to(T)
    lam = torch.tensor([0.3], device=DEV)
    a_dev = a.to(DEV)
    ops.blend_columns(a_dev[:, 8:32], b.to(DEV)[:, 16:40], lam)
    want = a.double().clone()
    want[:, 8:32] = 0.7 * a.double()[:, 8:32] + 0.3 * b.double()[:, 16:40]
    assert rel_err(a_dev, want) <= (1e-6 if dtype == "float32" else 6e-3)
    assert torch.equal(a_dev[:, :8].cpu(), a[:, :8]) and torch.equal(a_dev[:, 32:].cpu(), a[:, 32:])


@pytest.mark.parametrize("experts,top,groups", [(6, 2, (2, 1)), (15, 3, (5, 2)), (16, 4, (4, 1)), (5, 5, None), (1, 1, None),
                                                 (130, 6, (10, 3)), (64, 8, (8, 8))])
def test_softmax_router_with_groups_that_score_as_their_best(experts, top, groups):
    from dryft_amd.csrc import ops
    g = torch.Generator().manual_seed(experts)
    rows = 50
    z = 2 * torch.randn(rows, experts, generator=g)
    z[0, :] = 0.0                                                     # all equal: the lowest indices win
    if groups and experts >= 6:
        size = experts // groups[0]
        z[1] = -4.0                                                   # one outstanding expert in the last group, and a group
        z[1, experts - 1] = 5.0                                       # whose sum is larger but whose best is smaller
        z[1, :size] = 1.0
    chosen = torch.empty(rows, top, dtype=torch.int32, device=DEV)
    weights = torch.empty(rows, top, dtype=torch.float32, device=DEV)
    count, keep = groups or (1, 1)
    ops.moe_route(z.to(DEV), None, experts, count, keep, 1.0, chosen, weights, softmax=True, group_best=True, renorm=False)
    want_c, want_w = P.route(z.double(), top, {"count": count, "keep": keep} if groups else None)
    assert torch.equal(chosen.cpu().long(), want_c)
    assert torch.allclose(weights.cpu().double(), want_w, atol=1e-6, rtol=1e-5)
    if groups and experts >= 6 and keep < count:
        assert experts - 1 in chosen[1].tolist()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,ff,experts,top,shared", [(64, 40, 6, 2, 24), (72, 12, 5, 5, None), (128, 100, 16, 4, 64)])
def test_gateless_experts_part(dtype, hidden, ff, experts, top, shared):
    """The part alone at 3, 40 and 300 rows (the grouped products' forms for few and for many rows)."""
    from dryft_amd.parts.experts import RoutedExperts
    T = TORCH[dtype]
    mlp = moe(experts, top, ff, groups=(1, 1), shared=shared)
    t = tensors_for(config(hidden, 16, [with_mlp(sinked(1, 1, 8, 8), mlp)]), seed=hidden)
    w = {k[len("l0.mlp."):]: v for k, v in t.items() if k.startswith("l0.mlp.")}
    part = RoutedExperts(hidden, experts, top, ff, groups=None, shared=(shared,) if shared else None, unit="relu2",
                         score="softmax", correction=False, group_score="best", renormalize=False, shared_gate=False)
    part.compute_dtype = T
    names = {"router": "router", **{f"e{e}_{n}": f"e{e}.{n}" for e in range(experts) for n in ("up", "down")}}
    if shared:
        names.update({"shared_up": "shared.up", "shared_down": "shared.down"})
    assert set(part.tensor_specs()) == set(names)
    part.load({k: w[v].to(T).to(DEV) for k, v in names.items()})
    g = torch.Generator().manual_seed(2)
    for rows in (3, 40, 300):
        h = torch.randn(rows, hidden, generator=g).to(T)
        out = part.forward(h.to(DEV), None)
        want = P.routed_experts(h.double(), double(w), mlp)
        assert rel_err(out, want) <= MIXER_TOL[dtype], rows


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_side_part(dtype):
    from types import SimpleNamespace

    from dryft_amd.parts.base import Partials
    from dryft_amd.parts.stream import TokenSide, settle
    T = TORCH[dtype]
    g = torch.Generator().manual_seed(4)
    width, dim, count, vocab, rows = 72, 12, 3, 30, 11
    w = {"gate": torch.randn(dim, width, generator=g) / 8, "proj": torch.randn(width, dim, generator=g),
         "norm": 0.5 + 0.2 * torch.randn(width, generator=g)}
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    table = torch.randn(vocab, count * dim, generator=g).to(torch.bfloat16).float()
    part = TokenSide(width, dim, 1, count, vocab, EPS)
    part.compute_dtype = T
    part.load({"table": table.to(T).to(DEV), "gate": w["gate"].to(T).to(DEV), "proj": w["proj"].to(T).to(DEV),
               "norm": w["norm"].to(DEV)})
    x = (2 * torch.randn(rows, width, generator=g)).to(T)
    tokens = torch.randint(0, vocab, (rows,), generator=g)
    pending = part.forward(x.to(DEV), SimpleNamespace(tokens=tokens.to(torch.int32).to(DEV)))
    stream = torch.zeros(rows, width, dtype=torch.float32, device=DEV)
    got = settle(stream, pending)
    want = P.token_side(x.double(), tokens, table.double(), double(w), 1, dim, EPS)
    assert rel_err(got, want) <= MIXER_TOL[dtype]


@pytest.mark.parametrize("options", ["chunk", "chunk+bias", "window+sink", "bias+sink", "chunk+bias+sink"])
@pytest.mark.parametrize("heads,kv,D,lengths,tq", [(8, 2, 128, [700, 330, 65], 290), (4, 2, 32, [300, 129, 70], 300),
                                                    (6, 2, 64, [200, 150, 1], 1), (16, 4, 128, [2100], 2100)])
def test_attention_options_on_the_matrix_cores(options, heads, kv, D, lengths, tq):
    """Chunks, the bias by distance and a sink in every way of running the prompt kernel (16 or 32 rows a wave, two
    heads a wave, pages staged or straight into LDS, a bias table in LDS or too long for it) and in the decode kernel,
    against dense float64 arithmetic; rows continue after cached tokens, and chunks are counted from position 0."""
    from dryft_amd.csrc import ops
    from helpers import build_pages
    g = torch.Generator().manual_seed(len(options) + D)
    B, L = len(lengths), max(lengths)
    chunk = 100 if "chunk" in options else 0
    window = 90 if "window" in options else 0
    sink = torch.full((heads,), 0.0) if "sink" in options else None
    scale = 1.5 / D ** 0.5
    k = torch.randn(B, L, kv, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, L, kv, D, generator=g).to(torch.bfloat16)
    q_lens = [min(tq, n) for n in lengths]
    q = torch.randn(B, max(q_lens), heads, D, generator=g).to(torch.bfloat16)
    k_pages, v_pages, table, slots = build_pages(k, v, lengths, sum((n + 63) // 64 for n in lengths) + 3, B + 2, seed=1, poison=1e4)
    cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    tiles = np.concatenate([[0], np.cumsum([(ql + 63) // 64 for ql in q_lens])]).astype(np.int32)
    q_packed = torch.cat([q[b, :ql] for b, ql in enumerate(q_lens)]).contiguous()
    d = lambda t: t.to(DEV)                                                    # noqa: E731
    for n_dist in ((40, 5000) if "bias" in options else (0,)):
        rel = 2 * torch.randn(n_dist, heads, generator=g) if n_dist else None
        want = []
        for b, (n, ql) in enumerate(zip(lengths, q_lens)):
            pos_q, pos_k = torch.arange(n - ql, n), torch.arange(n)
            sc = torch.einsum("qhd,khd->hqk", q[b, :ql].double(), k[b, :n].double().repeat_interleave(heads // kv, 1)) * scale
            if rel is not None:
                sc = sc + rel.double()[(pos_q[:, None] - pos_k[None, :]).clamp(0, n_dist - 1)].permute(2, 0, 1)
            mask = P.chunk_mask(pos_q, pos_k, chunk) if chunk else P.window_mask(pos_q, pos_k, window or None)
            want.append(P.weigh(sc, mask, v[b, :n].double(), heads // kv, sink=sink is not None))
        want = torch.cat(want)
        common = dict(sink=d(sink) if sink is not None else None, chunk=chunk, rel=d(rel) if rel is not None else None)
        seq_slot = d(torch.tensor(slots, dtype=torch.int32))
        if tq == 1:
            for splits in (1, 3):
                out = torch.zeros(sum(q_lens), heads, D, dtype=torch.bfloat16, device=DEV)
                part_o = torch.empty(B * heads * splits * D, dtype=torch.float32, device=DEV)
                part_ml = torch.empty(B * heads * splits * 2, dtype=torch.float32, device=DEV)
                ops.attn_split_bf16(d(q_packed), d(k_pages), d(v_pages), d(table), seq_slot, d(torch.from_numpy(cu)),
                                    d(torch.tensor(lengths, dtype=torch.int32)), B, part_o, part_ml, splits, out, heads, kv, D,
                                    scale, window, **common)
                assert rel_err(out, want) <= 2e-2, (options, n_dist, splits)
            continue
        for mode in (0, 1, 2, 3, 5, 7):
            if mode in (2, 3, 7) and D > 128:
                continue
            out = torch.zeros(sum(q_lens), heads, D, dtype=torch.bfloat16, device=DEV)
            ops.attn_causal_bf16(d(q_packed), d(k_pages), d(v_pages), d(table), seq_slot, d(torch.from_numpy(cu)),
                                 d(torch.from_numpy(tiles)),
                                 d(torch.tensor([n - ql for n, ql in zip(lengths, q_lens)], dtype=torch.int32)), B,
                                 int(tiles[-1]) + 1, out, heads, kv, D, scale, window, mode, **common)
            assert rel_err(out, want) <= 2e-2, (options, n_dist, mode)


# ------------------------------------------------------------------------------------------ mixers alone
def mixer_case(layer, width, seed):
    from dryft_amd.config.podenex import PodenexConfig
    from dryft_amd.models.podenex import podenex_plan
    cfg = config(width, 16, [layer], eps=EPS)
    t = tensors_for(cfg, seed)
    return cfg, t, podenex_plan(PodenexConfig.from_dict(cfg))


def load_mixer(plan, t, dtype, max_len=256):
    from dryft_amd.cache import CacheStore
    from dryft_amd.parts import build_part
    T = TORCH[dtype]
    spec = plan.layers[0].parts["mixer"]
    part = build_part(spec)
    part.compute_dtype = T
    part.load({logical: t[spec.tensors[logical]].to(DEV).to(T) for logical in part.tensor_specs()})
    cache = CacheStore({0: part.cache_need()}, max_tokens=64 * 16, n_slots=4, max_len=max_len, dtype=T, device=DEV)
    positions = {}
    for name, ps in plan.positions.items():
        positions[name] = build_part(ps)
        positions[name].prepare(max_len, T, DEV)
    return part, cache, positions


def inputs(dtype, width, lengths=(201, 9, 70), seed=12):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(n, width, generator=g).to(TORCH[dtype]).float() for n in lengths]


def plain_mixer(layer, h, w, past=None):
    m = layer["mixer"]
    if layer["type"] == "attention":
        return P.chunked_attention(h, w, m, past, None, True)[:2]
    if layer["type"] == "attention_2":
        return P.sink_attention(h, w, m, EPS, past, None, True)[:2]
    return P.latent_attention(h, w, m, EPS, past)


MIXER_SHAPES = {
    "chunked-small": chunked(4, 2, 16, 32, conv=3, chunk=24, bias=(12, 18), v_mix=True),
    "chunked-cores": chunked(4, 2, 32, 32, conv=4, chunk=64, bias=(16, 128)),
    "chunked-page-and-one": chunked(2, 1, 16, 48, conv=2, chunk=65, bias=(6, 200)),
    "chunked-bare": chunked(3, 3, 20, 12, conv=1),                         # one tap, no chunk, no table
    "chunked-no-conv": chunked(2, 2, 64, 64, chunk=100, bias=(32, 64)),
    "chunked-128": chunked(2, 1, 128, 128, conv=4, chunk=128, bias=(16, 110), scale=0.05),
    "chunked-128-no-table": chunked(2, 1, 128, 128, conv=2, chunk=100, scale=0.05),
    "chunked-long-table": chunked(2, 2, 32, 32, bias=(8, 5000)),          # too long for LDS: read from memory
    "sinked-cores": sinked(4, 2, 32, 32, window=20, v_mix=True),
    "sinked-wide-values": sinked(2, 1, 24, 64, window=65),
    "sinked-odd": sinked(6, 3, 10, 12),
    "sinked-itself": sinked(8, 2, 16, 16, window=1),
    "sinked-128": sinked(4, 2, 128, 128, window=130, scale=0.05),
    "latent-cores": latent(2, 16, 16, 16, 24, 20, window=70, rot_dims=16, base=100.0),
    "latent-part-rotated": latent(3, 8, 16, 24, 16, 12, rot_dims=8),
    "latent-odd": latent(3, 12, 6, 20, 10, 14, rot_dims=6, base=50.0),
    "latent-192": latent(2, 128, 64, 128, 96, 64, window=128, rot_dims=64, base=5e5, scale=0.04),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(MIXER_SHAPES))
def test_mixer_alone(dtype, shape):
    layer = MIXER_SHAPES[shape]
    cfg, t, plan = mixer_case(layer, 64, seed=len(shape))
    part, cache, positions = load_mixer(plan, t, dtype)
    seqs = inputs(dtype, 64)
    w = double(P.sub(t, "l0.mix."))
    want = [plain_mixer(layer, s.double(), w)[0] for s in seqs]
    for cuts in MORE_CUTS:
        for got, ref in zip(run_mixer(part, cache, positions, dtype, seqs, cuts), want):
            assert rel_err(got, ref) <= MIXER_TOL[dtype], (shape, cuts[:3])


def sharpened(layer, factor):
    out = {"type": layer["type"], "mixer": dict(layer["mixer"])}
    out["mixer"]["scale"] = factor
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [None, 20, 64, 65, 130])
def test_chunks_bias_and_history_show(dtype, chunk):
    """A score scale large enough that a row gives most of its weight to one or two keys, wherever they are: then a
    chunk that is one token off, a key lost behind a page border, a bias row that is one off, a convolution that forgets
    its history or a gate left out moves some row by far more than the tolerance (the plain implementation with each of
    those faults shows it), in prompts, portions and decoding."""
    tol = {"float32": MIXER_TOL["float32"], "bfloat16": 2 * MIXER_TOL["bfloat16"]}[dtype]
    layer = chunked(2, 1, 32, 32, conv=3, chunk=chunk, bias=(16, 100), scale=0.4)
    m = layer["mixer"]
    cfg, t, plan = mixer_case(layer, 32, seed=3)
    t["l0.mix.rel"] = (3 * t["l0.mix.rel"]).to(torch.bfloat16).float()
    part, cache, positions = load_mixer(plan, t, dtype)
    h = inputs(dtype, 32, (200,), seed=4)[0]
    w = double(P.sub(t, "l0.mix."))
    want = plain_mixer(layer, h.double(), w)[0]

    def other(w2, m2):
        return P.chunked_attention(h.double(), w2, m2, None, None, True)[0]
    if chunk:
        for off in (-1, 1):
            assert rel_err(other(w, {**m, "mask": {"size": chunk + off}}), want) > 0.2
    else:
        near_only = P.chunked_attention(h[64:].double(), w, m, None, None, True)[0]
        assert rel_err(near_only[86:], want[150:]) > 0.2                  # keys of the first page matter to rows 150..
    faults = {"no history": ({**w, **{n + ".conv": torch.cat([0 * w[n + ".conv"][:, :-1], w[n + ".conv"][:, -1:]], 1) for n in "qkv"}}, m),
              "no bias": ({**w, "rel": 0 * w["rel"]}, m),
              "bias rows shifted": ({**w, "rel": torch.roll(w["rel"], 1, 0)}, m),
              "bias reaches its end elsewhere": (w, {**m, "bias_max": 60}),
              "no gate": ({**w, "g": 0 * w["g"]}, m)}
    for what, (w2, m2) in faults.items():
        assert rel_err(other(w2, m2), want) > 0.1, what
    for cuts in ([], list(range(120, 200)), [64, 128], [2, 63, 65, 127, 129], [19, 20, 21], [1, 2, 3]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got, want) <= tol, cuts[:3]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 20, 64, 65, 130])
def test_window_sink_and_norms_show(dtype, window):
    tol = {"float32": MIXER_TOL["float32"], "bfloat16": 2 * MIXER_TOL["bfloat16"]}[dtype]
    layer = sinked(2, 1, 32, 32, window=window, scale=0.5)         # normed q and k: scores of order scale * dim
    m = layer["mixer"]
    cfg, t, plan = mixer_case(layer, 32, seed=5)
    part, cache, positions = load_mixer(plan, t, dtype)
    h = inputs(dtype, 32, (200,), seed=6)[0]
    w = double(P.sub(t, "l0.mix."))
    want = plain_mixer(layer, h.double(), w)[0]

    def other(w2, m2, sink=True):
        if sink:
            return P.sink_attention(h.double(), w2, m2, EPS, None, None, True)[0]
        saved, P.weigh = P.weigh, lambda s, mask, v, group, sink=False: saved(s, mask, v, group, False)
        try:
            return P.sink_attention(h.double(), w2, m2, EPS, None, None, True)[0]
        finally:
            P.weigh = saved
    if window:
        for off in (-1, 1):
            assert rel_err(other(w, {**m, "mask": {"size": window + off}}), want) > 0.1
    else:
        near_only = P.sink_attention(h[64:].double(), w, m, EPS, None, None, True)[0]
        assert rel_err(near_only[86:], want[150:]) > 0.1
    assert rel_err(other(w, m, sink=False), want) > 0.02, "no sink"
    faults = {"no key norm weight": ({**w, "k.norm": torch.ones_like(w["k.norm"])}, m),
              "no bias": ({**w, "k.b": 0 * w["k.b"], "q.b": 0 * w["q.b"]}, m),
              "no value bias": ({**w, "v.b": 0 * w["v.b"]}, m), "no output bias": ({**w, "o.b": 0 * w["o.b"]}, m)}
    for what, (w2, m2) in faults.items():
        assert rel_err(other(w2, m2), want) > 0.05, what
    for cuts in ([], list(range(120, 200)), [64, 128], [2, 63, 65, 127, 129], [19, 20, 21], [1, 2, 3]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got, want) <= tol, cuts[:3]


def rotate_halves(x, pos, dims, base):
    """The other pairing (entry ``i`` with ``i + dims/2``), which this design does not use."""
    f = base ** (-2 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    a = (pos.to(torch.float64)[:, None] * f[None, :])[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), x[..., dims:]], -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 20, 64, 65, 130])
def test_latent_window_rotation_and_gate_show(dtype, window):
    tol = {"float32": MIXER_TOL["float32"], "bfloat16": 2 * MIXER_TOL["bfloat16"]}[dtype]
    layer = latent(2, 16, 16, 32, 24, 20, window=window, rot_dims=16, base=100.0, scale=0.25)
    m = layer["mixer"]
    cfg, t, plan = mixer_case(layer, 32, seed=7)
    part, cache, positions = load_mixer(plan, t, dtype)
    h = inputs(dtype, 32, (200,), seed=8)[0]
    w = double(P.sub(t, "l0.mix."))
    want = plain_mixer(layer, h.double(), w)[0]
    if window:
        for off in (-1, 1):
            assert rel_err(P.latent_attention(h.double(), w, {**m, "mask": {"size": window + off}}, EPS)[0], want) > 0.1
    else:
        assert rel_err(P.latent_attention(h[64:].double(), w, m, EPS)[0][86:], want[150:]) > 0.1
    saved = P.rotate_pairs
    try:
        P.rotate_pairs = rotate_halves
        assert rel_err(P.latent_attention(h.double(), w, m, EPS)[0], want) > 0.1, "pairs, not halves"
    finally:
        P.rotate_pairs = saved
    faults = {"no rotation": (w, {**m, "rot": None}), "another base": (w, {**m, "rot": {"dims": 16, "base": 1e4}}),
              "a gate per head only": ({**w, "g": w["g"][::32].repeat_interleave(32, 0)}, m),
              "no latent norm weight": ({**w, "dkv.norm": torch.ones_like(w["dkv.norm"])}, m)}
    for what, (w2, m2) in faults.items():
        assert rel_err(P.latent_attention(h.double(), w2, m2, EPS)[0], want) > 0.05, what
    for cuts in ([], list(range(120, 200)), [64, 128], [2, 63, 65, 127, 129], [19, 20, 21], [1, 2, 3]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got, want) <= tol, cuts[:3]


# ------------------------------------------------------------------------------------------ whole models
# The router picks the experts with the largest scores, and random weights bring close calls: where two scores are
# nearer than bfloat16 activations resolve, the library and the float64 plain model may pick different experts, and
# the row moves by a whole expert's output (a jump, not rounding; about one row in a hundred per layer here). So
# every case runs twice in bfloat16: as it is, where the typical row must agree and few rows may jump, and with every
# expert chosen (``all_chosen``: nothing to pick, everything else the same), where every row must agree. float32
# resolves the test models' calls and must agree in every row of both.
def all_chosen(cfg):
    out = json.loads(json.dumps(cfg))
    for layer in out["layers"]:
        if layer["mlp"]:
            r = layer["mlp"]["router"]
            r["top"] = r["experts"]
            if r["groups"]:
                r["groups"]["keep"] = r["groups"]["count"]
    return out


def row_errors(got, want):
    d = got.double().cpu() - want.double().cpu()
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.double().pow(2).mean().sqrt()


def assert_rows(rows, dtype, strict, tol, where):
    rows = torch.as_tensor(rows, dtype=torch.float64).flatten()
    if dtype == "float32" or strict:
        assert float(rows.max()) <= tol, (where, float(rows.max()))
    else:
        jumps = int((rows > tol).sum())
        assert float(rows.median()) <= tol / 2 and jumps <= max(3, 0.08 * rows.numel()) and float(rows.max()) <= 1.0, \
            (where, float(rows.median()), jumps, float(rows.max()))


class Model:
    def __init__(self, tmp, name, cfg=None, seed=None):
        self.name, self.cfg = name, cfg or CASES[name]
        self.tensors = tensors_for(self.cfg, seed=seed if seed is not None else ord(name[0]))
        self.dir = write_dir(os.path.join(tmp, name), self.cfg, self.tensors)
        self.vocab = self.cfg["vocab"]
        self._plain, self._engines = {}, {}

    def tokens(self, n, seed=0):
        return [int(x) for x in np.random.default_rng(1000 * seed + n).integers(0, self.vocab, size=n)]

    def plain(self, tokens) -> torch.Tensor:
        key = tuple(tokens)
        if key not in self._plain:
            self._plain[key] = P.forward(self.cfg, double(self.tensors), list(tokens))[0]
        return self._plain[key]

    def engine(self, dtype, **kw):
        from dryft_amd import Engine
        key = (dtype, tuple(sorted(kw.items())))
        if key not in self._engines:
            args = dict(max_batch=4, max_len=320, max_tokens=64 * 24, use_graph=False)
            args.update(kw)
            self._engines[key] = Engine(self.dir, dtype=dtype, **args)
        return self._engines[key]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    tmp = str(tmp_path_factory.mktemp("podenex"))
    out = {name: Model(tmp, name) for name in CASES}
    out.update({name + "*": Model(tmp, name + "*", cfg=all_chosen(CASES[name])) for name in CASES})
    return out


def variants(models, name):
    """``(model, must every row agree in bfloat16 too?)``"""
    return [(models[name], False), (models[name + "*"], True)]


LENGTHS = [1, 2, 5, 63, 64, 65, 130]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CASES))
def test_whole_prompts_portions_and_single_tokens(models, name, dtype):
    for model, strict in variants(models, name):
        engine = model.engine(dtype)
        requests = {f"r{n}": model.tokens(n) for n in LENGTHS}
        for what, cuts_of in (("whole", lambda n: []), ("last tokens one by one", lambda n: list(range(max(1, n - 24), n))),
                              ("portions", lambda n: [2, 4, 7, 64, 66, 129]), ("first tokens one by one", lambda n: [1, 2, 3])):
            got = feed(engine, requests, cuts_of)
            rows = torch.cat([row_errors(got[rid], model.plain(toks)) for rid, toks in requests.items()])
            assert_rows(rows, dtype, strict, TOL[dtype], (model.name, what))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_layer_by_layer(models, name, dtype):
    """The residual stream after every layer against the plain one (float32 in both precisions)."""
    from dryft_amd import SeqStep
    for model, strict in variants(models, name):
        engine = model.engine(dtype)
        toks = model.tokens(37)
        want = P.forward(model.cfg, double(model.tensors), toks)[1]
        got = []
        slot = engine.acquire(1)[0]
        engine.step([SeqStep(slot, toks, [36])], tap=lambda i, x: got.append(x.cpu()))
        engine.release([slot])
        assert len(got) == len(want) == len(model.cfg["layers"])
        for i, (g, w) in enumerate(zip(got, want)):
            assert g.dtype == torch.float32
            assert_rows(row_errors(g, w), dtype, strict, 2e-5 if dtype == "float32" else 6e-2, (model.name, i))


@pytest.mark.parametrize("dtype", DTYPES)
def test_shared_values_reach_the_later_layers(models, dtype):
    """The later layers' blend shows in the logits: the plain model without it is far away, the library is not."""
    model = models["A*"]
    toks = model.tokens(90, seed=4)
    want = model.plain(toks)
    other = double(model.tensors)
    other["l2.mix.vmix"], other["l3.mix.vmix"] = other["l2.mix.vmix"] * 0, other["l3.mix.vmix"] * 0
    assert float(row_errors(P.forward(model.cfg, other, toks)[0], want).median()) > 0.2
    got = feed(model.engine(dtype), {"r": toks}, lambda n: [40, 41, 89])["r"]
    assert rel_err(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CASES))
def test_unequal_batches_and_slots_used_again(models, name, dtype):
    """Three batches one after another in the same slots and pages: unequal prompts start together and decode
    together, the shorter ones end earlier. Against the plain implementation, and against each request alone."""
    from dryft_amd import SeqStep
    for model, strict in variants(models, name):
        engine = model.engine(dtype, max_batch=3, max_tokens=64 * 9)
        batches = [{f"b{b}r{n}": (model.tokens(n, seed=b + 1), k) for n, k in sizes}
                   for b, sizes in enumerate([[(70, 6), (3, 2), (130, 20)], [(1, 0), (66, 65), (20, 3)], [(129, 1), (64, 10)]])]
        records = list(trace_batches(batches))
        slot_of, outputs = {}, {}
        for rec in records:
            seqs = []
            for e in rec["entries"]:
                if e["id"] not in slot_of:
                    slot_of[e["id"]] = engine.acquire(1)[0]
                seqs.append(SeqStep(slot_of[e["id"]], e["tokens"], e["want"]))
            outputs[rec["step"]] = engine.step(seqs).cpu()
            engine.release([slot_of.pop(r) for r in rec["end"]])
        got = collect_positions(records, outputs)
        alone = feed(model.engine(dtype), {rid: toks for b in batches for rid, (toks, _) in b.items()}, lambda n: [])
        against_plain, against_alone = [], []
        for (rid, pos), row in got.items():
            toks = next(b[rid][0] for b in batches if rid in b)
            against_plain.append(float(row_errors(row[None], model.plain(toks)[pos][None])))
            # what else is in the batch, and how the prompt was cut, changes a row by rounding only
            scale = model.plain(toks).double().pow(2).mean().sqrt() / alone[rid][pos].double().pow(2).mean().sqrt()
            against_alone.append(float(row_errors(row[None], alone[rid][pos][None]) / scale))
        assert_rows(against_plain, dtype, strict, TOL[dtype], (model.name, "plain"))
        assert_rows(against_alone, dtype, strict, 2e-5 if dtype == "float32" else TOL[dtype], (model.name, "alone"))


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(models, dtype):
    """300 tokens one at a time: every window and chunk of the model passes over decoded tokens several times."""
    from dryft_amd import SeqStep
    for model, strict in variants(models, "A"):
        engine = model.engine(dtype)
        toks = model.tokens(300, seed=7)
        want = model.plain(toks)
        slot = engine.acquire(1)[0]
        rows = [engine.step([SeqStep(slot, toks[:2], [1])])]
        for t in toks[2:]:
            rows.append(engine.step([SeqStep(slot, [t], [0])]))
        engine.release([slot])
        assert_rows(row_errors(torch.cat(rows), want[1:]), dtype, strict, TOL[dtype], model.name)


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(seed, tmp_path):
    """Configurations drawn at random: three unequal prompts start together and decode together. float32 must agree
    with the plain implementation to rounding in every row; in bfloat16 the typical row must (single rows of a deep
    random model magnify rounding whatever computes them, and a router's close call moves a row by a whole expert)."""
    import random

    from dryft_amd import Engine, SeqStep
    cfg = random_config(random.Random(seed))
    tensors = tensors_for(cfg, seed)
    path = write_dir(str(tmp_path / "m"), cfg, tensors)
    g = np.random.default_rng(seed)
    reqs = [[int(x) for x in g.integers(0, cfg["vocab"], size=n)] for n in (1, 37, 150)]
    want = [P.forward(cfg, double(tensors), r)[0] for r in reqs]
    for dtype in DTYPES:
        engine = Engine(path, dtype=dtype, max_batch=4, max_len=256, max_tokens=64 * 16, use_graph=False)
        slots = engine.acquire(3)
        heads = [max(1, len(r) - 6) for r in reqs]
        got = [[] for _ in reqs]
        out = engine.step([SeqStep(s, r[:h], list(range(h))) for s, r, h in zip(slots, reqs, heads)]).cpu()
        at = 0
        for i, h in enumerate(heads):
            got[i].append(out[at:at + h])
            at += h
        for k in range(6):
            live = [(i, s) for i, s in enumerate(slots) if heads[i] + k < len(reqs[i])]
            if live:
                out = engine.step([SeqStep(s, [reqs[i][heads[i] + k]], [0]) for i, s in live]).cpu()
                for j, (i, _) in enumerate(live):
                    got[i].append(out[j:j + 1])
        engine.release(slots)
        for mine, ref in zip(got, want):
            mine = torch.cat(mine).double()
            d = mine - ref
            d = d - d.mean(-1, keepdim=True)
            rows = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()
            if dtype == "float32":
                assert float(rows.max()) <= TOL[dtype], (seed, cfg["layers"])
            else:
                # a row where a router's close call went the other way moves by an expert's output, however large
                assert float(rows.median()) <= 0.1 and float((rows > 0.3).double().mean()) <= 0.05, \
                    (seed, float(rows.median()), float(rows.max()))


def plain_greedy(model, prompt, n):
    toks, out, logits = list(prompt), [], []
    for _ in range(n):
        row = P.forward(model.cfg, double(model.tensors), toks)[0][-1]
        logits.append(row)
        out.append(int(row.argmax()))
        toks.append(out[-1])
    return out, logits


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(models, name, dtype):
    """``Engine.generate`` with captured steps: the scheduler, the sampler and the graphs serve this design as they
    serve the others. Every token is the plain loop's, or one the plain logits leave within the tolerance of the best
    (in bfloat16 on the models whose experts are all chosen, so that no close call of a router decides a token)."""
    model = models[name if dtype == "float32" else name + "*"]
    prompts = [model.tokens(n, seed=3) for n in (5, 17, 2)]
    for use_graph in (True, False):
        engine = model.engine(dtype, max_batch=4, max_len=64, max_tokens=64 * 4, use_graph=use_graph)
        got = engine.generate_all(prompts, 8)
        assert [len(g) for g in got] == [8, 8, 8]
        for prompt, mine in zip(prompts, got):
            want, logits = plain_greedy(model, prompt, 8)
            for t in range(8):
                if mine[t] != want[t]:
                    spread = float(logits[t].max() - logits[t].min())
                    assert float(logits[t].max() - logits[t][mine[t]]) <= 4 * TOL[dtype] * spread, (name, t)
                    break
    # a second generation in the same engine reuses slots, pages and captured steps, and repeats the first token for token
    engine = model.engine(dtype, max_batch=4, max_len=64, max_tokens=64 * 4, use_graph=True)
    first = engine.generate_all(prompts, 8)
    assert engine.generate_all(prompts, 8) == first


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_program(models, dtype, tmp_path):
    model = models["C*"]
    batches = [{f"r{n}": (model.tokens(n, seed=9), k) for n, k in [(40, 5), (2, 1), (90, 12)]}, {"s": (model.tokens(65, seed=2), 64)}]
    records = list(trace_batches(batches))
    live = max(sum(len(t) for t, _ in b.values()) for b in batches)
    out_dir = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model.dir, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(live)]
    proc = subprocess.run(cmd, input="".join(json.dumps(r) + "\n" for r in records), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {r['step']}" for r in records]
    outputs = {}
    for r in records:
        n_want = sum(len(e["want"]) for e in r["entries"])
        if n_want:
            outputs[r["step"]] = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{r['step']}.f32"), dtype="<f4").reshape(n_want, model.vocab))
    for (rid, pos), row in collect_positions(records, outputs).items():
        toks = next(b[rid][0] for b in batches if rid in b)
        assert rel_err(row[None], model.plain(toks)[pos][None]) <= TOL[dtype], (rid, pos)
