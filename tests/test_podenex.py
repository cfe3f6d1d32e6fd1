"""Podenex without a GPU: the configuration reader, the plan's tensor names and cache needs, the bias table's rows,
and the plain implementation against itself (a prompt whole, in portions and token by token), against library
routines and against hand-made cases of its masks, sink, router and shared values."""

import math
import random

import pytest
import torch
import torch.nn.functional as F

from podenex_cases import CASES, chunked, config, double, latent, moe, random_config, sinked, tensors_for, with_mlp
from plain import podenex_plain as P


def build(cfg):
    from dryft_amd.config.podenex import PodenexConfig
    from dryft_amd.engine.model import DecoderModel
    from dryft_amd.models import resolve_architecture
    arch = resolve_architecture(cfg)
    assert arch.config_class is PodenexConfig
    return DecoderModel(arch.plan(arch.config_class.from_dict(cfg)), torch.float32, "cpu")


def same_shape(spec, shape):
    return len(spec) == len(shape) and all(a in (-1, b) for a, b in zip(spec, shape))


@pytest.mark.parametrize("name", sorted(CASES))
def test_plan_names_every_tensor(name):
    cfg = CASES[name]
    model = build(cfg)
    specs = {s.name: s.shape for s in model.tensor_specs()}
    tensors = tensors_for(cfg, 1)
    assert set(specs) == set(tensors)
    for n, shape in specs.items():
        assert same_shape(tuple(shape), tuple(tensors[n].shape)), n
    assert len(model.cache_needs()) == len(cfg["layers"])


def test_cache_needs_follow_windows_chunks_and_taps():
    from dryft_amd.cache.spec import KVNeed, StateNeed
    needs = build(CASES["A"]).cache_needs()
    assert needs[0] == KVNeed(2, 32, 20, None)
    assert needs[2] == {"kv": KVNeed(2, 16, 24, 32), "tail": StateNeed((2, 4 * 16 + 2 * 16 + 2 * 32))}
    assert needs[3] == KVNeed(1, 24, 65, 64)
    assert needs[4].window is None and needs[4].num_kv_heads == 3 and needs[4].head_dim == 24
    needs = build(CASES["B"]).cache_needs()
    assert needs[0] == KVNeed(3, 20, None, 12)                  # one tap: no history; no chunk: every key is kept


def test_only_the_first_sharing_layer_leaves_its_values():
    model = build(CASES["C"])
    flags = [getattr(b.mixer, "value_mix", None) for b in model.blocks]
    assert flags == [None, ("v_mix", True), None, None, ("v_mix", False)]


def test_random_configurations_are_read():
    for seed in range(40):
        cfg = random_config(random.Random(seed))
        model = build(cfg)
        assert {s.name for s in model.tensor_specs()} == set(tensors_for(cfg, seed))


def test_configuration_problems_come_in_one_error():
    from dryft_amd.config.base import ConfigError
    from dryft_amd.config.podenex import PodenexConfig
    no_window = sinked(3, 2, 16, 8)
    no_window["mixer"]["mask"] = {"size": 0}
    bad = config(64, 100, [with_mlp(no_window, {"kind": "dense"}),
                           with_mlp(latent(2, 8, 8, 8, 8, 8, rot_dims=10), moe(6, 7, 8, groups=(4, 5))),
                           {"type": "wkv", "mixer": {}, "mlp": None}])
    with pytest.raises(ConfigError) as e:
        PodenexConfig.from_dict(bad)
    text = "\n".join(e.value.problems)
    for piece in ("layers[0].mixer.heads (3) is not a multiple", "layers[0].mixer.mask.size", "layers[0].mlp.kind",
                  "layers[1].mixer.rot.dims", "layers[1].mlp.router.top", "layers[1].mlp.router.groups.count", "layers[2]"):
        assert piece in text, piece
    mixed = config(64, 100, [chunked(2, 1, 8, 16, v_mix=True), sinked(2, 2, 8, 16, v_mix=True)])
    with pytest.raises(ConfigError):
        PodenexConfig.from_dict(mixed)


# ------------------------------------------------------------------------------------------ the bias table's rows
@pytest.mark.parametrize("rows,far", [(16, 128), (12, 18), (6, 200), (2, 2), (32, 17), (16, 100)])
def test_distance_rows(rows, far):
    from dryft_amd.parts.attention import distance_row
    half = rows // 2
    got = [distance_row(n, rows, far) for n in range(far + 50)]
    assert got == [P.distance_bucket(n, rows, far) for n in range(far + 50)]
    assert got[:half] == list(range(half))                        # every short distance has a row of its own
    assert got[half] == half and all(b >= a for a, b in zip(got, got[1:])) and max(got) == rows - 1
    assert all(g == rows - 1 for g in got[far:])                  # and from `far` on all share the last row
    for n in range(half, far):                                    # row k begins where (n / half) = (far / half)^(k / (rows - half))
        k = got[n] - half
        assert half * (far / half) ** (k / (rows - half)) <= n * (1 + 1e-12)
        if got[n] < rows - 1:
            assert n < half * (far / half) ** ((k + 1) / (rows - half)) * (1 + 1e-12)


def test_exact_borders_of_the_logarithmic_half():
    # 16 rows reaching distance 128: the upper half's rows begin at 8 * 2^(k/2), so 16, 32 and 64 begin rows 10, 12, 14
    assert [P.distance_bucket(n, 16, 128) for n in (15, 16, 31, 32, 63, 64, 127, 128)] == [9, 10, 11, 12, 13, 14, 15, 15]


# ------------------------------------------------------------------------------------------ plain against library routines
def test_gelu_and_norms_against_torch():
    g = torch.Generator().manual_seed(0)
    z = 3 * torch.randn(1000, generator=g, dtype=torch.float64)
    assert torch.allclose(P.gelu_tanh(z), F.gelu(z, approximate="tanh"), atol=1e-12)
    x = torch.randn(7, 40, generator=g, dtype=torch.float64) + 2.0
    w = torch.randn(40, generator=g, dtype=torch.float64)
    assert torch.allclose(P.layer_norm(x, w, 1e-5), F.layer_norm(x, (40,), w, None, 1e-5), atol=1e-12)
    assert torch.allclose(P.rms(x, 1e-5) * w, F.rms_norm(x, (40,), w, 1e-5), atol=1e-12)


def test_sink_is_one_more_key_of_score_zero_without_a_value():
    g = torch.Generator().manual_seed(1)
    s = 4 * torch.randn(2, 5, 9, generator=g, dtype=torch.float64)
    v = torch.randn(9, 2, 3, generator=g, dtype=torch.float64)
    mask = P.window_mask(torch.arange(4, 9), torch.arange(9), 4)
    got = P.weigh(s, mask, v, 1, sink=True)
    padded = torch.cat([s.masked_fill(~mask[None], -math.inf), torch.zeros(2, 5, 1, dtype=torch.float64)], -1)
    p = torch.softmax(padded, -1)[..., :9]
    assert torch.allclose(got, torch.einsum("hqk,khd->qhd", p, v), atol=1e-12)
    assert float(p.sum(-1).max()) < 1.0
    plain = P.weigh(s, mask, v, 1)
    assert not torch.allclose(got, plain, atol=1e-3)


def test_masks_by_hand():
    pos = torch.arange(10)
    w = P.window_mask(pos, pos, 3)
    assert w[5].tolist() == [False, False, False, True, True, True, False, False, False, False]
    assert w[1].tolist()[:3] == [True, True, False]
    c = P.chunk_mask(pos, pos, 4)
    assert c[5].tolist() == [False, False, False, False, True, True, False, False, False, False]
    assert c[4].tolist()[3:6] == [False, True, False] and c[3].tolist()[:4] == [True] * 4
    # chunks are counted from position 0 whatever portion a row comes in
    later = P.chunk_mask(torch.arange(6, 8), pos, 4)
    assert later[0].tolist() == [False] * 4 + [True, True, True] + [False] * 3


def test_router_by_hand():
    # 2 groups of 3: the group with the single best expert stays although the other has the larger sum
    z = torch.tensor([[2.0, -5.0, -5.0, 1.5, 1.4, 1.3]], dtype=torch.float64)
    s = torch.softmax(z, -1)
    chosen, weights = P.route(z, 2, {"count": 2, "keep": 1})
    assert chosen.tolist() == [[0, 1]] and torch.allclose(weights, s[:, [0, 1]])
    assert float(weights.sum()) < 1.0                                   # the scores are taken as they are
    chosen, _ = P.route(z, 2, {"count": 2, "keep": 2})
    assert chosen.tolist() == [[0, 3]]
    chosen, _ = P.route(z, 3, None)
    assert chosen.tolist() == [[0, 3, 4]]


def test_rotation_by_hand():
    x = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 5.0, 6.0]]], dtype=torch.float64)
    out = P.rotate_pairs(x, torch.tensor([3]), 4, 100.0)
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    want = [math.cos(a0), math.sin(a0), -2 * math.sin(a1), 2 * math.cos(a1), 5.0, 6.0]
    assert torch.allclose(out[0, 0], torch.tensor(want, dtype=torch.float64), atol=1e-12)


# ------------------------------------------------------------------------------------------ plain against itself
@pytest.mark.parametrize("name", sorted(CASES))
def test_plain_whole_in_portions_and_token_by_token(name):
    cfg = CASES[name]
    t = double(tensors_for(cfg, 3))
    g = torch.Generator().manual_seed(5)
    toks = torch.randint(0, cfg["vocab"], (150,), generator=g).tolist()
    whole, streams, _ = P.forward(cfg, t, toks)
    assert streams.shape == (len(cfg["layers"]), 150, cfg["width"])
    for cuts in ([2, 3, 64, 66, 129], list(range(100, 150))):
        past, rows = None, []
        edges = [0] + cuts + [150]
        for a, b in zip(edges[:-1], edges[1:]):
            out, _, past = P.forward(cfg, t, toks[a:b], past)
            rows.append(out)
        assert torch.allclose(torch.cat(rows), whole, atol=1e-9), cuts[:3]


def test_shared_values_matter_and_the_first_layers_blend_does_not():
    cfg = CASES["A"]
    t = double(tensors_for(cfg, 4))
    toks = list(range(40))
    want = P.forward(cfg, t, toks)[0]
    other = dict(t)
    other["l0.mix.vmix"] = t["l0.mix.vmix"] + 0.3                 # the first sharing layer never blends
    assert torch.equal(P.forward(cfg, other, toks)[0], want)
    other = dict(t)
    other["l3.mix.vmix"] = t["l3.mix.vmix"] * 0
    assert not torch.allclose(P.forward(cfg, other, toks)[0], want, atol=1e-3)


def test_token_side_reads_its_own_run_of_columns():
    cfg = CASES["A"]
    t = double(tensors_for(cfg, 6))
    toks = list(range(10, 30))
    want = P.forward(cfg, t, toks)[1]
    other = dict(t)
    table = t["side.embed"].clone()
    table[:, 8:16] += 1.0                                          # layer 1's columns
    other["side.embed"] = table
    got = P.forward(cfg, other, toks)[1]
    assert torch.equal(got[0], want[0]) and not torch.allclose(got[1], want[1], atol=1e-3)
