"""Barilix without a GPU: the configuration reader, the plan's tensor names and cache needs, the tables of the
stretched rotation, random expert tables, and the plain implementation against itself (a prompt whole, in portions
and token by token) and against hand-made cases of its window, convolution and table."""

import math
import random

import pytest
import torch

from barilix_cases import (CASES, STRETCH, attention, config, delta, dense, double, moe, parallel, random_config,
                           state_space, tensors_for, with_mlp)
from plain import barilix_plain as P


def build(cfg):
    from dryft_amd.config.barilix import BarilixConfig
    from dryft_amd.engine.model import DecoderModel
    from dryft_amd.models import resolve_architecture
    arch = resolve_architecture(cfg)
    assert arch.config_class is BarilixConfig
    return DecoderModel(arch.plan(arch.config_class.from_dict(cfg)), torch.float32, "cpu")


@pytest.mark.parametrize("name", sorted(CASES))
def test_plan_names_every_tensor(name):
    cfg = CASES[name]
    model = build(cfg)
    specs = {s.name: s.shape for s in model.tensor_specs()}
    tensors = tensors_for(cfg, 1)
    assert set(specs) == set(tensors)
    for n, shape in specs.items():
        assert tuple(shape) == tuple(tensors[n].shape), n
    assert len(model.cache_needs()) == len(cfg["layers"])


def test_cache_needs_follow_the_taps_and_windows():
    from dryft_amd.cache.spec import KVNeed, StateNeed
    needs = build(CASES["A"]).cache_needs()
    assert needs[0] == {"memory": StateNeed((4, 16, 24)), "tail": StateNeed((2, 2 * 2 * 16 + 4 * 24))}
    assert needs[1]["left.kv"] == KVNeed(2, 32, 20, None) and needs[1]["left.tail"] == StateNeed((1, 4 * 32 + 2 * 32 + 2 * 32))
    assert needs[1]["right.state"] == StateNeed((4, 24, 16)) and needs[1]["right.tail"] == StateNeed((3, 64 + 2 * 2 * 24))
    assert needs[3]["left.kv"] == KVNeed(1, 16, 70, 24)
    # one tap: no history is kept at all
    needs = build(CASES["B"]).cache_needs()
    assert needs[0] == {"left": KVNeed(3, 20, None, 12), "right.state": StateNeed((2, 8, 40))}
    assert needs[1] == {"memory": StateNeed((3, 24, 40))}


def test_random_configurations_are_read():
    for seed in range(30):
        cfg = random_config(random.Random(seed))
        model = build(cfg)
        assert {s.name for s in model.tensor_specs()} == set(tensors_for(cfg, seed))


def test_configuration_problems_come_in_one_error():
    from dryft_amd.config.barilix import BarilixConfig
    from dryft_amd.config.base import ConfigError
    bad = config(64, 100, [with_mlp(delta(3, 2, 16, 8, 4), {"kind": "sparse"}),
                           with_mlp(parallel(attention(4, 2, 16, 16, 2, rot_dims=18), state_space(3, 8, 16, 2, 2, 5)),
                                    moe(4, 6, 8))])
    del bad["embedding"]
    bad["layers"][1]["mixer"]["left"]["rot"]["scaling"] = {"factor": 2.0, "low": 1.0, "high": 1.0, "original": 64}
    with pytest.raises(ConfigError) as e:
        BarilixConfig.from_dict(bad)
    text = str(e.value)
    for piece in ("embedding", "layers[0].mlp.kind", "layers[0].mixer.heads", "layers[1].mixer.left.rot.dims",
                  "layers[1].mixer.left.rot.scaling.low", "layers[1].mixer.right.heads", "layers[1].mixer.right.norm_groups",
                  "layers[1].mlp.router.top"):
        assert piece in text, piece
    good = BarilixConfig.from_dict(CASES["A"])
    assert BarilixConfig.from_dict(good.to_dict()) == good


def test_stretched_frequencies_of_all_three_kinds():
    from dryft_amd.parts.rope import HalfRotaryPositions
    dims, base = 16, 100.0
    table = HalfRotaryPositions(dims, base, STRETCH)
    f = table.frequencies()
    plain = base ** (-2 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    want = P.scaled_frequencies(dims, base, STRETCH)
    assert torch.allclose(f, want, rtol=1e-12)
    kinds = set()
    for fi, pi in zip(f.tolist(), plain.tolist()):
        wave = 2 * math.pi / pi
        if wave < STRETCH["original"] / STRETCH["high"]:
            assert fi == pi
            kinds.add("kept")
        elif wave > STRETCH["original"] / STRETCH["low"]:
            assert math.isclose(fi, pi / STRETCH["factor"])
            kinds.add("stretched")
        else:
            assert pi / STRETCH["factor"] < fi < pi
            kinds.add("blended")
    assert kinds == {"kept", "stretched", "blended"}
    table.prepare(50, torch.float32, "cpu")
    angle = torch.arange(50, dtype=torch.float64)[:, None] * want[None]
    assert table.cos.dtype == torch.float32 and torch.allclose(table.cos.double(), angle.cos(), atol=1e-7)
    assert torch.allclose(HalfRotaryPositions(dims, base).frequencies(), plain)


def test_random_tables_hold_different_experts_in_every_row():
    from dryft_amd.weights.random_init import random_tensors
    model = build(CASES["A"])
    tensors = random_tensors(model.tensor_specs(), 3, torch.bfloat16)
    table = tensors["l1.mlp.table"]
    assert table.dtype == torch.int32 and table.shape == (200, 3)
    assert int(table.min()) >= 0 and int(table.max()) < 8
    assert all(len(set(row)) == 3 for row in table.tolist())
    assert len({tuple(r) for r in table.tolist()}) > 20


# ------------------------------------------------------------------------------------------ the plain implementation
@pytest.mark.parametrize("name", sorted(CASES))
def test_plain_whole_equals_portions_and_single_tokens(name):
    cfg = CASES[name]
    t = double(tensors_for(cfg, 5))
    toks = [int(x) for x in torch.randint(0, cfg["vocab"], (90,), generator=torch.Generator().manual_seed(2))]
    whole, _ = P.forward(cfg, t, toks)
    for cuts in ([1, 2, 3, 4], [2, 30, 64, 66], list(range(60, 90))):
        past, rows = None, []
        for a, b in zip([0] + cuts, cuts + [len(toks)]):
            out, past = P.forward(cfg, t, toks[a:b], past)
            rows.append(out)
        assert torch.allclose(torch.cat(rows), whole, atol=1e-9), (name, cuts[:3])


def test_plain_window_counts_the_token_itself():
    c = attention(1, 1, 4, 4, 1, window=3)
    g = torch.Generator().manual_seed(0)
    w = {"q": torch.zeros(4, 4), "k": torch.zeros(4, 4), "v": torch.eye(4), "o": torch.eye(4)}
    w.update({n + ".b": torch.zeros(4) for n in "qkvo"})
    w.update({n + ".conv": torch.ones(4, 1) for n in "qkv"})
    w.update({"q.norm": torch.ones(4), "k.norm": torch.ones(4)})
    h = torch.randn(6, 4, generator=g).double()
    out, _ = P.conv_attention(h, double(w), c, 1e-6)
    # equal scores: the output is the mean of the values of the token and the two before it
    assert torch.allclose(out[5], h[3:6].mean(0)) and torch.allclose(out[1], h[0:2].mean(0))


def test_plain_convolution_last_column_is_the_current_token():
    u = torch.arange(12.0).view(6, 2)
    kernel = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]])
    y, hist = P.short_conv(u, kernel)
    assert torch.equal(y[:, 0], u[:, 0])
    assert torch.equal(y[:, 1], torch.tensor([0.0, 0.0, 1.0, 3.0, 5.0, 7.0]))
    assert torch.equal(hist, u[4:])
    y2, _ = P.short_conv(u[3:], kernel, u[1:3])
    assert torch.equal(y2, y[3:])


def test_plain_table_gives_equal_weights():
    cfg = config(8, 5, [with_mlp(delta(1, 1, 4, 4, 1), moe(3, 2, 4))])
    t = double(tensors_for(cfg, 1))
    w = P.part_tensors(t, "l0.mlp.")
    h = torch.randn(5, 8, dtype=torch.float64)
    out = P.table_experts(h, torch.arange(5), w, cfg["layers"][0]["mlp"])
    for r in range(5):
        a, b = w["table"][r].tolist()
        assert a != b
        want = 0.5 * (P.gated_unit(h[r:r + 1], w, f"e{a}.") + P.gated_unit(h[r:r + 1], w, f"e{b}."))
        assert torch.allclose(out[r], want[0])
