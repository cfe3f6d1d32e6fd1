"""Barilix: from ``BarilixConfig`` to a model plan.

A decoder on a float32 residual stream that starts as the embedding times a factor. No norm stands in front of a
sublayer; each sublayer's output goes through a layer norm (a weight, no bias) before it is added:
``x <- x + norm1(mixer(x))``, ``x <- x + norm2(ff(x))``. A layer's mixer is either two mixers side by side on the
same input (``parallel``: attention over a sliding window, with biases, a short convolution on q, k and v, a norm per
head and a partial rotation over halves; and a state-space recurrence behind a short convolution; each output
rms-normed with a weight of its own, then half their sum) or the gated delta rule (``delta``). The feed-forward is
a gated unit with silu, dense or as experts that a table from token id to experts chooses, all with equal weight,
plus an optional shared one; a layer may have none. A final layer norm, and an output head of its own.

What the design fixes rather than the file: the ``1e-6`` under the delta rule's unit lengths and its ``dim^-1/2``
on the queries (defaults of that part), silu everywhere, equal expert weights. Checkpoint names: ``embed``, ``head``,
``final.norm`` and per layer ``l<i>.norm1``, ``norm2``, ``l<i>.mix.*`` (``left.*``, ``right.*`` in a parallel layer),
``l<i>.mlp.*``.
"""

from __future__ import annotations

from ..config.barilix import BarilixConfig
from ..config.plan import LayerSpec, ModelPlan, PartSpec, Run
from . import register_architecture


def _norm(cfg: BarilixConfig, name: str) -> PartSpec:
    return PartSpec("stream_layernorm", dict(size=cfg.width, eps=cfg.norm_eps), {"weight": name})


def _attention(cfg: BarilixConfig, m: dict, positions: dict[str, PartSpec]) -> PartSpec:
    rot, name = m["rot"], None
    if rot is not None:
        spec = PartSpec("half_rotary", dict(dims=rot["dims"], base=rot["base"], scaling=rot["scaling"]))
        name = next((n for n, s in positions.items() if s == spec), None)     # layers with equal rotations share tables
        if name is None:
            name = f"rotary{len(positions)}"
            positions[name] = spec
    return PartSpec(
        "gqa_attention",
        dict(hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"],
             value_dim=m["vdim"], qk_norm_eps=cfg.norm_eps, positions=name, scale=m["scale"],
             window=m["mask"]["size"] if m["mask"] else None, float_weights=True, bias=True, conv_taps=m["conv"]))


_ATTENTION_NAMES = {"q_proj": "q", "k_proj": "k", "v_proj": "v", "o_proj": "o", "q_bias": "q.b", "k_bias": "k.b",
                    "v_bias": "v.b", "o_bias": "o.b", "q_norm": "q.norm", "k_norm": "k.norm", "q_conv": "q.conv",
                    "k_conv": "k.conv", "v_conv": "v.conv"}
_STATE_SPACE_NAMES = {"in_proj": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log",
                      "d_skip": "D", "out_norm": "norm", "o_proj": "o"}
_DELTA_NAMES = {"q_proj": "q", "k_proj": "k", "v_proj": "v", "g_proj": "g", "q_conv": "q.conv", "k_conv": "k.conv",
                "v_conv": "v.conv", "a_proj": "a", "b_proj": "b", "dt_bias": "dt_bias", "a_log": "A_log",
                "out_norm": "norm", "o_proj": "o"}


def _mixer(cfg: BarilixConfig, kind: str, m: dict, p: str, positions: dict[str, PartSpec]) -> PartSpec:
    if kind == "delta":
        return PartSpec(
            "gated_delta",
            dict(hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], key_dim=m["dim"],
                 value_dim=m["vdim"], conv_taps=m["conv"], norm_eps=cfg.norm_eps),
            {k: p + v for k, v in _DELTA_NAMES.items()})
    r = m["right"]
    right = PartSpec(
        "state_space",
        dict(hidden_size=cfg.width, num_heads=r["heads"], head_dim=r["vdim"], state_size=r["state"], groups=r["groups"],
             conv_taps=r["conv"], norm_parts=r["norm_groups"], norm_eps=cfg.norm_eps))
    names = {"left." + k: p + "left." + v for k, v in _ATTENTION_NAMES.items()}
    names.update({"right." + k: p + "right." + v for k, v in _STATE_SPACE_NAMES.items()})
    names.update({"left_out": p + "left.out", "right_out": p + "right.out"})
    return PartSpec("parallel_mixers",
                    dict(hidden_size=cfg.width, branches={"left": _attention(cfg, m["left"], positions), "right": right},
                         norm_eps=cfg.norm_eps),
                    names)


def _mlp(cfg: BarilixConfig, mlp: dict, p: str) -> PartSpec:
    if mlp["kind"] == "dense":
        return PartSpec("swiglu", dict(hidden_size=cfg.width, intermediate_size=mlp["ff"]),
                        {"gate_proj": p + "gate", "up_proj": p + "up", "down_proj": p + "down"})
    r, shared = mlp["router"], mlp["shared"]
    names = {"table": p + "table"}
    for e in range(r["experts"]):
        for t in ("gate", "up", "down"):
            names[f"e{e}_{t}"] = f"{p}e{e}.{t}"
    if shared:
        names.update({"shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down"})
    return PartSpec(
        "routed_experts",
        dict(hidden_size=cfg.width, experts=r["experts"], top=r["top"], intermediate_size=mlp["expert"]["ff"],
             router="table", unit="silu", vocab_size=cfg.vocab, shared=(shared["ff"],) if shared else None),
        names)


def barilix_plan(cfg: BarilixConfig) -> ModelPlan:
    positions: dict[str, PartSpec] = {}
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer": _mixer(cfg, layer.type, layer.mixer, p + "mix.", positions),
                 "mixer_post_norm": _norm(cfg, p + "norm1")}
        if layer.mlp is None:
            layers.append(LayerSpec("post_norm_mixer", parts))
            continue
        parts.update({"ffn": _mlp(cfg, layer.mlp, p + "mlp."), "ffn_post_norm": _norm(cfg, p + "norm2")})
        layers.append(LayerSpec("post_norm", parts))
    return ModelPlan(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, scale=cfg.embedding_scale),
                           {"weight": "embed"}),
        layers=tuple(layers),
        schedule=tuple(Run(i, i, True) for i in range(len(layers))),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "head"}),
        positions=positions,
        max_positions=None,
    )


register_architecture(BarilixConfig.architecture, BarilixConfig, barilix_plan)
