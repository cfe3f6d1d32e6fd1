"""Podenex: from ``PodenexConfig`` to a model plan.

A decoder on a float32 residual stream with a layer norm (a weight, no bias) in front of every sublayer and none
behind it: ``x <- x + mixer(norm1(x))``, ``x <- x + ff(norm2(x))``, and then what the token id brings to the layer,
``x <- x + rms(W_proj (gelu_tanh(W_gate x) * e)) * w`` with ``e`` the layer's run of columns of a second embedding
table. A layer's mixer is one of three kinds of attention, none of which sees all earlier keys:

* ``attention``: grouped queries, a short causal convolution on q, k and v straight after the projection, no
  rotation; a learned bias by distance on the scaled score; chunks (a row sees the earlier keys of its own run of
  ``mask.size`` positions, counted from position 0); one output gate per head, ``sigmoid(W_g h)``;
* ``attention_2``: grouped queries with biases on all four projections, an rms norm per head on q and k with one
  weight for all heads, no positions at all, a sliding window, and a softmax with ``1`` added to its denominator;
* ``latent_attention``: queries and keys/values through normed low-rank latents, one rotated key part shared by all
  heads (neighbouring features turn together), a sliding window, a gate on every output feature.

Layers of the first two kinds that say ``v_mix`` share values: the first of them computes its values as usual, every
later one takes ``(1 - l) v + l v_first`` with a learned ``l`` before it caches them. The feed-forward is routed
experts without gates, ``down(relu(up(h))^2)``: softmax scores over all experts, groups of neighbours that score as
their best expert, the ``top`` best experts of the best ``keep`` groups, weighted by their scores as they are, plus a
shared expert of the same form. A final layer norm and an output head of its own.

What the design fixes rather than the file: ``gelu_tanh``, the squared relu, the sink's score 0, the bias table's
split into an exact and a logarithmic half. Checkpoint names: ``embed``, ``side.embed``, ``head``, ``final.norm`` and
per layer ``l<i>.norm1``, ``norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.side.{gate,proj,norm}``.
"""

from __future__ import annotations

from ..config.plan import LayerSpec, ModelPlan, PartSpec, Run
from ..config.podenex import PodenexConfig
from . import register_architecture

VALUES = "v_mix"        # the name under which the layers that share values find the first one's


def _norm(cfg: PodenexConfig, name: str) -> PartSpec:
    return PartSpec("stream_layernorm", dict(size=cfg.width, eps=cfg.norm_eps), {"weight": name})


def _grouped(cfg: PodenexConfig, kind: str, m: dict, p: str, first_mix: bool) -> PartSpec:
    args = dict(hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"],
                value_dim=m["vdim"], scale=m["scale"], float_weights=True, pad_pages=True,
                value_mix=(VALUES, first_mix) if m["v_mix"] else None)
    names = {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "o_proj": p + "o"}
    if m["v_mix"]:
        names["vmix"] = p + "vmix"
    size = m["mask"]["size"] if m["mask"] else None
    if kind == "attention":
        args.update(chunk=size, conv_taps=m["conv"] or None, output_gate="head",
                    distance_bias=(m["bias_rows"] or -1, m["bias_max"]) if m["bias_max"] else None)
        names["g_proj"] = p + "g"
        if m["conv"]:
            names.update({"q_conv": p + "q.conv", "k_conv": p + "k.conv", "v_conv": p + "v.conv"})
        if m["bias_max"]:
            names["rel"] = p + "rel"
    else:
        args.update(window=size, bias=True, qk_norm_eps=cfg.norm_eps, sink_value=0.0)
        names.update({"q_bias": p + "q.b", "k_bias": p + "k.b", "v_bias": p + "v.b", "o_bias": p + "o.b",
                      "q_norm": p + "q.norm", "k_norm": p + "k.norm"})
    return PartSpec("gqa_attention", args, names)


def _latent(cfg: PodenexConfig, m: dict, p: str, positions: dict[str, PartSpec]) -> PartSpec:
    rot, name = m["rot"], None
    if rot is not None:
        spec = PartSpec("pair_rotary", dict(dims=rot["dims"], base=rot["base"]))
        name = next((n for n, s in positions.items() if s == spec), None)     # layers with equal rotations share tables
        if name is None:
            name = f"rotary{len(positions)}"
            positions[name] = spec
    return PartSpec(
        "latent_attention",
        dict(hidden_size=cfg.width, num_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], value_dim=m["vdim"],
             q_rank=m["q_rank"], kv_rank=m["kv_rank"], scale=m["scale"], positions=name,
             window=m["mask"]["size"] if m["mask"] else None, norm_eps=cfg.norm_eps, sink=False, gate="element"),
        {"q_down": p + "dq", "q_norm": p + "dq.norm", "q_up": p + "uq", "kv_down": p + "dkv", "kv_norm": p + "dkv.norm",
         "k_up": p + "uk", "v_up": p + "uv", "g_proj": p + "g", "o_proj": p + "o"})


def _mlp(cfg: PodenexConfig, mlp: dict, p: str) -> PartSpec:
    r, shared = mlp["router"], mlp["shared"]
    names = {"router": p + "router"}
    for e in range(r["experts"]):
        names[f"e{e}_up"] = f"{p}e{e}.up"
        names[f"e{e}_down"] = f"{p}e{e}.down"
    if shared:
        names.update({"shared_up": p + "shared.up", "shared_down": p + "shared.down"})
    return PartSpec(
        "routed_experts",
        dict(hidden_size=cfg.width, experts=r["experts"], top=r["top"], intermediate_size=mlp["expert"]["ff"],
             groups=(r["groups"]["count"], r["groups"]["keep"]) if r["groups"] else None,
             shared=(shared["ff"],) if shared else None, unit="relu2", score="softmax", correction=False,
             group_score="best", renormalize=False, shared_gate=False),
        names)


def podenex_plan(cfg: PodenexConfig) -> ModelPlan:
    positions: dict[str, PartSpec] = {}
    layers = []
    mixing_seen = False
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        if layer.type == "latent_attention":
            mixer = _latent(cfg, m, p + "mix.", positions)
        else:
            mixer = _grouped(cfg, layer.type, m, p + "mix.", first_mix=not mixing_seen)
            mixing_seen = mixing_seen or m["v_mix"]
        parts = {"mixer_norm": _norm(cfg, p + "norm1"), "mixer": mixer}
        block = "pre_norm_mixer"
        if layer.mlp is not None:
            parts.update({"ffn_norm": _norm(cfg, p + "norm2"), "ffn": _mlp(cfg, layer.mlp, p + "mlp.")})
            block = "pre_norm"
        if cfg.side_dim:
            parts["side"] = PartSpec(
                "token_side", dict(hidden_size=cfg.width, dim=cfg.side_dim, index=i, count=len(cfg.layers),
                                   vocab_size=cfg.vocab, eps=cfg.norm_eps),
                {"table": "side.embed", "gate": p + "side.gate", "proj": p + "side.proj", "norm": p + "side.norm"})
            block += "_side"
        layers.append(LayerSpec(block, parts))
    return ModelPlan(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "embed"}),
        layers=tuple(layers),
        schedule=tuple(Run(i, i, True) for i in range(len(layers))),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "head"}),
        positions=positions,
        max_positions=None,
    )


register_architecture(PodenexConfig.architecture, PodenexConfig, podenex_plan)
