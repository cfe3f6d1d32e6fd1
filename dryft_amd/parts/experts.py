"""Routed experts: every row goes through a few of many small feed-forwards, and through a shared one.

Router: ``z = W_router h`` and ``s = sigmoid(z)`` in float32. A row's *choice scores* are ``s + correction``; its
weights use ``s`` without the correction. Experts form ``count`` equal groups of neighbours; a group's score is the
sum of its two largest choice scores, and only experts of the ``keep`` best groups can be chosen (the others drop
out, whatever sign their scores have). The ``top`` largest choice scores that remain are the row's experts, with
weights ``s_e / (sum of the chosen s + 1e-20) * route_scale``. An expert is a clamped gated unit,
``down(g * sigmoid(alpha g) * (u + 1))`` with ``g = min(gate(h), limit)``, ``u = clamp(up(h), -limit, limit)``. The
shared expert, of the same form with sizes of its own, runs for every row and is added times ``sigmoid(w_s . h)``.

Other forms, by constructor arguments. ``router="table"``: no scores at all; an integer table ``[vocab, top]`` (the
entries of a row differ) names each token id's experts, every one with weight ``1 / top`` (the step's token ids come
with the step context). ``unit="silu"``: an expert is ``down(silu(gate(h)) * up(h))``, nothing clamped, and so is
the shared expert, which is then added as it is.

``score="softmax"``: the scores are the softmax of ``z`` over all experts; ``correction=False``: no correction, the
scores themselves decide; ``group_score="best"``: a group scores as its best expert; ``renormalize=False``: the weights
are the chosen scores times ``route_scale`` as they are; ``shared_gate=False``: the shared expert is added as it is.
``unit="relu2"``: an expert has no gate, ``down(relu(up(h))^2)``, and so has the shared expert.

On the device throughout, so a step can be captured: the router picks, a small kernel sorts the (row, expert) pairs
by expert and cuts each expert's run into tiles, and two grouped products walk the tiles (gate/up with the unit in
the epilogue, then down); a last kernel adds each row's weighted outputs and the shared expert in a fixed order.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from ..weights.spec import INT_TABLE, VECTOR
from . import register_part
from .base import FeedForward, Partials, matrix
from .linear import linear
from .mlp import ClampedGLU, SquaredReLU, SwiGLU


class RoutedExperts(FeedForward):
    def __init__(self, hidden_size: int, experts: int, top: int, intermediate_size: int, limit: float | None = None,
                 route_scale: float = 1.0, groups: tuple[int, int] | None = None,
                 shared: tuple | None = None, alpha: float = 1.702, router: str = "scores", unit: str = "clamped",
                 vocab_size: int | None = None, score: str = "sigmoid", correction: bool = True,
                 group_score: str = "top2", renormalize: bool = True, shared_gate: bool = True):
        self.hidden, self.n_experts, self.top, self.inter = int(hidden_size), int(experts), int(top), int(intermediate_size)
        if router not in ("scores", "table") or unit not in ("clamped", "silu", "relu2"):
            raise ValueError(f"router is 'scores' or 'table', unit 'clamped', 'silu' or 'relu2'; got {router!r}, {unit!r}")
        if score not in ("sigmoid", "softmax") or group_score not in ("top2", "best"):
            raise ValueError(f"score is 'sigmoid' or 'softmax', group_score 'top2' or 'best'; got {score!r}, {group_score!r}")
        self.score, self.has_correction, self.group_score = score, bool(correction), group_score
        self.renormalize, self.shared_gate = bool(renormalize), bool(shared_gate) and router == "scores"
        self.gated = unit != "relu2"
        if router == "table" and not vocab_size:
            raise ValueError("a table router needs the vocabulary's size")
        if unit == "clamped" and limit is None:
            raise ValueError("the clamped unit needs its limit")
        self.router, self.unit, self.vocab = router, unit, int(vocab_size or 0)
        # the gated unit as the kernels take it: (limit, slope of the sigmoid, what is added to the up branch)
        self.glu = (float(limit), float(alpha), 1.0) if unit == "clamped" else (float("inf"), 1.0, 0.0)   # gated units only
        self.limit, self.alpha, self.route_scale = limit, float(alpha), float(route_scale)
        if not 1 <= self.top <= self.n_experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"1 <= top <= experts <= {ops.MOE_MAX_EXPERTS}, got top {top} of {experts}")
        self.groups = (int(groups[0]), int(groups[1])) if groups else (1, 1)
        count, keep = self.groups
        if self.n_experts % count or not 1 <= keep <= count or count > 64 or keep * (self.n_experts // count) < self.top:
            raise ValueError(f"{experts} experts in {count} groups of which {keep} are kept cannot give {top}")
        self.shared = None
        if shared:
            self.shared = ClampedGLU(hidden_size, shared[0], shared[1], alpha) if unit == "clamped" else \
                SwiGLU(hidden_size, shared[0]) if unit == "silu" else SquaredReLU(hidden_size, shared[0])
        self.w_router = self.correction = self.w_gate_up = self.w_down = self.table = None

    def tensor_specs(self):
        if self.router == "table":
            specs = {"table": ((self.vocab, self.top), INT_TABLE, f"distinct<{self.n_experts}")}
        else:
            specs = {"router": matrix((self.n_experts, self.hidden))}
            if self.has_correction:
                specs["correction"] = ((self.n_experts,), VECTOR, "zeros")
        for e in range(self.n_experts):
            if self.gated:
                specs[f"e{e}_gate"] = matrix((self.inter, self.hidden))
            specs[f"e{e}_up"] = matrix((self.inter, self.hidden))
            specs[f"e{e}_down"] = matrix((self.hidden, self.inter))
        if self.shared is not None:
            specs.update({"shared_" + k.split("_")[0]: v for k, v in self.shared.tensor_specs().items()})
            if self.shared_gate:
                specs["shared_weight"] = matrix((1, self.hidden))
        return specs

    def load(self, tensors):
        E = self.n_experts
        if self.gated:
            self.w_gate_up = torch.stack([torch.cat([tensors[f"e{e}_gate"], tensors[f"e{e}_up"]], dim=0) for e in range(E)]).contiguous()
        else:
            self.w_gate_up = torch.stack([tensors[f"e{e}_up"] for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors[f"e{e}_down"] for e in range(E)]).contiguous()
        if self.shared is not None:
            self.shared.compute_dtype = self.compute_dtype
            self.shared.load({k + "_proj": tensors["shared_" + k] for k in (("gate", "up", "down") if self.gated else ("up", "down"))})
        if self.router == "table":
            self.table = tensors["table"].to(torch.int32).contiguous()
            if self.table.numel() and not (0 <= int(self.table.min()) and int(self.table.max()) < E):
                raise ValueError(f"the experts' table names experts outside 0..{E - 1}")
            return
        if self.has_correction:
            self.correction = tensors["correction"].float().contiguous()
        router = [tensors["router"]]
        if self.shared is not None and self.shared_gate:
            router.append(tensors["shared_weight"])
        self.w_router = torch.cat(router, dim=0).contiguous()          # the shared expert's weight is one more logit

    def kernel_modules(self, dtype):
        return ("gemm", "activation", "moe")

    def forward(self, h, ctx):
        rows, E, top = h.shape[0], self.n_experts, self.top
        dev = h.device
        chosen = torch.empty((rows, top), dtype=torch.int32, device=dev)
        weights = torch.empty((rows, top), dtype=torch.float32, device=dev)
        logits = None
        if self.router == "table":
            ops.moe_table_route(ctx.tokens, self.table, E, chosen, weights)
        else:
            logits = linear(h, self.w_router, out_dtype=torch.float32)
            ops.moe_route(logits, self.correction, E, self.groups[0], self.groups[1], self.route_scale, chosen, weights,
                          softmax=self.score == "softmax", group_best=self.group_score == "best",
                          renorm=self.renormalize)
        plan = ops.moe_plan(chosen, E)
        act = torch.empty((rows * top, self.inter), dtype=h.dtype, device=dev)
        if self.gated:
            ops.moe_products(h, self.w_gate_up, plan, act, top, glu=self.glu)
        else:
            ops.moe_products(h, self.w_gate_up, plan, act, top, act="relu2")
        y = torch.empty((rows * top, self.hidden), dtype=torch.float32, device=dev)
        ops.moe_products(act, self.w_down, plan, y, 0)
        shared = None
        if self.shared is not None:
            shared = self.shared.forward(h, ctx)
            if isinstance(shared, Partials):
                shared = shared.summed(h.dtype)
        out = torch.empty((rows, self.hidden), dtype=h.dtype, device=dev)
        ops.moe_combine(y, plan, weights, shared, logits if self.shared_gate else None, E, out)
        return out

    def reads_whole(self) -> bool:
        return True

    def flops(self, rows, spans):
        per_row = (6.0 if self.gated else 4.0) * self.top * self.inter * self.hidden
        if self.router == "scores":
            per_row += 2.0 * self.hidden * (self.n_experts + 1)
        if self.shared is not None:
            per_row += (6.0 if self.gated else 4.0) * self.shared.inter * self.hidden
        return rows * per_row


register_part("routed_experts", RoutedExperts)
