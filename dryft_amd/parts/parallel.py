"""Two mixers side by side on the same input.

Both read the same rows ``h``. Each one's output is divided by its root mean square over the model width (``eps``
inside the root) and multiplied by a weight of its own (``<name>_out``); the result is half the sum of the two. The
two mixers are ordinary parts, named in the plan by their own ``PartSpec``; what each keeps per sequence (keys and
values, fixed-size state) is handed to it under its name, so one cache line holds both.

The norms and the mean are float arithmetic and come out as float32 (one launch, which also adds up the partial sums
of the branches' last products and a branch's output bias on its way in).
"""

from __future__ import annotations

import torch

from ..csrc import ops
from ..weights.spec import VECTOR
from . import build_part, register_part
from .base import Mixer, Partials, StepContext


class ParallelMixer(Mixer):
    def __init__(self, hidden_size: int, branches: dict, norm_eps: float):
        """``branches``: two names, each with the ``PartSpec`` of a mixer (its ``tensors`` are not used here: this part's
        logical names are ``<branch>.<the mixer's own name>``, and ``<branch>_out`` for the weight after it)."""
        self.hidden, self.norm_eps = int(hidden_size), float(norm_eps)
        if len(branches) != 2:
            raise ValueError(f"two mixers side by side, got {list(branches)}")
        self.names = list(branches)
        self.mixers = {name: build_part(spec) for name, spec in branches.items()}
        self.out_weight: dict[str, torch.Tensor] = {}

    def _sub(self, name: str, mapping: dict) -> dict:
        return {k[len(name) + 1:]: v for k, v in mapping.items() if k.startswith(name + ".")}

    def tensor_specs(self):
        specs = {}
        for name, mixer in self.mixers.items():
            specs.update({f"{name}.{k}": v for k, v in mixer.tensor_specs().items()})
            specs[f"{name}_out"] = ((self.hidden,), VECTOR, "ones")
        return specs

    def load(self, tensors):
        for name, mixer in self.mixers.items():
            mixer.compute_dtype = self.compute_dtype
            mixer.load(self._sub(name, tensors))
            self.out_weight[name] = tensors[f"{name}_out"].float().contiguous()

    def cache_need(self):
        need = {}
        for name, mixer in self.mixers.items():
            one = mixer.cache_need()
            if isinstance(one, dict):
                need.update({f"{name}.{k}": v for k, v in one.items()})
            elif one is not None:
                need[name] = one
        return need

    def _line(self, name: str, line: dict):
        if name in line:
            return line[name]
        return self._sub(name, line) or None

    def kernel_modules(self, dtype):
        mods = {"norm"}
        for mixer in self.mixers.values():
            mods.update(mixer.kernel_modules(dtype))
        return tuple(sorted(mods))

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        outs = []
        for name in self.names:
            delta, bias = self.mixers[name].forward_split(h, ctx, self._line(name, line), writes_cache)
            outs += [(delta.data, delta.count) if isinstance(delta, Partials) else delta, bias, self.out_weight[name]]
        out = torch.empty((1, h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
        ops.rms_pair_mean(*outs, self.norm_eps, out[0], h.dtype)
        return Partials(out, 1)                # float32, for the norm that takes it into the stream

    def reads_whole(self) -> bool:
        return True

    def flops(self, rows, spans):
        return sum(m.flops(rows, spans) for m in self.mixers.values())


register_part("parallel_mixers", ParallelMixer)
