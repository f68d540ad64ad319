"""Several mixers side by side on the same input.

Every branch reads the same activations; the result is the mean of the branches' outputs, each
first normalised over the model width, ``u * rsqrt(mean(u^2) + eps) * w_b`` with a weight of
its own (float32, one kernel for all branches).  What the branches ask of the cache is put
together: at most one of them keeps paged keys and values, and their fixed-size states are
kept under ``<branch>.<name>``.
"""

from __future__ import annotations

import dataclasses

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView
from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Mixer, ParamSpec, build_part
from .plan import PartSpec


class ParallelMixers(Mixer):
    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, eps: float,
                 branches: dict[str, PartSpec], out_leaf: str = "out") -> None:
        """``branches``: name -> the branch's mixer; branch b's output weight is the tensor
        ``<prefix>.<b>.<out_leaf>``."""
        super().__init__(ctx, prefix)
        if not 1 <= len(branches) <= 4:
            raise ValueError("one to four mixers side by side")
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.out_leaf = out_leaf
        self.branches = {name: build_part("mixer", spec, ctx) for name, spec in branches.items()}
        self.out_weights: Tensor | None = None

    def _out_name(self, branch: str) -> str:
        return self.name(f"{branch}.{self.out_leaf}")

    def param_specs(self):
        specs = {self._out_name(b): ParamSpec((self.hidden_size,), kind="vector", init="norm") for b in self.branches}
        for mixer in self.branches.values():
            specs.update(mixer.param_specs())
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        for index, (branch, mixer) in enumerate(self.branches.items()):
            if name == self._out_name(branch):
                if self.out_weights is None:
                    self.out_weights = torch.zeros((len(self.branches), self.hidden_size), dtype=torch.float32,
                                                   device=tensor.device)
                self.out_weights[index].copy_(tensor)
                return
            if name in mixer.param_specs():
                mixer.set_param(name, tensor)
                return
        raise KeyError(name)

    def finalize(self) -> None:
        for mixer in self.branches.values():
            mixer.finalize()

    @property
    def graph_safe(self) -> bool:
        return all(mixer.graph_safe for mixer in self.branches.values())

    def cache_needs(self) -> CacheNeeds:
        paged, states = None, {}
        for branch, mixer in self.branches.items():
            needs = mixer.cache_needs()
            if needs.paged is not None:
                if paged is not None:
                    raise ValueError("only one of the mixers side by side may keep paged keys and values")
                paged = needs.paged
            for name, state in needs.states().items():
                states[f"{branch}.{name}"] = state
        return CacheNeeds(paged=paged, state=states or None)

    def forward(self, x: Tensor, batch, cache: CacheView | None, writes_cache: bool = True) -> Tensor:
        outputs = []
        for branch, mixer in self.branches.items():
            lead = branch + "."
            own = {n[len(lead):]: t for n, t in (cache.states if cache is not None else {}).items() if n.startswith(lead)}
            view = CacheView(states=own) if cache is None else dataclasses.replace(cache, states=own)
            outputs.append(mixer.forward(x, batch, view, writes_cache))
        out = torch.empty((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
        return ops.rmsnorm_mean(outputs, self.out_weights, self.eps, out)

    def token_inputs(self):
        asked = {}
        for mixer in self.branches.values():
            asked.update(mixer.token_inputs())
        return asked

    def kernel_libraries(self):
        names = {"stream_ops"}
        for mixer in self.branches.values():
            names |= mixer.kernel_libraries()
        return names


register_part("mixer", "parallel_mixers", ParallelMixers)
