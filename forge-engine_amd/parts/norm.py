"""RMSNorm over the residual stream, fused with the add of the pending update.

``y = sum * rsqrt(mean(sum^2) + eps) * w`` with ``sum = h + update``
(reference: src/forge_engine/qwen3.py:99-105 and kernels/__init__.py:12-26).
The reference rounds the normalised value to the model dtype before the weight
product; here the whole expression is float32 with one rounding at the store.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Norm, ParamSpec, Residual


class RMSNorm(Norm):
    def __init__(self, ctx: BuildContext, prefix: str, *, size: int, eps: float, leaf: str = "weight") -> None:
        """``leaf``: the weight's name behind the prefix ("": the prefix itself is the name)."""
        super().__init__(ctx, prefix)
        self.size = size
        self.eps = float(eps)
        self.leaf = leaf
        self.weight: Tensor | None = None

    def param_specs(self):
        return {self.name(self.leaf): ParamSpec((self.size,), kind="vector", init="norm")}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name != self.name(self.leaf):
            raise KeyError(name)
        self.weight = tensor

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        if rows is not None:    # the chosen rows of stream + pending update; both are left as they are
            h = residual.h
            out = torch.empty((rows.numel(), self.size), dtype=self.ctx.dtype, device=h.device)
            return ops.add_rmsnorm(h, residual.pending, self.weight, self.eps, out, rows=rows, store_sum=False)
        update, residual.pending = residual.pending, None
        out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
        return ops.add_rmsnorm(residual.h, update, self.weight, self.eps, out)

    def kernel_libraries(self):
        return {"rowwise"}


class UpdateRMSNorm(RMSNorm):
    """RMSNorm of a sublayer's output instead of its input: the pending update u is normalised,
    ``u * rsqrt(mean(u^2) + eps) * w``, and added into the stream, all in float32 and in one
    kernel.  Returns the new stream in the compute dtype (what the next sublayer reads: the
    sublayers of such a layer see the stream itself)."""

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        if rows is not None:
            raise ValueError("a norm of updates serves whole steps, not chosen rows")
        update, residual.pending = residual.pending, None
        if update is None:
            raise ValueError("a norm of updates needs a pending update")
        out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
        return ops.rmsnorm_update(residual.h, update, self.weight, self.eps, out)

    def kernel_libraries(self):
        return {"rowwise", "stream_ops"}


register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "rms_norm_of_update", UpdateRMSNorm)
