"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root (src/vec_ops.rs:500-522
of yusiwen/minfer; the three places it stands in the layer, src/models/qwen2/graph.rs:63,
155,180).  Statistics in 32-bit over the float32 residual stream."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Norm, register_norm
from .spec import PartSpec


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """params: size, eps, weight (tensor name)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.size, self.eps, self.name = int(spec.params["size"]), float(spec.params["eps"]), spec.params["weight"]
        self.weight = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.size,), init="ones")}

    def load(self, get):
        self.weight = get(self.name).to(torch.float32).contiguous()

    def rms_scale(self):
        return self.weight, self.eps

    def forward(self, h, out: Optional[torch.Tensor] = None, row_idx: Optional[torch.Tensor] = None):
        rows = h.shape[0] if row_idx is None else row_idx.numel()
        if out is None:
            out = torch.empty((rows, self.size), dtype=self.rt.dtype, device=h.device)
        ops.rmsnorm(h, self.weight, self.eps, out, row_idx)
        return out


@register_norm("group_rmsnorm")
class GroupRMSNorm(Norm):
    """RMS norm taken over `groups` equal consecutive parts of the vector: each part is divided by
    its own sqrt(mean(part^2) + eps), then the whole is multiplied by the weight.  One group is the
    plain RMS norm.  params: size, eps, groups, weight (tensor name)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.size, self.eps, self.groups = int(p["size"]), float(p["eps"]), int(p.get("groups", 1))
        self.name = p["weight"]
        if self.groups < 1 or self.size % self.groups:
            raise ValueError(f"group_rmsnorm: {self.size} values do not split into {self.groups} equal parts")
        self.weight = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.size,), init="ones")}

    def load(self, get):
        self.weight = get(self.name).to(torch.float32).contiguous()

    def rms_scale(self):
        return (self.weight, self.eps) if self.groups == 1 else None

    def forward(self, h, out: Optional[torch.Tensor] = None, row_idx: Optional[torch.Tensor] = None):
        rows = h.shape[0] if row_idx is None else row_idx.numel()
        if out is None:
            out = torch.empty((rows, self.size), dtype=self.rt.dtype, device=h.device)
        ops.group_rmsnorm(h, self.weight, self.eps, self.groups, out, row_idx)
        return out

    def add_normed(self, y, h, cast_out: Optional[torch.Tensor] = None) -> None:
        """h += norm(y) in one kernel; `cast_out` (bfloat16) also gets the new rows rounded."""
        ops.group_rmsnorm(y, self.weight, self.eps, self.groups, h, add=True, cast_out=cast_out)


@register_norm("scalar_rmsnorm")
class ScalarRMSNorm(RMSNorm):
    """RMS norm with one gain for the whole vector: x / sqrt(mean(x^2) + eps) * g, g a tensor of a single
    number.  Kept as a vector of equal gains, so every kernel and fold of `rmsnorm` serves it.
    params: size, eps, weight (tensor name)."""

    def tensor_specs(self):
        return {self.name: TensorSpec((), init="ones")}

    def load(self, get):
        g = get(self.name).to(torch.float32).reshape(1)
        self.weight = g.expand(self.size).contiguous()


@register_norm("offset_rmsnorm")
class OffsetRMSNorm(GroupRMSNorm):
    """RMS norm whose gain is one plus the stored weight: x / sqrt(mean(x^2) + eps) * (1 + w).  The gain 1 + w is
    formed once, in 32-bit, when the weights arrive, so every kernel and fold of the plain norm serves it,
    also the one that adds a normed branch result into the stream.  params: size, eps, weight (tensor name)."""

    def __init__(self, spec, rt):
        super().__init__(PartSpec(spec.kind, dict(spec.params, groups=1)), rt)

    def tensor_specs(self):
        return {self.name: TensorSpec((self.size,), init="zeros")}

    def load(self, get):
        self.weight = (get(self.name).to(torch.float32) + 1.0).contiguous()
