"""RMS norm (/root/reference/core/src/nn/norm.cpp:25-42), whole rows or in groups."""
from __future__ import annotations

from .. import ops
from .base import Part, register_part
from .spec import PartSpec, TensorSpec


def rmsnorm_spec(weight_name: str, width: int, eps: float, groups: int = 1, offset: float = 0.0) -> PartSpec:
    """``groups`` > 1: the row is cut into that many equal consecutive parts and each is divided by
    its own root mean square; the weight spans the whole row.  ``offset``: what is added to the
    stored weight (1 for weights that are kept around zero)."""
    return PartSpec("norm", "rmsnorm", {"width": width, "eps": float(eps), "groups": int(groups), "offset": float(offset)},
                    {"weight": TensorSpec(weight_name, (width,), init=(1.0 - float(offset), 0.02))})


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """y = (x * 1/sqrt(mean(x^2) + eps)) * (offset + w); the weight multiplies as it is unless the
    spec gives an offset.  With ``groups`` the mean is taken over each of that many consecutive parts
    of the row."""
    category = "norm"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.groups = int(spec.params.get("groups", 1) or 1)
        if self.groups < 1 or self.width % self.groups:
            raise ValueError(f"{self.groups} groups do not divide a row of {self.width}")
        self.offset = float(spec.params.get("offset", 0.0) or 0.0)
        if self.offset and self.groups != 1:
            raise ValueError("a norm with an offset on its weight takes whole rows")
        # a projection's last pass may apply this norm (it exposes weight, eps and groups); the fused
        # passes multiply by the weight as it is
        self.fusable = self.offset == 0.0
        self.weight = tensors.get("weight")

    def forward(self, x, out_dtype, rows=None):
        if self.offset:
            return ops.offset_norm(x, self.weight, self.eps, self.offset, out_dtype, rows)
        return ops.rmsnorm(x, self.weight, self.eps, out_dtype, rows, groups=self.groups)
