"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * (offset + weight).

eps is added to the mean inside the root; sum, root and product are 32-bit
(v3/kernels/rmsnorm_inplace_f16.cu:29-62, v3/crates/rvllm-fused/src/reference.rs:58-76).
``unit_offset`` selects the zero-centred form of the Gemma checkpoints, where
the stored weight is the gain minus one.

``rmsnorm`` takes ``suffix`` (what the tensor's name is followed by, ``.weight`` if
absent).  Where the model keeps its residual stream in 32 bits and its
activations in bf16, the norm reads the one and writes the other.

``rmsnorm_scalar``: the same with one number as the gain of the whole row,
y = x * rsqrt(mean(x^2) + eps) * g.  Its input may be a residual stream that a
bf16 model keeps in 32 bits; the output has the activations' type.  ``suffix``
is what the tensor's name is followed by (``.weight`` if absent).

``layernorm``: y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias, all in 32-bit.  ``suffix`` follows
the weight's name (``.weight`` if absent) and ``bias_suffix`` the bias's (``.bias`` if absent).  Reads a 32-bit
stream or the activations' type, writes the activations' type.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Norm, ParamSpec, tensor_path
from .registry import NORMS
from .spec import PartSpec


class RMSNorm(Norm):
    def __init__(self, spec: PartSpec, *, width: int, name: str):
        self.width = int(width)
        self.name = name
        self.eps = float(spec["eps"])
        self.offset = 1.0 if spec.get("unit_offset", False) else 0.0
        self.suffix = str(spec.get("suffix", ".weight"))
        self.weight: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def _tensor_name(self, prefix: str) -> str:
        return tensor_path(prefix, self.name) + self.suffix

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [ParamSpec(self._tensor_name(prefix), (self.width,), init=("normal", 0.1))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        # The weight keeps the type it was loaded in (bf16, or 32-bit).
        self.weight = tensors[self._tensor_name(prefix)].to(device).contiguous()
        self.out_dtype = dtype

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if x.dtype != self.out_dtype:  # a 32-bit residual stream under bf16 activations
            return ops.rmsnorm_cast(x, self.weight, self.eps, self.offset, self.out_dtype, out=out)
        return ops.rmsnorm(x, self.weight, self.eps, self.offset, out=out)

    def forward_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        if x.dtype != self.out_dtype:
            return ops.rmsnorm_cast(x, self.weight, self.eps, self.offset, self.out_dtype, rows=rows)
        return ops.rmsnorm(x, self.weight, self.eps, self.offset, rows=rows)

    def add_into(self, branch, residual, then=None, then_out=None, scale=None):
        """``scale``: one learned number a channel that the normed branch is multiplied by before it is added."""
        if scale is not None or residual.dtype != self.out_dtype:
            # the general kernel: a 32-bit stream whatever the branch's type, an optional scale
            if residual.dtype != torch.float32:
                raise ValueError("a scaled branch is added to a 32-bit residual stream")
            if isinstance(then, RMSNorm):
                return ops.add_rmsnorm_scaled(branch, self.weight, self.eps, self.offset, scale, residual, then.weight,
                                              then.eps, then.offset)
            ops.add_rmsnorm_scaled(branch, self.weight, self.eps, self.offset, scale, residual)
            return then.forward(residual, out=then_out) if then is not None else None
        if then is None:
            return ops.add_rmsnorm(branch, self.weight, self.eps, self.offset, residual)
        if isinstance(then, RMSNorm):
            return ops.add_rmsnorm(branch, self.weight, self.eps, self.offset, residual, then.weight, then.eps,
                                   then.offset, then_out)
        ops.add_rmsnorm(branch, self.weight, self.eps, self.offset, residual)
        return then.forward(residual, out=then_out)


class ScalarRMSNorm(Norm):
    def __init__(self, spec: PartSpec, *, width: int, name: str):
        self.width = int(width)
        self.name = name
        self.eps = float(spec["eps"])
        self.suffix = str(spec.get("suffix", ".weight"))
        self.gain: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [ParamSpec(tensor_path(prefix, self.name) + self.suffix, (), init=("normal_about", 1.0, 0.1))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        self.gain = tensors[tensor_path(prefix, self.name) + self.suffix].to(device).reshape(1).contiguous()
        self.out_dtype = dtype

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.scalar_rmsnorm(x, self.gain, self.eps, self.out_dtype, out=out)

    def forward_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.scalar_rmsnorm(x, self.gain, self.eps, self.out_dtype, rows=rows)


class LayerNorm(Norm):
    def __init__(self, spec: PartSpec, *, width: int, name: str):
        self.width = int(width)
        self.name = name
        self.eps = float(spec["eps"])
        self.suffix = str(spec.get("suffix", ".weight"))
        self.bias_suffix = str(spec.get("bias_suffix", ".bias"))
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = tensor_path(prefix, self.name)
        return [ParamSpec(at + self.suffix, (self.width,), init=("normal_about", 1.0, 0.1)),
                ParamSpec(at + self.bias_suffix, (self.width,), init=("normal", 0.1))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = tensor_path(prefix, self.name)
        self.weight = tensors[at + self.suffix].to(device=device, dtype=torch.float32).contiguous()
        self.bias = tensors[at + self.bias_suffix].to(device=device, dtype=torch.float32).contiguous()
        self.out_dtype = dtype

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.layernorm(x, self.weight, self.bias, self.eps, self.out_dtype, out=out)

    def forward_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.layernorm(x, self.weight, self.bias, self.eps, self.out_dtype, rows=rows)


NORMS.register("rmsnorm", RMSNorm)
NORMS.register("layernorm", LayerNorm)
NORMS.register("rmsnorm_scalar", ScalarRMSNorm)
