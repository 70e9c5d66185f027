"""RMS norm over the fp32 residual stream (src/tokenvault/model.py:28-38)."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import Norm, WeightSpec
from kvforge_amd.registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """``y = x * rsqrt(mean(x^2) + eps) * weight`` in fp32, rounded once to the output type."""

    replayable = True

    def __init__(self, prefix: str, width: int, eps: float) -> None:
        self.prefix, self.width, self.eps = prefix, int(width), float(eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self._name("weight"): WeightSpec((self.width,), init="norm", std=0.1)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self._name("weight")]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}

    def num_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size() if self.weight is not None else 0

    def held_tensors(self) -> list[torch.Tensor]:
        return [] if self.weight is None else [self.weight]

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: torch.Tensor | None = None,
                add: torch.Tensor | None = None) -> None:
        ops.rmsnorm(x, self.weight, self.eps, out, rows, add)

    def add_to(self, stream: torch.Tensor, y: torch.Tensor) -> None:
        if self.weight.dtype != torch.float32:
            self.weight = self.weight.float()    # the kernel multiplies by an fp32 vector
        ops.rms_add(stream, y, self.weight, self.eps)

    def fp32_weight(self) -> torch.Tensor | None:
        """The weight vector as the fused kernels take it (fp32, as it multiplies), or ``None``
        for a norm that is not a plain ``x * rsqrt(mean(x^2) + eps) * weight`` with such a weight."""
        if type(self).forward is not RMSNorm.forward or self.weight is None or self.weight.dtype != torch.float32:
            return None
        return self.weight

    def foldable_into(self, matrix: torch.Tensor) -> bool:
        """Whether this norm's weight may be multiplied into the columns of a bf16 matrix: only
        when it is itself held in bf16 (a weight stored in 32-bit stays a 32-bit multiply)."""
        return (self.weight is not None and self.weight.dtype == torch.bfloat16
                and matrix.dtype == torch.bfloat16 and matrix.shape[1] == self.width)


@register_norm("rmsnorm_one_plus")
class OnePlusRMSNorm(RMSNorm):
    """RMS norm whose stored weight lies around zero: ``y = x * rsqrt(mean(x^2) + eps) * (1 + w)``.
    The checkpoint holds ``w [width]`` under ``name``; ``1 + w`` is formed once at load in fp32
    and kept in fp32, which is what the norm kernels multiply by."""

    def __init__(self, name: str, width: int, eps: float) -> None:
        super().__init__("", width, eps)
        self.name = name

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.width,), init="normal", std=0.1)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.weight = (1.0 + tensors[self.name].float()).contiguous()

    def foldable_into(self, matrix: torch.Tensor) -> bool:
        return False


@register_norm("rmsnorm_named")
class NamedRMSNorm(RMSNorm):
    """RMS norm with a plain weight vector that the checkpoint holds under ``name`` (the whole
    name, no ``.weight`` behind it).  The weight is kept in fp32, so the product with it is a
    32-bit one in every mode."""

    def __init__(self, name: str, width: int, eps: float) -> None:
        super().__init__("", width, eps)
        self.name = name

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.width,), init="norm", std=0.1)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name].float().contiguous()

    def foldable_into(self, matrix: torch.Tensor) -> bool:
        return False


@register_norm("rmsnorm_scalar")
class ScalarRMSNorm(RMSNorm):
    """RMS norm whose gain is one number for all coordinates: ``y = x * rsqrt(mean(x^2) + eps) * g``.
    The checkpoint holds ``g`` as a tensor without dimensions under ``name``; it is kept as an
    fp32 vector of ``width`` equal entries, which is what the norm kernels multiply by."""

    def __init__(self, name: str, width: int, eps: float) -> None:
        super().__init__("", width, eps)
        self.name = name

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.name: WeightSpec((), init="norm", std=0.1)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        g = tensors[self.name]
        self.weight = g.float().reshape(1).expand(self.width).contiguous()

    def foldable_into(self, matrix: torch.Tensor) -> bool:
        return False
