"""Two mixers side by side: both read the same input, and their outputs add into the stream
(each scaled by its own constant, which the mixers apply themselves)."""

from __future__ import annotations

import torch

from kvforge_amd.parts.base import CacheSpec, LayerState, Mixer, Part, StateSpec, WeightSpec
from kvforge_amd.registry import register_mixer


@register_mixer("pair")
class MixerPair(Mixer):
    """``left`` and ``right`` are whole mixers with prefixes of their own.  A call has one set of
    pages and one state slot, so at most one of the two may keep pages (``cache_spec``) and at
    most one a state (``state_spec``): attention beside a recurrence, say.  Each is handed the
    call's ``LayerState`` and takes from it what it declared."""

    def __init__(self, left: Mixer, right: Mixer) -> None:
        self.left, self.right = left, right
        if left.cache_spec is not None and right.cache_spec is not None:
            raise ValueError("two mixers side by side: only one of them may keep pages")
        if left.state_spec is not None and right.state_spec is not None:
            raise ValueError("two mixers side by side: only one of them may keep a state")

    @property
    def cache_spec(self) -> CacheSpec | None:
        return self.left.cache_spec if self.left.cache_spec is not None else self.right.cache_spec

    @property
    def state_spec(self) -> StateSpec | None:
        return self.left.state_spec if self.left.state_spec is not None else self.right.state_spec

    @property
    def replayable(self) -> bool:
        return self.left.replayable and self.right.replayable

    def _both(self) -> tuple[Part, Part]:
        return self.left, self.right

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {**self.left.weight_specs(), **self.right.weight_specs()}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        for m in self._both():
            m.load(tensors)

    def seal(self) -> None:
        for m in self._both():
            m.seal()

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return self.left.kernel_modules(dtype) | self.right.kernel_modules(dtype)

    def num_bytes(self) -> int:
        return self.left.num_bytes() + self.right.num_bytes()

    def held_tensors(self) -> list[torch.Tensor]:
        return self.left.held_tensors() + self.right.held_tensors()

    def launch_key(self, shape):
        return self.left.launch_key(shape), self.right.launch_key(shape)

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations.  What the first leaves owed to the stream the second
        settles (or takes along) as any part does."""
        self.left.forward(x, step, layer, residual)
        self.right.forward(x, step, layer, residual)
