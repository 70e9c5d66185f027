"""Token embedding and the output head (src/tokenvault/model.py:153-158,169-170,190-191)."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import Embedding, Head, WeightSpec


class TokenEmbedding(Embedding):
    """``h0 = table[ids] * scale`` into the fp32 residual stream (the product in fp32; ``scale``
    1 by default).  ``tensor``: the table's whole checkpoint name where it is not
    ``<prefix>.weight``."""

    replayable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, tensor: str | None = None,
                 scale: float = 1.0) -> None:
        self.prefix, self.vocab, self.hidden = prefix, int(vocab), int(hidden)
        self.scale = float(scale)
        self.tensor = tensor if tensor is not None else self._name("weight")
        self.table: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.tensor: WeightSpec((self.vocab, self.hidden))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.tensor]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}

    def held_tensors(self) -> list[torch.Tensor]:
        return [] if self.table is None else [self.table]

    def forward(self, ids: torch.Tensor, out: torch.Tensor) -> None:
        ops.embed(ids, self.table, out, self.scale)

    def pick_table(self) -> torch.Tensor | None:
        t = self.table
        return t if t is not None and t.dtype == torch.bfloat16 and self.scale == 1.0 else None


class LMHead(Head):
    """``logits = x @ W^T`` in fp32 output.  ``tied_to``: the checkpoint name of the embedding
    table when the head shares it (then no tensor of its own is expected).  ``tensor``: the
    matrix's whole checkpoint name where it is not ``<prefix>.weight``.  ``scale``: the logits are
    multiplied by it.  ``softcap``: the (scaled) logits become ``softcap * tanh(logits /
    softcap)`` (``None``: as they are)."""

    replayable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, tied_to: str | None = None,
                 tensor: str | None = None, softcap: float | None = None, scale: float = 1.0) -> None:
        self.prefix, self.vocab, self.hidden, self.tied_to = prefix, int(vocab), int(hidden), tied_to
        self.softcap = float(softcap) if softcap else None
        self.scale = float(scale)
        if not self.scale > 0.0:
            raise ValueError(f"the logits' scale must be positive, got {scale}")
        self.tensor = tied_to if tied_to is not None else (tensor if tensor is not None else self._name("weight"))
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.tensor: WeightSpec((self.vocab, self.hidden))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return ({"gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())
                | ({"elementwise"} if self.softcap or self.scale != 1.0 else set()))

    def num_bytes(self) -> int:
        w = ops.plain_of(self.weight)
        return w.numel() * w.element_size() if w is not None else 0

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.weight)

    def seal(self) -> None:
        # a tied table stays as it is for the embedding; the head streams a tiled copy
        self.weight = ops.streamed(ops.plain_of(self.weight))

    def forward(self, x: torch.Tensor, logits: torch.Tensor) -> None:
        ops.gemm(x, self.weight, logits)
        if self.softcap or self.scale != 1.0:
            ops.softcap(logits, self.softcap, self.scale)

    def can_pick(self, rows: int) -> bool:
        """Whether ``pick`` takes so many rows with this weight.  Never under a soft cap: where
        the cap saturates, equal capped logits go to the lowest index, which the pick among the
        raw ones would not reproduce."""
        return (isinstance(self.weight, ops.StreamedWeight) and 0 < rows <= ops.FUSED_NORM_MAX_M
                and self.hidden % 8 == 0 and not self.softcap)

    def pick(self, x: torch.Tensor, residual: torch.Tensor, step, tail) -> None:
        """The tail of a greedy decode step in one kernel (``ops.gemm_pick``): ``x`` holds the
        normalised row of every sequence, all of them wanted."""
        ops.gemm_pick(x, self.weight, residual, tail.tokens, step.token_ids, step.positions,
                      step.ctx_lens, tail.ring, tail.run_counter, tail.embed_table, tail.work)
