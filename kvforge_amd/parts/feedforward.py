"""Gated feed-forward: ``down(act(gate(x)) * up(x))``.  ``SwiGLU`` is the form with ``act = silu``
and no biases (src/tokenvault/model.py:118-132); ``GatedFeedForward`` takes the activation, biases
on the three projections and the checkpoint names as arguments."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import FeedForward, WeightSpec, add_product
from kvforge_amd.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    replayable = True
    settles_residual = True  # its norm kernel adds what is owed to the stream

    def __init__(self, prefix: str, hidden: int, intermediate: int) -> None:
        self.prefix, self.hidden, self.inter = prefix, int(hidden), int(intermediate)
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {
            self._name("gate_proj.weight"): WeightSpec((self.inter, self.hidden)),
            self._name("up_proj.weight"): WeightSpec((self.inter, self.hidden)),
            self._name("down_proj.weight"): WeightSpec((self.hidden, self.inter)),
        }

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        g, u = tensors[self._name("gate_proj.weight")], tensors[self._name("up_proj.weight")]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        # one product for gate and up, rows interleaved: row 2i is gate_i, row 2i+1 is up_i, so
        # a kernel that holds neighbouring output columns holds a whole (gate, up) pair
        self.w_gate_up = torch.stack([g, u], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = tensors[self._name("down_proj.weight")]
        self.norm_eps = None

    def absorb_norm(self, norm) -> bool:
        if self.norm_eps is not None or not getattr(norm, "foldable_into", lambda m: False)(self.w_gate_up):
            return False
        self.w_gate_up = (self.w_gate_up.float() * norm.weight.float()[None, :]).to(
            torch.bfloat16).contiguous()
        self.norm_eps = norm.eps
        return True

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        mods = {"elementwise", "gemm_generic"}
        if dtype == torch.bfloat16:
            mods |= {"gemm_bf16"}
        return mods

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size()
                   for t in map(ops.plain_of, (self.w_gate_up, self.w_down)) if t is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.w_gate_up) + ops.copies_of(self.w_down)

    def seal(self) -> None:
        self.w_gate_up = ops.streamed(ops.plain_of(self.w_gate_up))
        self.w_down = ops.streamed(ops.plain_of(self.w_down))

    def forward(self, x, step, residual) -> None:
        """``x``: normalised activations, or (after ``absorb_norm``) the fp32 residual stream."""
        n = x.shape[0]
        ws, dt, rms = step.ws, step.act_dtype, self.norm_eps
        act = ws.buf("ffn_act", (n, self.inter), dt)
        if rms is not None and not ops.bf16_kernel_takes(x, self.w_gate_up, True):
            # too many rows for the norm to ride in the projection: a norm kernel of its own,
            # which also adds what the mixer still owes the stream
            normed = ws.buf("normed", (n, self.hidden), dt)
            ops.rmsnorm(x, None, rms, normed, add=step.take_owed(residual))
            x, rms = normed, None
        else:
            step.settle()
        if ops.bf16_kernel_takes(x, self.w_gate_up, rms is not None, True) and self.inter % 2 == 0:
            # one kernel: (norm,) gate/up projection, SwiGLU gate
            ops.gemm_fused(x, self.w_gate_up, act, rms_eps=rms, silu_pairs=True)
        else:
            gu = ws.buf("gate_up", (n, 2 * self.inter), dt)
            ops.gemm(x, self.w_gate_up, gu)
            ops.silu_mul(gu, act, paired=True)
        add_product(step, act, self.w_down, residual)


@register_feed_forward("gated")
class GatedFeedForward(SwiGLU):
    """``down(act(gate x + b_gate) * (up x + b_up)) + b_down``.

    ``activation``: ``"silu"`` or ``"gelu_tanh"`` (``0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))``).
    ``bias``: whether the three projections have biases; they are held in fp32 and added in
    fp32, the first two inside the activation kernel.  The bias of the down projection belongs
    to the stream: ``forward`` adds it with a kernel of its own unless the block asks to add it
    itself (``defer_down_bias``), in which case it is found in ``down_bias``.
    ``names``: checkpoint names under the prefix, by ``gate up down``; a bias is ``<name><bias_suffix>``."""

    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu",
                 bias: bool = False, names: dict[str, str] | None = None,
                 bias_suffix: str = ".bias") -> None:
        super().__init__(prefix, hidden, intermediate)
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.activation, self.bias = activation, bool(bias)
        self.names = dict(self.NAMES, **(names or {}))
        self.bias_suffix = bias_suffix
        self.gate_bias = self.up_bias = self.down_bias = None
        self.defer_down_bias = False

    def weight_specs(self) -> dict[str, WeightSpec]:
        shapes = {"gate": (self.inter, self.hidden), "up": (self.inter, self.hidden),
                  "down": (self.hidden, self.inter)}
        out = {self._name(self.names[n]): WeightSpec(sh) for n, sh in shapes.items()}
        if self.bias:
            out.update({self._name(self.names[n] + self.bias_suffix): WeightSpec((sh[0],))
                        for n, sh in shapes.items()})
        return out

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        g, u = tensors[self._name(self.names["gate"])], tensors[self._name(self.names["up"])]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = torch.stack([g, u], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = tensors[self._name(self.names["down"])]
        self.norm_eps = None
        if self.bias:
            self.gate_bias, self.up_bias, self.down_bias = (
                tensors[self._name(self.names[n] + self.bias_suffix)].float().contiguous()
                for n in ("gate", "up", "down"))

    def absorb_norm(self, norm) -> bool:
        return False

    def num_bytes(self) -> int:
        return super().num_bytes() + sum(4 * b.numel() for b in (self.gate_bias, self.up_bias, self.down_bias)
                                         if b is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return super().held_tensors() + [b for b in (self.gate_bias, self.up_bias, self.down_bias)
                                         if b is not None]

    def forward(self, x, step, residual) -> None:
        """``x``: normalised activations."""
        n = x.shape[0]
        ws, dt = step.ws, step.act_dtype
        step.settle()
        act = ws.buf("ffn_act", (n, self.inter), dt)
        if ops.bf16_kernel_takes(x, self.w_gate_up, False, True) and self.inter % 2 == 0:
            # one kernel: gate/up projection, biases, activation, gate
            ops.gemm_gated(x, self.w_gate_up, act, self.activation, self.gate_bias, self.up_bias)
        else:
            gu = ws.buf("gate_up", (n, 2 * self.inter), dt)
            ops.gemm(x, self.w_gate_up, gu)
            ops.gated_act(gu, act, self.activation, paired=True, gate_bias=self.gate_bias,
                          up_bias=self.up_bias)
        add_product(step, act, self.w_down, residual)
        if self.down_bias is not None and not self.defer_down_bias:
            step.settle()
            ops.add_bias(residual, self.down_bias)


@register_feed_forward("plain")
class PlainFeedForward(FeedForward):
    """``down(act(up x))`` without gate and biases.  ``activation``: ``"relu2"`` (the square of
    relu), ``"silu"`` or ``"gelu_tanh"``, applied in fp32 to the stored product and rounded once.
    ``names``: checkpoint names under the prefix, by ``up down``."""

    NAMES = {"up": "up_proj.weight", "down": "down_proj.weight"}

    replayable = True

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "relu2",
                 names: dict[str, str] | None = None) -> None:
        if activation not in ops.PLAIN_ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {sorted(ops.PLAIN_ACTIVATIONS)}")
        self.prefix, self.hidden, self.inter = prefix, int(hidden), int(intermediate)
        self.activation = activation
        self.names = dict(self.NAMES, **(names or {}))
        self.w_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self._name(self.names["up"]): WeightSpec((self.inter, self.hidden)),
                self._name(self.names["down"]): WeightSpec((self.hidden, self.inter))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.w_up = tensors[self._name(self.names["up"])]
        self.w_down = tensors[self._name(self.names["down"])]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise", "gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in map(ops.plain_of, (self.w_up, self.w_down)) if t is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.w_up) + ops.copies_of(self.w_down)

    def seal(self) -> None:
        self.w_up, self.w_down = ops.streamed(ops.plain_of(self.w_up)), ops.streamed(ops.plain_of(self.w_down))

    def forward(self, x, step, residual) -> None:
        """``x``: normalised activations."""
        n = x.shape[0]
        step.settle()
        act = step.ws.buf("ffn_act", (n, self.inter), step.act_dtype)
        ops.gemm(x, self.w_up, act)
        ops.plain_act(act, act, self.activation)
        add_product(step, act, self.w_down, residual)
