"""Pre-norm residual block: ``h += mixer(norm1(h)); h += ffn(norm2(h))``
(src/tokenvault/model.py:135-143,185-187).  The residual stream is fp32 in every mode; the
mixer's and the feed-forward's last products add into it."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import (Block, FeedForward, LayerState, Mixer, Norm, Part, StateSpec,
                                    WeightSpec)
from kvforge_amd.registry import register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    """``ffn`` (and its norm) may be ``None``: a layer of the mixer alone."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None) -> None:
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")

        self.mixer_takes_residual = self.ffn_takes_residual = False

    def parts(self) -> list[Part]:
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def load(self, tensors) -> None:
        super().load(tensors)
        # a part may apply the norm in front of it inside its own first kernel
        self.mixer_takes_residual = self.mixer.absorb_norm(self.mixer_norm)
        self.ffn_takes_residual = self.ffn is not None and self.ffn.absorb_norm(self.ffn_norm)

    def forward(self, residual, step, layer: LayerState) -> None:
        if self.mixer_takes_residual:
            if not self.mixer.settles_residual:
                step.settle()
            self.mixer.forward(residual, step, layer, residual)
        else:
            x = step.ws.buf("normed", tuple(residual.shape), step.act_dtype)
            self.mixer_norm.forward(residual, x, add=step.take_owed(residual))
            self.mixer.forward(x, step, layer, residual)
        if self.ffn is None:
            return
        if self.ffn_takes_residual:
            if not self.ffn.settles_residual:
                step.settle()
            self.ffn.forward(residual, step, residual)
        else:
            x = step.ws.buf("normed", tuple(residual.shape), step.act_dtype)
            self.ffn_norm.forward(residual, x, add=step.take_owed(residual))
            self.ffn.forward(x, step, residual)


@register_block("parallel")
class ParallelBlock(Block):
    """One norm, both sublayers read its output: ``h = norm(x); x += mixer(h) + ffn(h)`` (``ffn``
    may be ``None``), then an optional part that feeds something more into the stream
    (``after``, called as ``after.forward(residual, step, bias=...)``).  With ``ffn_norm`` the
    feed-forward has a norm of its own over the same ``x``: ``x += mixer(norm(x)) + ffn(ffn_norm(x))``.

    ``shift_name``: checkpoint name of a vector ``mu [hidden]``; the *mixer* then reads
    ``h_t + (h_{t-1} - h_t) * mu`` instead of ``h_t`` (token shift: ``h_{t-1}`` is the previous
    token's ``h`` before this replacement, zeros for a sequence's first token), while the
    feed-forward reads ``h`` as it is.  The last ``h`` of every live sequence is the block's
    state (one fp32 row per request and call), so that a prompt may be cut anywhere.  Norm,
    shift and the state's upkeep are one kernel."""

    def __init__(self, norm: Norm, mixer: Mixer, ffn: FeedForward | None, hidden: int,
                 shift_name: str | None = None, after: Part | None = None,
                 ffn_norm: Norm | None = None) -> None:
        self.norm, self.mixer, self.ffn, self.after = norm, mixer, ffn, after
        self.ffn_norm = ffn_norm if ffn is not None else None
        self.hidden, self.shift_name = int(hidden), shift_name
        self.mu: torch.Tensor | None = None
        if shift_name is not None:
            if mixer.state_spec is not None:
                raise ValueError("token shift beside a mixer with state of its own is not supported")
            if not hasattr(norm, "weight") or not hasattr(norm, "eps"):
                raise ValueError("token shift is fused with an RMS norm (a norm with weight and eps)")
        if ffn is not None and after is not None and hasattr(ffn, "defer_down_bias"):
            ffn.defer_down_bias = True   # `after` adds it on its way

    @property
    def state_spec(self) -> StateSpec | None:
        if self.shift_name is not None:
            return StateSpec((self.hidden,), torch.float32)
        return self.mixer.state_spec

    def parts(self) -> list[Part]:
        return [p for p in (self.norm, self.ffn_norm, self.mixer, self.ffn, self.after) if p is not None]

    def _norms_pair(self) -> bool:
        """Whether the two norms are RMS norms with fp32 weight vectors and one eps, which one
        kernel then takes together."""
        a, b = self.norm, self.ffn_norm
        return (b is not None and type(a).forward is type(b).forward
                and all(isinstance(getattr(n, "weight", None), torch.Tensor) and n.weight.dtype == torch.float32
                        for n in (a, b))
                and getattr(a, "eps", None) == getattr(b, "eps", 0.0))

    def weight_specs(self) -> dict[str, WeightSpec]:
        out = super().weight_specs()
        if self.shift_name is not None:
            out[self.shift_name] = WeightSpec((self.hidden,), init="normal", std=0.3)
        return out

    def load(self, tensors) -> None:
        super().load(tensors)
        if self.shift_name is not None:
            self.mu = tensors[self.shift_name].float().contiguous()
            # the fused kernel multiplies by fp32 vectors
            if self.norm.weight.dtype != torch.float32:
                self.norm.weight = self.norm.weight.float()

    def kernel_modules(self, dtype) -> set[str]:
        return super().kernel_modules(dtype) | {"elementwise"}

    def held_tensors(self) -> list[torch.Tensor]:
        return super().held_tensors() + ([self.mu] if self.mu is not None else [])

    def num_bytes(self) -> int:
        return super().num_bytes() + (4 * self.mu.numel() if self.mu is not None else 0)

    def forward(self, residual, step, layer: LayerState) -> None:
        shape = tuple(residual.shape)
        h = step.ws.buf("parallel_normed", shape, step.act_dtype)
        if self.mu is not None:
            step.settle()
            hs = step.ws.buf("parallel_shifted", shape, step.act_dtype)
            ops.norm_shift(residual, self.norm.weight, self.mu, layer.state, step.slot_ids,
                           step.seq_of_token, step.cu_q, step.positions, self.norm.eps, h, hs)
        elif self._norms_pair():
            # two RMS norms of the same stream: one pass over it, two weights
            hs = h
            h = step.ws.buf("parallel_normed_ffn", shape, step.act_dtype)
            ops.rmsnorm_pair(residual, self.norm.weight, self.ffn_norm.weight, self.norm.eps, hs, h,
                             add=step.take_owed(residual))
        else:
            self.norm.forward(residual, h, add=step.take_owed(residual))
            hs = h
        if self.ffn_norm is not None and not (self.mu is None and self._norms_pair()):
            # of the same stream as the mixer's norm: taken before the mixer adds to it
            h = step.ws.buf("parallel_normed_ffn", shape, step.act_dtype)
            self.ffn_norm.forward(residual, h)
        self.mixer.forward(hs, step, layer, residual)
        bias = None
        if self.ffn is not None:
            if not self.ffn.settles_residual:
                step.settle()
            self.ffn.forward(h, step, residual)
            if getattr(self.ffn, "defer_down_bias", False):
                bias = self.ffn.down_bias
        if self.after is not None:
            self.after.forward(residual, step, bias=bias)


@register_block("sandwich")
class SandwichBlock(Block):
    """A norm before and after each sublayer: ``x += post(mixer(pre(x)))`` and then, if the layer
    has a feed-forward, ``x += ffn_post(ffn(ffn_pre(x)))``.  A sublayer's output does not join
    the stream as it is, so its last product is written to rows of its own (fp32; the step
    holds them as ``fresh``, see ``parts.base.add_product``), and the norm behind the sublayer
    adds them to the stream (``Norm.add_to``: norm and sum in one pass, in fp32)."""

    def __init__(self, pre: Norm, mixer: Mixer, post: Norm, ffn_pre: Norm | None = None,
                 ffn: FeedForward | None = None, ffn_post: Norm | None = None) -> None:
        if ffn is not None and (ffn_pre is None or ffn_post is None):
            raise ValueError("a feed-forward in a sandwich block needs its two norms")
        self.pre, self.mixer, self.post = pre, mixer, post
        self.ffn_pre, self.ffn, self.ffn_post = (ffn_pre, ffn, ffn_post) if ffn is not None else (None, None, None)

    def parts(self) -> list[Part]:
        return [p for p in (self.pre, self.mixer, self.post, self.ffn_pre, self.ffn, self.ffn_post)
                if p is not None]

    def kernel_modules(self, dtype) -> set[str]:
        return super().kernel_modules(dtype) | {"elementwise"}

    def forward(self, residual, step, layer: LayerState) -> None:
        shape = tuple(residual.shape)
        x = step.ws.buf("normed", shape, step.act_dtype)
        self._norm_in(self.pre, residual, x, step)
        branch = step.ws.buf("sublayer_out", shape, torch.float32)
        step.fresh = branch
        self.mixer.forward(x, step, layer, branch)
        self._join(residual, branch, self.post, step)
        if self.ffn is None:
            return
        self._norm_in(self.ffn_pre, residual, x, step)
        step.fresh = branch
        self.ffn.forward(x, step, branch)
        self._join(residual, branch, self.ffn_post, step)

    @staticmethod
    def _join(residual, branch, post: Norm, step) -> None:
        """The sublayer's rows stay owed to the stream, through their norm, until the stream is
        read next: by the norm in front of the next sublayer (one kernel for the sum and that
        norm), or by whoever settles the step."""
        if step.fresh is branch:
            raise RuntimeError("a sublayer of a sandwich block must end in parts.base.add_product")
        step.settle()
        weight = post.fp32_weight() if hasattr(post, "fp32_weight") else None
        if weight is None:
            post.add_to(residual, branch)
        else:
            step.owed = (residual, branch, weight, post.eps)

    @staticmethod
    def _norm_in(norm: Norm, residual, x, step) -> None:
        owed = step.take_owed_normed(residual)
        weight = norm.fp32_weight() if hasattr(norm, "fp32_weight") else None
        if owed is not None and weight is not None:
            ops.rms_add_norm(residual, owed[0], owed[1], owed[2], weight, norm.eps, x)
            return
        if owed is not None:
            ops.rms_add(residual, *owed)
        norm.forward(residual, x, add=step.take_owed(residual))
