"""A matrix memory with a data-dependent decay per key channel (RWKV-style time mixing) as a
mixer with per-request state.

With ``h`` the mixer's input and ``h'`` the previous token's (zeros for a sequence's first
token), each of five inputs is a mix of its own, ``h + (h' - h) * mu_s``.  ``r, k, v`` are
projections of their mixes (``heads x dim``), the gate is ``silu(W_g mix_g)``, and the decay of
head ``h``, key channel ``i`` is ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))``.  Per head, with
a state ``S [dim, dim]`` that starts at zero::

    o_t = (S + diag(u) k_t v_t^T)^T r_t;        S <- diag(w_t) S + k_t v_t^T

Every head's ``o`` is divided by its root mean square, the heads side by side are multiplied by
a weight vector and by the gate, and projected out.  A request's state slot holds every head's
``S`` and the last token's ``h``, all in fp32, so that a prompt may be cut anywhere.  Decays,
their exponentials, the state and the head norm are fp32 in every mode; the decay's
pre-activations come from products with fp32 sums stored in fp32.
"""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import LayerState, Mixer, StateSpec, WeightSpec, add_product
from kvforge_amd.registry import register_mixer

MIXES = ("r", "k", "v", "g", "w")


@register_mixer("wkv")
class DecayMemory(Mixer):
    """``decay_rank``: rows of ``W_w1`` (columns of ``W_w2``); ``None`` takes it from the
    checkpoint's tensors.  ``names``: checkpoint names under
    the prefix, by ``r k v g o w1 w2 w0 u norm``; the mix vector of input ``s`` is
    ``<mu_prefix><s>``."""

    NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "o": "o", "w1": "w1", "w2": "w2", "w0": "w0",
             "u": "u", "norm": "norm"}

    replayable = True
    cache_spec = None

    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, decay_rank: int | None, norm_eps: float,
                 names: dict[str, str] | None = None, mu_prefix: str = "mu.") -> None:
        self.prefix, self.hidden = prefix, int(hidden)
        self.H, self.dk = int(heads), int(dim)
        self.L = int(decay_rank) if decay_rank is not None else None   # None: the checkpoint decides
        if min(self.H, self.dk, self.L or 1) <= 0 or self.dk > 256:
            raise ValueError(f"wkv kernels take heads of up to 256 elements, got heads {heads}, dim {dim}, "
                             f"decay rank {decay_rank}")
        self.norm_eps = float(norm_eps)
        self.names, self.mu_prefix = dict(self.NAMES, **(names or {})), mu_prefix
        self.state_spec = StateSpec((ops.wkv_state_floats(self.H, self.dk, self.hidden),), torch.float32)
        self.mu = self.w_proj = self.w_1 = self.w_2 = self.w0 = self.u = self.head_weight = self.w_o = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, HD = self.hidden, self.H * self.dk
        n = lambda key: self._name(self.names[key])  # noqa: E731
        out = {n(s): WeightSpec((HD, h)) for s in ("r", "k", "v", "g")}
        out.update({self._name(self.mu_prefix + s): WeightSpec((h,), init="normal", std=0.3) for s in MIXES})
        out.update({n("o"): WeightSpec((h, HD)), n("w1"): WeightSpec((self.L, h)),
                    n("w2"): WeightSpec((HD, self.L)), n("w0"): WeightSpec((HD,), std=1.0),
                    n("u"): WeightSpec((self.H, self.dk), std=0.5),
                    n("norm"): WeightSpec((HD,), init="norm", std=0.1)})
        return out

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        t = lambda key: tensors[self._name(self.names[key])]  # noqa: E731
        self.mu = torch.stack([tensors[self._name(self.mu_prefix + s)].float() for s in MIXES]).contiguous()
        self.w_proj = [t(s) for s in ("r", "k", "v", "g")]
        # the decay's two small matrices, padded with zero rows / columns to a multiple of 16
        # (which every product kernel takes): tanh(0) = 0 meets zero columns
        w1, w2 = t("w1"), t("w2")
        if self.L is None:
            self.L = int(w1.shape[0])
        if w1.shape[0] != self.L or w2.shape[1] != self.L:
            raise ValueError(f"{self._name(self.names['w1'])} {list(w1.shape)} and "
                             f"{self._name(self.names['w2'])} {list(w2.shape)} do not agree on the decay's rank")
        self.L_pad = -(-self.L // 16) * 16
        self.w_1 = torch.cat([w1, w1.new_zeros(self.L_pad - self.L, self.hidden)], dim=0).contiguous()
        self.w_2 = torch.cat([w2, w2.new_zeros(w2.shape[0], self.L_pad - self.L)], dim=1).contiguous()
        self.w0 = t("w0").float().contiguous()
        self.u = t("u").float().reshape(-1).contiguous()
        self.head_weight = t("norm").float().contiguous()
        self.w_o = t("o")

    def seal(self) -> None:
        self.w_proj = [ops.streamed(ops.plain_of(w)) for w in self.w_proj]
        self.w_1, self.w_2 = ops.streamed(ops.plain_of(self.w_1)), ops.streamed(ops.plain_of(self.w_2))
        self.w_o = ops.streamed(ops.plain_of(self.w_o))

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"wkv", "elementwise", "gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())

    def _matrices(self) -> list:
        return [w for w in (*(self.w_proj or ()), self.w_1, self.w_2, self.w_o) if w is not None]

    def _small(self) -> list[torch.Tensor]:
        return [x for x in (self.mu, self.w0, self.u, self.head_weight) if x is not None]

    def num_bytes(self) -> int:
        return sum(x.numel() * x.element_size() for x in (*map(ops.plain_of, self._matrices()), *self._small()))

    def held_tensors(self) -> list[torch.Tensor]:
        return [c for w in self._matrices() for c in ops.copies_of(w)] + self._small()

    def _long_runs(self, step) -> dict | None:
        """Chunk and run tables of this step's long runs (made once per step, shared by the layers
        of the batch) and scratch from the step's workspace.  ``None`` when no run is that long."""
        key = "wkv.long_runs"
        plan = step.scratch.get(key)
        if plan is None:
            chunks, runs = ops.wkv_multi_plan(step.q_lens)
            plan = (step.upload_ints(chunks).view(-1, 4), step.upload_ints(runs).view(-1, 3)) if chunks else ()
            step.scratch[key] = plan
        if not plan:
            return None
        out = {"chunks": plan[0], "runs": plan[1]}
        for name, (shape, dtype) in ops.wkv_multi_scratch(plan[0].shape[0], self.H, self.dk).items():
            out[name] = step.ws.buf("wkv_multi_" + name, shape, dtype)
        return out

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations."""
        if layer.state is None:
            raise RuntimeError("the wkv mixer needs a state slot per request")
        n = x.shape[0]
        H, dk, HD = self.H, self.dk, self.H * self.dk
        ws, act = step.ws, step.act_dtype
        step.settle()
        mixes = ws.buf("wkv_mixes", (len(MIXES), n, self.hidden), act)
        ops.wkv_mix(x, self.mu, layer.state, H * dk * dk, step.slot_ids, step.seq_of_token, step.cu_q,
                    step.positions, mixes, step.n_seqs)
        rows = ws.buf("wkv_rows", (n, 4 * HD), act)
        for i, w in enumerate(self.w_proj):
            ops.gemm(mixes[i], w, rows[:, i * HD:(i + 1) * HD])
        low = ws.buf("wkv_low", (n, self.L_pad), torch.float32)
        ops.gemm(mixes[4], self.w_1, low)
        low_act = ws.buf("wkv_low_act", (n, self.L_pad), act)
        ops.tanh_cast(low, low_act)
        z = ws.buf("wkv_decay", (n, HD), torch.float32)
        ops.gemm(low_act, self.w_2, z)
        raw = ws.buf("wkv_raw", (n, HD), torch.float32)
        # which kernels have work is known from the runs' lengths (all ones in a captured step of
        # single tokens, so a replay launches what the capture launched)
        ops.wkv_scan(rows, 0, HD, 2 * HD, z, self.w0, self.u, step.cu_q, step.positions, step.slot_ids,
                     layer.state, raw, step.n_seqs, H, dk, multi=self._long_runs(step),
                     short_runs=any(q < ops.WKV_MULTI_FROM for q in step.q_lens))
        heads = ws.buf("wkv_heads", (n, HD), act)
        ops.wkv_out(raw, rows[:, 3 * HD:], self.head_weight, self.norm_eps, heads, H, dk)
        add_product(step, heads, self.w_o, residual)
