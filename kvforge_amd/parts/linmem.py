"""Linear attention with a decaying matrix memory, as a mixer with per-request state.

Per head a memory ``S [dim, vdim]`` that starts at zero; with ``q, k`` (``heads x dim``) and
``v`` (``heads x vdim``) projected from the mixer's input::

    S_t = diag(a_t) S_(t-1) + k_t v_t^T;        o_t = S_t^T q_t

The decays ``a_t`` (one number per head and key channel) are either *gates* of the input,
``a = sigmoid(W_2 (W_1 h) + b)^(1/tau)`` (gated linear attention), or *constants*, one number
per head (retention).  q and k may be rotated by position first and are multiplied by
constants.  Every head's ``o`` is divided by its root mean square (and multiplied by a weight
vector that the heads share, if there is one), the heads side by side are multiplied by
``silu(W_g h)`` and a constant, and projected out.  A request's state slot holds every head's
``S`` in fp32, so that a prompt may be cut anywhere.  Decays, rotation, the state and the head
norm are fp32 in every mode; the gates' pre-activations are a product with fp32 sums stored in
fp32.
"""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import LayerState, Mixer, StateSpec, WeightSpec, add_product
from kvforge_amd.parts.positions import RotaryPositions
from kvforge_amd.registry import register_mixer


@register_mixer("linear_memory")
class LinearMemory(Mixer):
    """``gate_tau``: the decays are gates with this ``tau`` (tensors ``a1 [rank, hidden]``,
    ``a2 [heads * dim, rank]`` and its bias; ``gate_rank`` is the rank, ``None`` takes it from the
    checkpoint's tensors).  ``head_decays``: the
    decays are these constants, one per head.  Exactly one of the two.
    ``rotary``: rotation of q and k over its first ``rot_dim`` elements, or ``None``.
    ``q_scale`` / ``k_scale``: constants on q and k (after the rotation, which is linear).
    ``head_weight``: whether the head norm has a weight vector ``[vdim]`` (shared by the heads).
    ``out_scale``: a constant on the mixer's output, applied in fp32 ahead of the (linear) output
    projection.  ``names``: checkpoint names under the prefix, by ``q k v g o a1 a2 a2_bias norm``."""

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "a1": "a1", "a2": "a2", "a2_bias": "a2.b",
             "norm": "norm"}

    replayable = True
    cache_spec = None

    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, norm_eps: float,
                 gate_tau: float | None = None, head_decays=None, rotary: RotaryPositions | None = None,
                 q_scale: float = 1.0, k_scale: float = 1.0, head_weight: bool = True,
                 out_scale: float = 1.0, names: dict[str, str] | None = None,
                 gate_rank: int | None = None) -> None:
        self.prefix, self.hidden = prefix, int(hidden)
        self.H, self.dk, self.dv = int(heads), int(dim), int(vdim)
        if min(self.H, self.dk, self.dv) <= 0 or self.dk > 256:
            raise ValueError(f"linear-memory kernels take key heads of up to 256 elements, got heads {heads}, "
                             f"dim {dim}, vdim {vdim}")
        if (gate_tau is None) == (head_decays is None):
            raise ValueError("the decays are gates (gate_tau) or constants per head (head_decays): one of the two")
        self.tau = float(gate_tau) if gate_tau is not None else None
        if self.tau is not None and not self.tau > 0:
            raise ValueError(f"gate_tau must be positive, got {gate_tau}")
        self.rank = int(gate_rank) if gate_rank is not None else None
        if self.rank is not None and (self.rank <= 0 or self.tau is None):
            raise ValueError(f"gate_rank goes with gates and is positive, got {gate_rank}")
        self.head_decays = [float(x) for x in head_decays] if head_decays is not None else None
        if self.head_decays is not None and len(self.head_decays) != self.H:
            raise ValueError(f"head_decays needs one number per head ({self.H}), got {len(self.head_decays)}")
        self.rotary = rotary
        if rotary is not None and rotary.rot_dim > self.dk:
            raise ValueError(f"rotary width {rotary.rot_dim} exceeds the key size {self.dk}")
        self.q_scale, self.k_scale, self.out_scale = float(q_scale), float(k_scale), float(out_scale)
        self.has_head_weight = bool(head_weight)
        self.norm_eps = float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.state_spec = StateSpec((ops.linmem_state_floats(self.H, self.dk, self.dv),), torch.float32)
        self.w_rows = self.w_a1 = self.w_a2 = self.gate_bias = self.decays = self.head_weight = self.w_o = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, Q, V = self.hidden, self.H * self.dk, self.H * self.dv
        n = lambda key: self._name(self.names[key])  # noqa: E731
        out = {n("q"): WeightSpec((Q, h)), n("k"): WeightSpec((Q, h)), n("v"): WeightSpec((V, h)),
               n("g"): WeightSpec((V, h)), n("o"): WeightSpec((h, V))}
        if self.tau is not None:
            out.update({n("a1"): WeightSpec((self.rank, h)), n("a2"): WeightSpec((Q, self.rank)),
                        n("a2_bias"): WeightSpec((Q,), std=1.0)})
        if self.has_head_weight:
            out[n("norm")] = WeightSpec((self.dv,), init="norm", std=0.1)
        return out

    def pair_permutation(self) -> torch.Tensor:
        """``perm[new] = old`` within a key head: the kernel rotates neighbouring elements, a
        checkpoint that pairs element ``i`` with ``i + rot/2`` has its pairs moved next to each
        other.  q, k and the decays take the same order, which changes no ``q . k``."""
        perm = torch.arange(self.dk)
        if self.rotary is None or self.rotary.interleaved:
            return perm
        rot = self.rotary.rot_dim
        for i in range(rot // 2):
            perm[2 * i], perm[2 * i + 1] = i, i + rot // 2
        return perm

    def _key_order(self, w: torch.Tensor) -> torch.Tensor:
        """Rows (or entries) that go by (head, key channel), in the kernel's order."""
        perm = self.pair_permutation().to(w.device)
        return w.view(self.H, self.dk, *w.shape[1:])[:, perm].reshape(w.shape).contiguous()

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        t = lambda key: tensors[self._name(self.names[key])]  # noqa: E731
        mats = [self._key_order(t("q")), self._key_order(t("k")), t("v"), t("g")]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # one product for q, k, v and the output gate: their heads side by side in that order
        self.w_rows = torch.cat(mats, dim=0).contiguous()
        dev = self.w_rows.device
        if self.tau is not None:
            # the gates' two small matrices, the rank padded with zero rows / columns to a multiple
            # of 16 (which every product kernel takes)
            a1, a2 = t("a1"), self._key_order(t("a2"))
            rank = int(a1.shape[0])
            if a2.shape[1] != rank or rank <= 0 or (self.rank is not None and rank != self.rank):
                raise ValueError(f"{self._name(self.names['a1'])} {list(a1.shape)} and "
                                 f"{self._name(self.names['a2'])} {list(a2.shape)} do not agree on the gates' rank")
            self.rank_pad = -(-rank // 16) * 16
            self.w_a1 = torch.cat([a1, a1.new_zeros(self.rank_pad - rank, self.hidden)], dim=0).contiguous()
            self.w_a2 = torch.cat([a2, a2.new_zeros(a2.shape[0], self.rank_pad - rank)], dim=1).contiguous()
            self.gate_bias = self._key_order(t("a2_bias").float())
        else:
            d = torch.tensor(self.head_decays, dtype=torch.float32, device=dev)
            self.decays = d[:, None].expand(self.H, self.dk).reshape(-1).contiguous()
        self.head_weight = t("norm").float().contiguous() if self.has_head_weight else None
        self.w_o = t("o")

    def seal(self) -> None:
        self.w_rows, self.w_o = ops.streamed(ops.plain_of(self.w_rows)), ops.streamed(ops.plain_of(self.w_o))
        if self.w_a1 is not None:
            self.w_a1, self.w_a2 = ops.streamed(ops.plain_of(self.w_a1)), ops.streamed(ops.plain_of(self.w_a2))

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"linmem", "elementwise", "gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())

    def _matrices(self) -> list:
        return [w for w in (self.w_rows, self.w_a1, self.w_a2, self.w_o) if w is not None]

    def _small(self) -> list[torch.Tensor]:
        return [x for x in (self.gate_bias, self.decays, self.head_weight) if x is not None]

    def num_bytes(self) -> int:
        return sum(x.numel() * x.element_size() for x in (*map(ops.plain_of, self._matrices()), *self._small()))

    def held_tensors(self) -> list[torch.Tensor]:
        return [c for w in self._matrices() for c in ops.copies_of(w)] + self._small()

    def _long_runs(self, step) -> dict | None:
        """Chunk and run tables of this step's long runs (made once per step, shared by the layers
        of the batch) and scratch from the step's workspace.  ``None`` when no run is that long."""
        key = "linmem.long_runs"
        plan = step.scratch.get(key)
        if plan is None:
            chunks, runs = ops.linmem_multi_plan(step.q_lens)
            plan = (step.upload_ints(chunks).view(-1, 4), step.upload_ints(runs).view(-1, 3)) if chunks else ()
            step.scratch[key] = plan
        if not plan:
            return None
        out = {"chunks": plan[0], "runs": plan[1]}
        for name, (shape, dtype) in ops.linmem_multi_scratch(plan[0].shape[0], self.H, self.dk, self.dv).items():
            out[name] = step.ws.buf("linmem_multi_" + name, shape, dtype)
        return out

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations."""
        if layer.state is None:
            raise RuntimeError("the linear-memory mixer needs a state slot per request")
        n = x.shape[0]
        H, dk, dv = self.H, self.dk, self.dv
        Q, V = H * dk, H * dv
        ws, act = step.ws, step.act_dtype
        step.settle()
        rows = ws.buf("linmem_rows", (n, 2 * Q + 2 * V), act)
        ops.gemm(x, self.w_rows, rows)
        if self.tau is not None:
            low = ws.buf("linmem_low", (n, self.rank_pad), act)
            ops.gemm(x, self.w_a1, low)
            decay = ws.buf("linmem_gates", (n, Q), torch.float32)
            ops.gemm(low, self.w_a2, decay)       # 32-bit sums, stored so
        else:
            decay = self.decays
        cos, sin = (self.rotary.cos, self.rotary.sin) if self.rotary is not None else (None, None)
        raw = ws.buf("linmem_raw", (n, V), torch.float32)
        # which kernels have work is known from the runs' lengths (all ones in a captured step of
        # single tokens, so a replay launches what the capture launched)
        ops.linmem_scan(rows[:, :Q], rows[:, Q:2 * Q], rows[:, 2 * Q:2 * Q + V], decay, step.cu_q,
                        step.positions, step.slot_ids, layer.state, raw, step.n_seqs, H, dk, dv,
                        gate_bias=self.gate_bias, tau=self.tau, q_scale=self.q_scale, k_scale=self.k_scale,
                        multi=self._long_runs(step),
                        short_runs=any(q < ops.LINMEM_MULTI_FROM for q in step.q_lens), cos=cos, sin=sin)
        heads = ws.buf("linmem_heads", (n, V), act)
        ops.linmem_out(raw, rows[:, 2 * Q + V:], self.head_weight, self.norm_eps, heads, H, dv, self.out_scale)
        add_product(step, heads, self.w_o, residual)
