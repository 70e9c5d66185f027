"""Feed-forward of routed experts: every token is sent to a few of many small gated
feed-forwards, chosen by a softmax router, plus (optionally) one that all tokens share.

Router: ``s = softmax(W_r x)`` over all its outputs, in fp32.  The ``top`` outputs with the
largest ``s + correction`` are chosen; their weights are their ``s`` divided by the sum of the
chosen ``s`` (+ 1e-20), so the correction steers the choice and never the weights.  The router's
last ``identity`` outputs name no expert: choosing one passes the token's input on, times the
weight.  An expert is ``down(silu(gate x) * (up x))`` without biases; the layer's output is the
weighted sum over the chosen experts, plus the shared expert's output.

Instead of a router a *table* may make the choice: an integer tensor ``[vocab, top]`` names the
experts of every token id (a row's entries differ), each with weight ``1 / top``.  The shared
expert's output may be multiplied by ``sigmoid(w . x)``, one number per token.
"""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import FeedForward, WeightSpec, add_product
from kvforge_amd.parts.feedforward import GatedFeedForward
from kvforge_amd.registry import register_feed_forward


@register_feed_forward("moe")
class RoutedExperts(FeedForward):
    """``names``: checkpoint names under the prefix, by ``expert`` (a format with ``{e}``),
    ``gate up down`` (under an expert and under ``shared``), ``router correction shared``,
    ``table`` and ``shared_gate``.  ``table_vocab``: the choice is made by the table
    ``[table_vocab, top]`` from the token's id; there is no router and no identity output.
    ``shared_gate``: the shared expert's output is multiplied by ``sigmoid(w . x)`` with ``w``
    the tensor ``[1, hidden]`` named ``shared_gate`` under the shared expert's prefix; the number
    is a product with fp32 sums and joins the expert's activation ahead of its (linear) down
    projection."""

    NAMES = {"expert": "e{e}", "gate": "gate", "up": "up", "down": "down", "router": "router",
             "correction": "correction", "shared": "shared", "table": "table", "shared_gate": "sg"}

    replayable = True

    def __init__(self, prefix: str, hidden: int, ff: int, experts: int, top: int, identity: int = 0,
                 shared_ff: int = 0, names: dict[str, str] | None = None, table_vocab: int | None = None,
                 shared_gate: bool = False) -> None:
        self.prefix, self.hidden, self.ff = prefix, int(hidden), int(ff)
        self.E, self.top, self.identity = int(experts), int(top), int(identity)
        self.R = self.E + self.identity
        self.table_vocab = int(table_vocab) if table_vocab else None
        if self.table_vocab is not None and self.identity:
            raise ValueError("a table names experts only: no identity outputs beside it")
        self.shared_gate = bool(shared_gate)
        if self.shared_gate and not shared_ff:
            raise ValueError("a gate on the shared expert goes with a shared expert")
        self.table = self.w_shared_gate = None
        if not 0 < self.top <= min(self.R, ops.MOE_MAX_TOP) or self.R > ops.MOE_MAX_ROUTER_OUTPUTS:
            raise ValueError(f"router of {self.R} outputs choosing {self.top}: the kernels take up to "
                             f"{ops.MOE_MAX_ROUTER_OUTPUTS} outputs and {ops.MOE_MAX_TOP} choices")
        self.names = dict(self.NAMES, **(names or {}))
        self.shared = None
        if shared_ff:
            self.shared = GatedFeedForward(
                self._name(self.names["shared"]), hidden, shared_ff, activation="silu",
                names={k: self.names[k] for k in ("gate", "up", "down")})
        self.w_router = self.correction = self.w_gate_up = self.w_down = None

    def _expert(self, e: int, which: str) -> str:
        return self._name(f"{self.names['expert'].format(e=e)}.{self.names[which]}")

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, ff = self.hidden, self.ff
        if self.table_vocab is not None:
            out = {self._name(self.names["table"]): WeightSpec((self.table_vocab, self.top), init="choices",
                                                                std=float(self.E), integer=True)}
        else:
            out = {self._name(self.names["router"]): WeightSpec((self.R, h)),
                   self._name(self.names["correction"]): WeightSpec((self.R,))}
        for e in range(self.E):
            out[self._expert(e, "gate")] = WeightSpec((ff, h))
            out[self._expert(e, "up")] = WeightSpec((ff, h))
            out[self._expert(e, "down")] = WeightSpec((h, ff))
        if self.shared is not None:
            out.update(self.shared.weight_specs())
        if self.shared_gate:
            out[self.shared._name(self.names["shared_gate"])] = WeightSpec((1, h))
        return out

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        # the router's rows padded with zero rows to a multiple of 16, which every product kernel
        # takes; in the engine's type: products of bfloat16 numbers are exact in 32 bits, and the
        # sums are 32-bit and stored so
        if self.table_vocab is not None:
            self.table = tensors[self._name(self.names["table"])].to(torch.int32).contiguous()
        else:
            r = tensors[self._name(self.names["router"])]
            self.R_pad = -(-self.R // 16) * 16
            self.w_router = torch.cat([r, r.new_zeros(self.R_pad - self.R, self.hidden)], dim=0).contiguous()
            self.correction = tensors[self._name(self.names["correction"])].float().contiguous()
        if self.shared_gate:
            # one row, padded with zero rows to 16 (which every product kernel takes)
            g = tensors[self.shared._name(self.names["shared_gate"])]
            self.w_shared_gate = torch.cat([g, g.new_zeros(15, self.hidden)], dim=0).contiguous()
        pairs, downs = [], []
        for e in range(self.E):
            g, u = tensors[self._expert(e, "gate")], tensors[self._expert(e, "up")]
            d = tensors[self._expert(e, "down")]
            if not (g.dtype == u.dtype == d.dtype):
                g, u, d = g.float(), u.float(), d.float()
            # an expert's gate and up rows interleaved, the experts one after the other
            pairs.append(torch.stack([g, u], dim=1).reshape(2 * self.ff, self.hidden))
            downs.append(d)
        if len({p.dtype for p in pairs}) > 1:
            pairs, downs = [p.float() for p in pairs], [d.float() for d in downs]
        self.w_gate_up = torch.cat(pairs, dim=0).contiguous()          # [E 2 ff, hidden]
        self.w_down = torch.cat(downs, dim=1).contiguous()             # [hidden, E ff]
        if self.shared is not None:
            self.shared.load(tensors)

    def seal(self) -> None:
        self.w_gate_up = ops.streamed(ops.plain_of(self.w_gate_up))
        self.w_down = ops.streamed(ops.plain_of(self.w_down))
        if self.w_router is not None:
            self.w_router = ops.streamed(ops.plain_of(self.w_router))
        if self.w_shared_gate is not None:
            self.w_shared_gate = ops.streamed(ops.plain_of(self.w_shared_gate))
        if self.shared is not None:
            self.shared.seal()

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        mods = {"moe", "elementwise", "gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())
        return mods | (self.shared.kernel_modules(dtype) if self.shared is not None else set())

    def num_bytes(self) -> int:
        """What one token reads: the router, its ``top`` experts' share of the experts' matrices,
        the shared expert."""
        experts = sum(t.numel() * t.element_size() for t in map(ops.plain_of, (self.w_gate_up, self.w_down))
                      if t is not None)
        small = sum(t.numel() * t.element_size()
                    for t in (ops.plain_of(self.w_router) if self.w_router is not None else None, self.correction,
                              ops.plain_of(self.w_shared_gate) if self.w_shared_gate is not None else None)
                    if t is not None)
        return (small + experts * min(self.top, self.E) // max(self.E, 1)
                + (self.shared.num_bytes() if self.shared is not None else 0))

    def held_tensors(self) -> list[torch.Tensor]:
        return (ops.copies_of(self.w_gate_up) + ops.copies_of(self.w_down)
                + (ops.copies_of(self.w_router) if self.w_router is not None else [])
                + (ops.copies_of(self.w_shared_gate) if self.w_shared_gate is not None else [])
                + [t for t in (self.correction, self.table) if t is not None]
                + (self.shared.held_tensors() if self.shared is not None else []))

    def forward(self, x, step, residual) -> None:
        """``x``: normalised activations."""
        n = x.shape[0]
        ws, dt = step.ws, step.act_dtype
        step.settle()
        chosen = ws.buf("moe_chosen", (n, self.top), torch.int32)
        weights = ws.buf("moe_weights", (n, self.top), torch.float32)
        if self.table is not None:
            ops.moe_table(step.token_ids, self.table, chosen, weights, self.E)
        else:
            logits = ws.buf("moe_logits", (n, self.R_pad), torch.float32)[:, :self.R]
            ops.gemm(x, self.w_router, ws.buf("moe_logits", (n, self.R_pad), torch.float32))   # 32-bit sums, stored so
            ops.moe_topk(logits, self.correction, chosen, weights)
        if ops.moe_grouped_takes(x, self.w_gate_up, self.w_down, self.E, self.ff) and x.is_contiguous():
            # bf16: every expert over only the rows that chose it, grouped on the device
            pairs, tiles = n * self.top, ops.moe_grouped_tiles(n, self.top, self.E)
            scratch = {"where": ws.buf("moe_where", (pairs,), torch.int32),
                       "order": ws.buf("moe_order", (pairs,), torch.int32),
                       "tiles": ws.buf("moe_tiles", (3 * tiles,), torch.int32),
                       "num_tiles": ws.buf("moe_num_tiles", (1,), torch.int32),
                       "act": ws.buf("moe_act_rows", (pairs, self.ff), dt),
                       "y": ws.buf("moe_y_rows", (pairs, self.hidden), dt)}
            ops.moe_grouped(x, self.w_gate_up, self.w_down, chosen, weights, residual, self.E, self.ff, scratch)
            self._shared_forward(x, step, residual)
            return
        # otherwise (32-bit, or sizes the grouped kernels do not take): every expert over every
        # row in one product, the rows that did not choose it multiplied by an exact zero
        if self.identity:
            ops.moe_identity(residual, x, chosen, weights, self.E)
        gu = ws.buf("moe_gate_up", (n, 2 * self.E * self.ff), dt)
        ops.gemm(x, self.w_gate_up, gu)
        act = ws.buf("moe_act", (n, self.E * self.ff), dt)
        ops.moe_dense_act(gu, chosen, weights, act, self.E, self.ff)
        add_product(step, act, self.w_down, residual)
        self._shared_forward(x, step, residual)

    def _shared_forward(self, x, step, residual) -> None:
        if self.shared is None:
            return
        if self.w_shared_gate is None:
            self.shared.forward(x, step, residual)
            return
        # the token's gate is a number per row: it joins the activation, ahead of the down projection
        n, sh = x.shape[0], self.shared
        step.settle()
        gate = step.ws.buf("moe_shared_gate", (n, 16), torch.float32)
        ops.gemm(x, self.w_shared_gate, gate)                      # 32-bit sums, stored so
        gu = step.ws.buf("gate_up", (n, 2 * sh.inter), step.act_dtype)
        ops.gemm(x, sh.w_gate_up, gu)
        act = step.ws.buf("ffn_act", (n, sh.inter), step.act_dtype)
        ops.gated_act_rowgate(gu, gate, act, sh.activation)
        add_product(step, act, sh.w_down, residual)
