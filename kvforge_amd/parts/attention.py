"""Grouped-query causal attention over the paged cache (src/tokenvault/model.py:64-92).

Order of work per call, as in the reference: project q, k, v; rotate q and k; write k and v into
the cache; attend from the cache (the current tokens' keys are read back from it); project out.
Query runs longer than one token go to the prefill kernel, single tokens to the decode kernel;
both read the same pages through the same block tables.
"""

from __future__ import annotations

import math

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import (CacheSpec, LayerState, Mixer, WeightSpec, add_product,
                                    attention_pages)
from kvforge_amd.parts.positions import RotaryPositions
from kvforge_amd.registry import register_mixer

# Launch planning of the decode kernels.  The key range of single-token queries is cut so that
# about one workgroup per compute unit pulls on the cache when the sequences alone do not fill
# the chip, each cut with at least KEYS_PER_CUT keys (below that the merge of the cuts costs more
# than they save), and further when contexts are uneven.  Everything the launches depend on
# besides the padded batch size is the pair (context cell, cuts for uneven contexts) that
# ``PagedAttention.launch_key`` returns, so that captured launches can be replayed for any step
# with the same pair.
KEYS_PER_CUT = 512
MAX_CUTS = 64            # what the merge kernels take
SKEW_MAX_CUTS = 8


def compute_units(device) -> int:
    return ops.compute_units(device)


def skew_cuts(max_ctx: int, sum_ctx: int, n: int) -> int:
    """Cuts of the key range that uneven contexts ask for, whatever the number of sequences: a
    sequence's keys are walked by the waves of one workgroup per kv head and cut, so one long
    context among short ones sets the step's time (measured at 32 sequences of 32 heads: 31
    contexts of 600 and one of 32,768 take 153 us with one cut, 60 with eight; one of 8,192
    takes 45 and 33).  The longest walk is brought down to about twice the mean one; a power of
    two, so that captured launches change seldom."""
    if n <= 1 or max_ctx < 4 * KEYS_PER_CUT or sum_ctx <= 0:
        return 1
    want = min(max_ctx * n / (2.0 * sum_ctx), max_ctx // KEYS_PER_CUT, SKEW_MAX_CUTS)
    cuts = 1
    while cuts * 2 <= want:
        cuts *= 2
    return cuts


def prefill_work_rows(q_lens, prefill_seqs, group_size: int, rows_per_item: int,
                      start_pos=None) -> list[tuple]:
    """Rows (sequence row, item, -1) for every query run longer than one token: a run of ``q``
    tokens has ``q * group_size`` rows per kv head, an item covers ``rows_per_item`` of them, and
    a workgroup takes one item.  Under the causal mask an item walks the keys up to its last
    row's position (``start_pos``: the keys before each run): the items of all runs are handed
    out longest walk first, so that the short ones fill the gaps the long ones leave as compute
    units come free.  (The kernels also take two items per row, an early one paired with a late
    one, which balances the workgroups among themselves; measured once the kv heads were spread
    over the XCDs it lost to this order, which keeps twice the workgroups in flight: 2,048
    queries of 32 heads of size 64 take 58 us in pairs and 47 us one by one, 2,048 at the end
    of 8,192 keys 398 and 301.)"""
    rows = []
    for b in prefill_seqs:
        n = -(-q_lens[b] * group_size // rows_per_item)
        before = start_pos[b] if start_pos is not None else 0
        rows += [(before + min(q_lens[b], -(-(i + 1) * rows_per_item // group_size)), b, i) for i in range(n)]
    rows.sort(key=lambda r: -r[0])        # stable: equal walks stay in sequence and item order
    return [(b, i, -1) for _, b, i in rows]


@register_mixer("attention")
class PagedAttention(Mixer):
    """``window``: ``None`` attends to every earlier position, ``w`` to the last ``w``.
    ``rotary``: the rotation of q and k, or ``None`` for none.  ``score_slopes``: one number per
    q head, or ``None``; the score of key ``j`` for a query at position ``p`` of head ``h`` then
    gets ``score_slopes[h] * (j - p)`` added, a position encoding by distance that lives in the
    scores instead of in q and k.
    ``keep_first``: with a window, the first so many keys of a sequence stay visible behind it
    (key ``j`` is seen from position ``p`` iff ``j <= p`` and (``p - j < window`` or
    ``j < keep_first``)), and their pages are kept.
    ``value_dim``: size of a value head where it differs from the query/key size ``head_dim``.
    The kernels take one size for both: the heads of the projections are padded with zero rows
    (zero columns of the output projection) up to the larger of the two, rounded up to the
    kernels' step of 16, which changes no score and no output.
    ``gated``: the heads' outputs are multiplied by ``sigmoid(W_g x)`` element by element before
    the output projection; ``W_g`` reads the same input as the other projections and rides in
    their product.
    ``own_kv``: ``False`` for a mixer without key and value projections, which reads the cache
    of another call (``LayerCall.cache_of``) with queries, mask and gate of its own.
    ``names``: checkpoint names of the matrices under the prefix, by ``q k v o g``.
    ``qk_norm``: ``(name of q's weight, name of k's weight, eps)`` under the prefix: every q head
    and every k head is divided by its root mean square over ``head_dim`` and multiplied by a
    weight vector ``[head_dim]`` that the heads share, before the rotation; in fp32, in the
    kernel that also rotates and writes the cache.
    ``sink``: name of a tensor ``[num_heads]`` under the prefix: the softmax's denominator of
    head ``h`` gets one more term ``exp(sink[h])`` (not scaled), which takes weight from the
    keys and has no value.
    ``score_cap``: the scaled score ``s`` becomes ``score_cap * tanh(s / score_cap)`` before
    mask and softmax.
    ``q_temp``: ``(coef, every)``; the query of position ``p`` is multiplied by
    ``1 + coef * ln(floor((p + 1) / every) + 1)``, in the kernel that norms q and k (so it goes
    with ``qk_norm``).
    ``row_norm``: ``(name of q's weight, name of k's weight, eps)`` under the prefix: q as a whole
    (all heads at once) and k as a whole are each divided by their root mean square and
    multiplied by a weight vector of their full size (``[heads * head_dim]``,
    ``[kv heads * head_dim]``), before the rotation; the projection's sums are kept in fp32 up to
    there.  ``bias``: ``(name of q's bias, name of k's bias)`` under the prefix, added to the
    projections in fp32 (goes with ``row_norm``, whose kernel adds them).
    ``values_are_keys``: there is no value projection; a token's values are its keys as they
    leave the projection (bias included), before norm and rotation (goes with ``row_norm`` and a
    rotation of neighbouring pairs or none).
    ``chunk``: instead of a window, positions are cut into chunks of so many, counted from
    position 0 of the sequence, and a query sees only the keys of its own chunk; pages wholly
    behind the chunk are given back.
    ``head_gate``: name of a matrix ``[num_heads, hidden]`` under the prefix: head ``h``'s output is
    multiplied by ``sigmoid(W x)_h``, one number per head, from the same input as the
    projections; a product of its own with fp32 sums stored in fp32.
    ``out_scale``: a constant on the heads' outputs, applied in fp32 ahead of the (linear) output
    projection."""

    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "g": "g_proj.weight"}

    replayable = True
    settles_residual = True  # its norm kernel adds what is owed to the stream

    def __init__(self, prefix: str, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 rotary: RotaryPositions | None, scale: float | None = None,
                 window: int | None = None, score_slopes=None, keep_first: int = 0,
                 value_dim: int | None = None, gated: bool = False, own_kv: bool = True,
                 names: dict[str, str] | None = None,
                 qk_norm: tuple[str, str, float] | None = None, sink: str | None = None,
                 score_cap: float | None = None, q_temp: tuple[float, int] | None = None,
                 row_norm: tuple[str, str, float] | None = None, bias: tuple[str, str] | None = None,
                 values_are_keys: bool = False, chunk: int | None = None, head_gate: str | None = None,
                 out_scale: float = 1.0) -> None:
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.dk = int(head_dim)
        self.dv = int(value_dim) if value_dim is not None else self.dk
        padded = -(-max(self.dk, self.dv) // 16) * 16
        if min(self.dk, self.dv) <= 0 or padded > 256:
            raise ValueError(
                f"attention kernels take head sizes up to 256, got {self.dk} / {self.dv}")
        if value_dim is None and head_dim % 16:
            raise ValueError(
                f"attention kernels take head sizes in steps of 16 up to 256, got {head_dim}")
        self.prefix = prefix
        self.hidden, self.H, self.KV, self.d = int(hidden), int(num_heads), int(num_kv_heads), padded
        self.rotary = rotary
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.dk)
        self.window = int(window) if window else None
        self.chunk = int(chunk) if chunk else None
        if self.chunk is not None and (self.chunk < 0 or self.window is not None):
            raise ValueError("chunks are positive and take the place of a window")
        self.keep_first = int(keep_first) if self.window else 0
        if self.keep_first < 0:
            raise ValueError(f"keep_first must not be negative, got {keep_first}")
        self.gated, self.own_kv = bool(gated), bool(own_kv)
        self.names = dict(self.NAMES, **(names or {}))
        self.score_slopes = None if score_slopes is None else [float(v) for v in score_slopes]
        if self.score_slopes is not None and len(self.score_slopes) != self.H:
            raise ValueError(f"score_slopes needs one number per q head ({self.H}), got {len(self.score_slopes)}")
        self.slopes: torch.Tensor | None = None
        self.qk_norm, self.sink = qk_norm, sink
        if qk_norm is not None and not own_kv:
            raise ValueError("a norm of q and k goes with key and value projections of the mixer's own")
        self.q_norm_w = self.k_norm_w = self.sinks = None
        self.score_cap = float(score_cap) if score_cap else None
        if self.score_cap is not None and not self.score_cap > 0.0:
            raise ValueError(f"score_cap must be positive, got {score_cap}")
        self.q_temp = (float(q_temp[0]), int(q_temp[1])) if q_temp else None
        if self.q_temp is not None and (qk_norm is None or self.q_temp[1] < 1):
            raise ValueError("q_temp goes with qk_norm and a positive step")
        self.row_norm, self.bias, self.values_are_keys = row_norm, bias, bool(values_are_keys)
        if row_norm is not None and (qk_norm is not None or not own_kv or gated):
            raise ValueError("a norm over whole q and k rows goes with key projections of the mixer's own, "
                             "without a norm per head and without an element-wise gate")
        if (bias is not None or self.values_are_keys) and row_norm is None:
            raise ValueError("biases on q and k, and values that are the keys, go with row_norm")
        if self.values_are_keys and (self.dv != self.dk or (rotary is not None and not rotary.interleaved)):
            raise ValueError("values that are the keys have the keys' size and order (a rotation of "
                             "neighbouring pairs, or none)")
        self.head_gate, self.out_scale = head_gate, float(out_scale)
        self.q_bias = self.k_bias = self.w_head_gate = None
        # a chunk's keys all lie within the last `chunk` positions
        self.cache_spec = CacheSpec(attention_pages(self.KV, self.d), self.window or self.chunk, self.keep_first)
        self.w_qkv: torch.Tensor | None = None
        self.w_o: torch.Tensor | None = None

    def _matrices(self) -> list[str]:
        kv = (["k"] if self.values_are_keys else ["k", "v"]) if self.own_kv else []
        return ["q"] + kv + (["g"] if self.gated else [])

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, H, KV = self.hidden, self.H, self.KV
        shapes = {"q": (H * self.dk, h), "k": (KV * self.dk, h), "v": (KV * self.dv, h),
                  "g": (H * self.dv, h)}
        out = {self._name(self.names[n]): WeightSpec(shapes[n]) for n in self._matrices()}
        out[self._name(self.names["o"])] = WeightSpec((h, H * self.dv))
        if self.qk_norm is not None:
            out[self._name(self.qk_norm[0])] = WeightSpec((self.dk,), init="norm", std=0.1)
            out[self._name(self.qk_norm[1])] = WeightSpec((self.dk,), init="norm", std=0.1)
        if self.sink is not None:
            out[self._name(self.sink)] = WeightSpec((H,), std=1.0)
        if self.row_norm is not None:
            out[self._name(self.row_norm[0])] = WeightSpec((H * self.dk,), init="norm", std=0.1)
            out[self._name(self.row_norm[1])] = WeightSpec((KV * self.dk,), init="norm", std=0.1)
        if self.bias is not None:
            out[self._name(self.bias[0])] = WeightSpec((H * self.dk,), std=0.5)
            out[self._name(self.bias[1])] = WeightSpec((KV * self.dk,), std=0.5)
        if self.head_gate is not None:
            out[self._name(self.head_gate)] = WeightSpec((H, h))
        return out

    def _padded_heads(self, w: torch.Tensor, heads: int, size: int, perm=None) -> torch.Tensor:
        """Rows of ``heads`` heads of ``size`` rows each, every head padded with zero rows up to
        the kernels' head size (and its rows permuted first, if asked)."""
        w = w.view(heads, size, -1)
        if perm is not None:
            w = w[:, perm]
        if size != self.d:
            w = torch.cat([w, w.new_zeros(heads, self.d - size, w.shape[2])], dim=1)
        return w.reshape(heads * self.d, -1)

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        mats = {n: tensors[self._name(self.names[n])] for n in self._matrices()}
        if len({m.dtype for m in mats.values()}) > 1:
            mats = {n: m.float() for n, m in mats.items()}
        # The kernels rotate neighbouring elements (2i, 2i+1); the checkpoint pairs element i
        # with i + rot/2.  Permuting the rows of the q and k projections inside each head moves
        # the checkpoint's pairs next to each other; q.k does not depend on the order, v and the
        # output projection keep theirs.
        perm = self.pair_permutation()
        rows = [self._padded_heads(mats["q"], self.H, self.dk, perm)]
        if self.own_kv:
            rows.append(self._padded_heads(mats["k"], self.KV, self.dk, perm))
            if not self.values_are_keys:
                rows.append(self._padded_heads(mats["v"], self.KV, self.dv))
        if self.gated:
            rows.append(self._padded_heads(mats["g"], self.H, self.dv))
        # one product for all projections: rows of q heads, then k heads, then v heads, then
        # the gate's heads
        self.w_qkv = torch.cat(rows, dim=0).contiguous()
        w_o = tensors[self._name(self.names["o"])]
        if self.dv != self.d:
            w_o = torch.cat([w_o.view(self.hidden, self.H, self.dv),
                             w_o.new_zeros(self.hidden, self.H, self.d - self.dv)], dim=2)
            w_o = w_o.reshape(self.hidden, self.H * self.d).contiguous()
        self.w_o = w_o
        self.norm_eps = None
        if self.qk_norm is not None:
            self.q_norm_w = tensors[self._name(self.qk_norm[0])].float().contiguous()
            self.k_norm_w = tensors[self._name(self.qk_norm[1])].float().contiguous()
        if self.sink is not None:
            self.sinks = tensors[self._name(self.sink)].float().contiguous()
        if self.row_norm is not None:
            # weights and biases go by (head, element): in the order the rows of q and k were given
            def by_head(name: str, heads: int) -> torch.Tensor:
                return tensors[self._name(name)].float().view(heads, self.dk)[:, perm.to(w_o.device)].reshape(-1).contiguous()
            self.q_norm_w, self.k_norm_w = by_head(self.row_norm[0], self.H), by_head(self.row_norm[1], self.KV)
            if self.bias is not None:
                self.q_bias, self.k_bias = by_head(self.bias[0], self.H), by_head(self.bias[1], self.KV)
        if self.head_gate is not None:
            # one row per head, padded with zero rows to a multiple of 16 (which every product
            # kernel takes); in the engine's type, its 32-bit sums are stored in fp32
            g = tensors[self._name(self.head_gate)]
            self.w_head_gate = torch.cat([g, g.new_zeros(-(-self.H // 16) * 16 - self.H, self.hidden)], dim=0).contiguous()
        if self.score_slopes is not None:
            self.slopes = torch.tensor(self.score_slopes, dtype=torch.float32, device=self.w_o.device)

    def pair_permutation(self) -> torch.Tensor:
        """``perm[new] = old`` within a head: new elements 2i and 2i+1 are the checkpoint's
        elements i and i + rot/2; elements beyond the rotary width stay."""
        rot = self.rotary.rot_dim if self.rotary is not None else 0
        perm = torch.arange(self.dk)
        if rot and getattr(self.rotary, "interleaved", False):
            return perm      # the checkpoint's pairs are neighbours already
        for i in range(rot // 2):
            perm[2 * i], perm[2 * i + 1] = i, i + rot // 2
        return perm

    def after_projection(self, qkv: torch.Tensor, step) -> None:
        """A place for a variant to change the projected rows before they are rotated and
        written to the cache (a bias on the projections, a norm per head of q and k): ``qkv``
        is ``[N, (H + 2 KV) d]`` in the step's activation type, q heads, then k heads, then v
        heads, each head's rotary pairs as neighbouring elements (``pair_permutation``); it is
        changed in place.  The default does nothing.  A subclass that overrides it runs
        projection, this, and rotation + cache write as kernels of their own in every step
        (the kernel that fuses the three has no place for it) and keeps its norm a kernel."""

    def _hooked(self) -> bool:
        return type(self).after_projection is not PagedAttention.after_projection

    def _plain(self) -> bool:
        """Whether the product holds q, k and v and nothing else, and nothing but the rotation
        lies between it and the cache."""
        return self.own_kv and not self.gated and self.qk_norm is None and self.row_norm is None

    def absorb_norm(self, norm) -> bool:
        if self._hooked() or not self._plain() or self.head_gate is not None:
            return False
        if self.norm_eps is not None or not getattr(norm, "foldable_into", lambda m: False)(self.w_qkv):
            return False
        self.w_qkv = (self.w_qkv.float() * norm.weight.float()[None, :]).to(torch.bfloat16).contiguous()
        self.norm_eps = norm.eps
        return True

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        mods = {"elementwise", "gemm_generic", "attn_generic"}
        if dtype == torch.bfloat16:
            mods |= {"gemm_bf16", "attn_mfma"}
        return mods

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size()
                   for t in (*map(ops.plain_of, (self.w_qkv, self.w_o)), *self._small()) if t is not None)

    def _small(self) -> list[torch.Tensor]:
        gate = ops.plain_of(self.w_head_gate) if self.w_head_gate is not None else None
        return [t for t in (self.q_norm_w, self.k_norm_w, self.sinks, self.q_bias, self.k_bias, gate)
                if t is not None]

    def held_tensors(self) -> list[torch.Tensor]:
        gate = ops.copies_of(self.w_head_gate) if self.w_head_gate is not None else []
        return (ops.copies_of(self.w_qkv) + ops.copies_of(self.w_o) + gate
                + [t for t in self._small() if t.dim() == 1])

    def seal(self) -> None:
        self.w_qkv, self.w_o = ops.streamed(ops.plain_of(self.w_qkv)), ops.streamed(ops.plain_of(self.w_o))
        if self.w_head_gate is not None:
            self.w_head_gate = ops.streamed(ops.plain_of(self.w_head_gate))

    # ------------------------------------------------------------------ launch planning
    def launch_key(self, shape) -> tuple[int, int]:
        """(context cell, cuts for uneven contexts): all that this part's decode launches depend
        on besides the padded batch size.  A cell is ``KEYS_PER_CUT`` keys of the longest
        context (of the window, for a windowed layer), and the plan is made for the cell's lower
        edge."""
        seen = self.window or self.chunk
        ctx = min(shape.max_ctx, seen + self.keep_first) if seen else shape.max_ctx
        cell = min(ctx // KEYS_PER_CUT, MAX_CUTS)
        return cell, skew_cuts(max(cell * KEYS_PER_CUT, 1), shape.sum_ctx, shape.n)

    def _decode_cuts(self, step, on_matrix_cores: bool) -> int:
        cell, skew = self.launch_key(step.decode_shape)
        chunks = -(-(self.H // self.KV) // (16 if on_matrix_cores else 8))
        workgroups = max(1, step.n_decode * self.KV * chunks)
        # the vector-ALU kernel's waves take 64 keys at a time and its workgroups are light: it is
        # worth cutting down to one such block per cut and to two workgroups per compute unit
        # (measured in fp32 at the 1B shape, 600 keys: 2.48 to 2.37 ms a step at batch 8, 1.91 to
        # 1.77 at batch 1)
        finest = cell if on_matrix_cores else 8 * cell
        room = compute_units(step.device) * (1 if on_matrix_cores else 2)
        cuts = max(1, min(room // workgroups, finest, MAX_CUTS))
        return max(cuts, min(skew, max(1, cell)))

    def _prefill_work(self, step, act: torch.dtype, block_size: int):
        """(work rows on the device, rows per item) of the step's query runs, or ``(None, 0)``.
        Items of two row tiles per wave halve what a key block costs per row (its page lookups,
        staging and barrier) and halve the workgroups.  They are taken where the kernel has them
        and their workgroups alone are as many as the chip holds of the one-tile kernel at a
        time (so that short items are left to fill in behind the long ones), or give every
        compute unit two while every run starts at least its own length into its sequence (then
        all items walk long and nothing needs filling in).  Measured at 32 heads over 8 kv heads,
        one against two tiles: 2,048 queries from position 0, 47 against 55 us at head size 64
        and 70 against 82 at 128; 4,096 queries, 140 against 114 and 231 against 196; 2,048
        queries behind 2,048 keys, 106 against 100 and 209 against 151.  The layers of a model
        that agree on group size and item share the rows through the step's scratch."""
        if not step.prefill_seqs:
            return None, 0
        G = self.H // self.KV
        key = ("attention.prefill_work", G, self.KV, self.d, act, block_size)
        found = step.scratch.get(key)
        if found is None:
            units = compute_units(step.device)
            per_item = ops.prefill_rows_per_item(act, self.d, block_size, 2)
            rows = prefill_work_rows(step.q_lens, step.prefill_seqs, G, per_item, step.start_pos)
            groups = len(rows) * self.KV
            fills = groups >= ops.prefill_blocks_per_cu(act, self.d, block_size, 1) * units
            deep = groups >= 2 * units and all(step.start_pos[b] >= step.q_lens[b] for b in step.prefill_seqs)
            if not (fills or deep):
                per_item = ops.prefill_rows_per_item(act, self.d, block_size, 1)
                rows = prefill_work_rows(step.q_lens, step.prefill_seqs, G, per_item, step.start_pos)
            found = (step.upload_ints([x for row in rows for x in row]).view(-1, 3), per_item)
            step.scratch[key] = found
        return found

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations, or (after ``absorb_norm``) the fp32 residual stream."""
        n = x.shape[0]
        H, KV, d = self.H, self.KV, self.d
        ws = step.ws
        act = step.act_dtype
        table = step.block_tables[layer.group]
        cos, sin = (self.rotary.cos, self.rotary.sin) if self.rotary is not None else (None, None)
        rms = self.norm_eps
        owed = None
        if rms is not None and not ops.bf16_kernel_takes(x, self.w_qkv, True):
            # too many rows for the norm to ride in the projection: a norm kernel of its own,
            # which also adds what the layer before still owes the stream
            normed = ws.buf("normed", (n, self.hidden), act)
            ops.rmsnorm(x, None, rms, normed, add=step.take_owed(residual))
            x, rms = normed, None
        fused = (not self._hooked() and self.qk_norm is None and self.row_norm is None
                 and ops.bf16_kernel_takes(x, self.w_qkv, rms is not None, True)
                 and layer.k_pages.dtype == torch.bfloat16)
        if fused and rms is not None:
            # what the layer before owes the stream rides in this projection's loads and is
            # added to the stream by the output projection
            owed = step.take_owed(residual)
            if owed is not None and (owed.dtype != torch.bfloat16 or owed.stride() != x.stride()):
                ops.add_rows(residual, owed)
                owed = None
        else:
            step.settle()
        g0 = H * d     # where the gate's columns begin in a row of qkv
        if fused:
            # one kernel: (norm,) projection, rotary, cache write; a gate's columns land behind q
            extra = H * d if self.gated else 0
            qkv = ws.buf("q_rot", (n, H * d + extra), act)
            ops.gemm_qkv_rope(x, self.w_qkv, qkv, step.positions, step.seq_of_token, cos, sin, table,
                              layer.k_pages, layer.v_pages, H, KV if self.own_kv else 0, d,
                              write_kv=layer.owns_cache and self.own_kv, rms_eps=rms, a_owed=owed,
                              extra_cols=extra)
        elif self.row_norm is not None:
            # the projection's 32-bit sums are kept up to the norm: biases, the values (which may
            # be the keys as they stand), the norm over whole rows, rotation and cache write are
            # one kernel, with one rounding behind it
            proj = ws.buf("qkv_f32", (n, self.w_qkv.shape[0]), torch.float32)
            ops.gemm(x, self.w_qkv, proj)
            qkv = ws.buf("q_rot", (n, H * d), act)
            ops.rownorm_rope_kvwrite(proj, qkv, step.positions, step.seq_of_token, cos, sin, table,
                                     layer.k_pages, layer.v_pages, H, KV, d, self.q_norm_w, self.k_norm_w,
                                     self.dk, self.row_norm[2], q_bias=self.q_bias, k_bias=self.k_bias,
                                     values_are_keys=self.values_are_keys, write_kv=layer.owns_cache)
        else:
            g0 = (H + (2 * KV if self.own_kv else 0)) * d
            qkv = ws.buf("qkv", (n, self.w_qkv.shape[0]), act)
            ops.gemm(x, self.w_qkv, qkv)
            self.after_projection(qkv, step)
            if self.qk_norm is not None:
                ops.qknorm_rope_kvwrite(qkv, step.positions, step.seq_of_token, cos, sin, table,
                                        layer.k_pages, layer.v_pages, H, KV, d, self.q_norm_w,
                                        self.k_norm_w, self.dk, self.qk_norm[2],
                                        write_kv=layer.owns_cache, q_temp=self.q_temp)
            elif self.own_kv or self.rotary is not None:
                ops.rope_kvwrite(qkv, step.positions, step.seq_of_token, cos, sin, table,
                                 layer.k_pages, layer.v_pages, H, KV, d,
                                 write_kv=layer.owns_cache and self.own_kv)
        head_gates = None
        if self.w_head_gate is not None:
            head_gates = ws.buf("attn_head_gates", (n, self.w_head_gate.shape[0]), torch.float32)
            ops.gemm(x, self.w_head_gate, head_gates)
        out = ws.buf("attn_out", (n, H * d), act)
        window, chunk = self.window or 0, self.chunk or 0
        bs = layer.k_pages.shape[2]
        work, rows_per_item = self._prefill_work(step, act, bs)
        gate = qkv[:, g0:g0 + H * d] if self.gated else None
        # the matrix-core kernels gate their output as they store it
        gate_in_kernel = gate if gate is not None and ops.attention_on_matrix_cores(act, bs) else None
        if work is not None:
            ops.attn_prefill(qkv, layer.k_pages, layer.v_pages, table, step.cu_q, step.ctx_lens,
                             work, out, H, KV, d, self.scale, window, self.slopes, rows_per_item,
                             keep_first=self.keep_first, gate=gate_in_kernel, sinks=self.sinks,
                             score_cap=self.score_cap, chunk=chunk)
        if step.n_decode:
            splits = self._decode_cuts(step, ops.attention_on_matrix_cores(act, bs))
            workspace = None
            if splits > 1:
                workspace = (ws.buf("decode_part_acc", (step.n_decode * H * splits * d,), torch.float32),
                             ws.buf("decode_part_ml", (step.n_decode * H * splits * 2,), torch.float32))
            ops.attn_decode(qkv, layer.k_pages, layer.v_pages, table, step.decode_seq_ids,
                            step.n_decode, step.cu_q, step.ctx_lens, out, H, KV, d, self.scale,
                            window, splits, workspace,
                            token_is_seq=step.decode_seq_ids is None and work is None,
                            slopes=self.slopes, keep_first=self.keep_first, gate=gate_in_kernel,
                            sinks=self.sinks, score_cap=self.score_cap, chunk=chunk)
        if gate is not None and gate_in_kernel is None:
            ops.sigmoid_gate(out, gate)
        if head_gates is not None or self.out_scale != 1.0:
            ops.head_gate(out, head_gates, H, d, self.out_scale)
        add_product(step, out, self.w_o, residual, owed=owed)
