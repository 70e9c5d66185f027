"""Latent attention: keys and values of all heads are read out of one small latent vector per
token, which (with one rotated key part that the heads share) is all the cache holds.

For a token with input ``x``: ``q = W_q x`` holds per head ``dim`` plain and ``rot_dim`` rotated
elements; ``W_dkv x`` holds the latent ``c`` (``kv_rank`` elements, RMS-normed with a weight) and
the shared key part ``k_r`` (``rot_dim`` elements, rotated like the queries' part).  Head ``h``
scores a key as ``(q_h . W_uk_h c + q_r_h . k_r) * scale`` and its value is ``W_uv_h c``.

Because ``q_h . (W_uk_h c) = (W_uk_h^T q_h) . c``, the read-outs never touch the keys: the
queries are taken through ``W_uk_h^T`` once (``ops.head_product``), attention runs with ONE
key/value head over pages of ``[k_r | c]`` (the built-in paged kernels, window and sink
included), and the weighted sums of ``c`` are read out per head by ``W_uv_h`` before the output
projection.  A page row is ``rot_dim + kv_rank`` elements (rounded up to the kernels' step of
16) whatever the number of heads.
"""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.attention import PagedAttention
from kvforge_amd.parts.base import CacheSpec, LayerState, WeightSpec, add_product, attention_pages
from kvforge_amd.parts.positions import RotaryPositions
from kvforge_amd.registry import register_mixer


@register_mixer("latent_attention")
class LatentAttention(PagedAttention):
    """``names``: checkpoint names under the prefix, by ``q dkv dkv_norm uk uv o``.  ``rotary``:
    the rotation of the ``rot_dim`` parts (its width must be ``rot_dim`` at most).  ``window``,
    ``sink``, ``scale``: as in ``PagedAttention``, whose launch planning and kernels this
    mixer uses with one kv head of ``rot_dim + kv_rank`` elements."""

    LATENT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o"}

    replayable = True
    settles_residual = False

    def __init__(self, prefix: str, hidden: int, num_heads: int, head_dim: int, rot_dim: int,
                 value_dim: int, kv_rank: int, rotary: RotaryPositions | None, scale: float,
                 norm_eps: float, window: int | None = None, sink: str | None = None,
                 names: dict[str, str] | None = None) -> None:
        self.prefix, self.hidden, self.H, self.KV = prefix, int(hidden), int(num_heads), 1
        self.dim, self.rot, self.dv_out, self.rank = int(head_dim), int(rot_dim), int(value_dim), int(kv_rank)
        if min(self.H, self.dv_out, self.rank) <= 0 or self.dim < 0 or self.rot < 0 or self.dim + self.rot <= 0:
            raise ValueError(f"latent attention: sizes must be positive, got heads {num_heads}, "
                             f"{head_dim} + {rot_dim}, values {value_dim}, rank {kv_rank}")
        self.d = -(-(self.rot + self.rank) // 16) * 16
        if self.d > 256:
            raise ValueError(f"attention kernels take heads up to 256 elements; rot_dim + kv_rank is "
                             f"{self.rot + self.rank}")
        self.dk = self.dv = self.d
        self.rotary = rotary
        if rotary is not None and (rotary.rot_dim > self.rot or not rotary.interleaved):
            raise ValueError("latent attention rotates neighbouring pairs within its rot_dim part")
        self.scale, self.norm_eps_c = float(scale), float(norm_eps)
        if not self.scale > 0.0:
            raise ValueError(f"scale must be positive, got {scale}")
        self.window = int(window) if window else None
        self.keep_first = 0
        self.names = dict(self.LATENT_NAMES, **(names or {}))
        self.sink = sink
        self.gated, self.own_kv, self.qk_norm = False, True, None
        self.score_slopes = self.slopes = self.sinks = None
        self.score_cap = self.q_temp = None
        self.cache_spec = CacheSpec(attention_pages(1, self.d), self.window, 0)
        self.w_in = self.w_uk_t = self.w_uv = self.w_o = self.c_norm_w = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, H = self.hidden, self.H
        n = lambda key: self._name(self.names[key])  # noqa: E731
        out = {n("q"): WeightSpec((H * (self.dim + self.rot), h)),
               n("dkv"): WeightSpec((self.rank + self.rot, h)),
               n("dkv_norm"): WeightSpec((self.rank,), init="norm", std=0.1),
               n("uk"): WeightSpec((H * self.dim, self.rank)),
               n("uv"): WeightSpec((H * self.dv_out, self.rank)),
               n("o"): WeightSpec((h, H * self.dv_out))}
        if self.sink is not None:
            out[self._name(self.sink)] = WeightSpec((H,), std=1.0)
        return out

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        t = lambda key: tensors[self._name(self.names[key])]  # noqa: E731
        q, dkv = t("q"), t("dkv")
        if q.dtype != dkv.dtype:
            q, dkv = q.float(), dkv.float()
        # one product for the queries, the latent and the shared key part
        self.w_in = torch.cat([q, dkv], dim=0).contiguous()
        # the queries go through the keys' read-out transposed: [H, rank, dim]
        self.w_uk_t = t("uk").view(self.H, self.dim, self.rank).transpose(1, 2).contiguous()
        self.w_uv = t("uv").view(self.H, self.dv_out, self.rank).contiguous()
        self.w_o = t("o")
        self.c_norm_w = t("dkv_norm").float().contiguous()
        if self.sink is not None:
            self.sinks = tensors[self._name(self.sink)].float().contiguous()

    def absorb_norm(self, norm) -> bool:
        return False

    def seal(self) -> None:
        self.w_in, self.w_o = ops.streamed(ops.plain_of(self.w_in)), ops.streamed(ops.plain_of(self.w_o))

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return super().kernel_modules(dtype) | {"latent"}

    def _small(self) -> list[torch.Tensor]:
        return [x for x in (self.w_uk_t, self.w_uv, self.c_norm_w, self.sinks) if x is not None]

    def num_bytes(self) -> int:
        return sum(x.numel() * x.element_size()
                   for x in (*map(ops.plain_of, (self.w_in, self.w_o)), *self._small()) if x is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.w_in) + ops.copies_of(self.w_o) + self._small()

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations."""
        n = x.shape[0]
        H, d, dim, rot, rank = self.H, self.d, self.dim, self.rot, self.rank
        ws, act = step.ws, step.act_dtype
        table = step.block_tables[layer.group]
        cos, sin = (self.rotary.cos, self.rotary.sin) if self.rotary is not None else (None, None)
        step.settle()
        proj = ws.buf("latent_proj", (n, self.w_in.shape[0]), act)
        ops.gemm(x, self.w_in, proj)
        qkv = ws.buf("latent_qkv", (n, (H + 2) * d), act)
        ops.latent_split(proj, qkv, self.c_norm_w, self.norm_eps_c, H, dim, rot, rank, d)
        if dim:
            # q_h -> W_uk_h^T q_h, next to the head's rotated part
            ops.head_product(proj[:, :H * (dim + rot)], dim + rot, self.w_uk_t, qkv[:, rot:H * d], d)
        ops.rope_kvwrite(qkv, step.positions, step.seq_of_token, cos, sin, table, layer.k_pages,
                         layer.v_pages, H, 1, d, write_kv=layer.owns_cache)
        out = ws.buf("attn_out", (n, H * d), act)
        bs = layer.k_pages.shape[2]
        work, rows_per_item = self._prefill_work(step, act, bs)
        window = self.window or 0
        if work is not None:
            ops.attn_prefill(qkv, layer.k_pages, layer.v_pages, table, step.cu_q, step.ctx_lens, work,
                             out, H, 1, d, self.scale, window, None, rows_per_item, sinks=self.sinks)
        if step.n_decode:
            splits = self._decode_cuts(step, ops.attention_on_matrix_cores(act, bs))
            workspace = None
            if splits > 1:
                workspace = (ws.buf("decode_part_acc", (step.n_decode * H * splits * d,), torch.float32),
                             ws.buf("decode_part_ml", (step.n_decode * H * splits * 2,), torch.float32))
            ops.attn_decode(qkv, layer.k_pages, layer.v_pages, table, step.decode_seq_ids, step.n_decode,
                            step.cu_q, step.ctx_lens, out, H, 1, d, self.scale, window, splits, workspace,
                            token_is_seq=step.decode_seq_ids is None and work is None, sinks=self.sinks)
        # the heads' weighted sums of the latent, read out by W_uv_h
        heads = ws.buf("latent_heads", (n, H * self.dv_out), act)
        ops.head_product(out[:, rot:], d, self.w_uv, heads, self.dv_out)
        add_product(step, heads, self.w_o, residual)
