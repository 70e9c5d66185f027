"""``Ludelix``: how a Ludelix configuration becomes a list of parts.

A pre-norm decoder in which every layer is described by itself in ``config.json``:
``x += mixer(N1(x))`` and, where the layer has a feed-forward, ``x += ff(N2(x))``, RMS norms with
plain weights.  The mixer is one of three.  *Gated linear attention*: a matrix memory per head
whose key rows decay by gates of the input.  *Attention whose values are its keys*: grouped
queries with biases on q and k, a norm over the whole of q and of k, neighbouring pairs rotated
with frequencies scaled by wavelength, a sliding window and a sink in the softmax.  *Two mixers
side by side*: attention within chunks of positions (halves rotated against each other with
YaRN-stretched frequencies, one sigmoid gate per head) beside a retention (a matrix memory with
one constant decay per head), each times a constant.  The feed-forward is dense with a squared
relu, or a layer of experts that a table chooses by the token's id, plus a shared expert behind
a sigmoid gate per token.  The logits come from the embedding table.  Checkpoint names:
``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.{q,k,v,g,o,norm,a1,a2,a2.b}`` (gla),
``l<i>.mix.{q,q.b,k,k.b,q.norm,k.norm,sink,o}`` (attention),
``l<i>.mix.left.{q,k,v,g,o}`` and ``l<i>.mix.right.{q,k,v,g,o}`` (side by side),
``l<i>.mlp.{up,down}`` (dense), ``l<i>.mlp.e<j>.{gate,up,down}``, ``l<i>.mlp.table``,
``l<i>.mlp.shared.{gate,up,down,sg}`` (experts), ``final.norm``.
"""

from __future__ import annotations

from kvforge_amd.config.ludelix import LudelixConfig, LudelixRotary, WavelengthScaling
from kvforge_amd.config.model import RopeScaling
from kvforge_amd.parts.base import ModelSpec
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.parts.positions import YarnStretch
from kvforge_amd.registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, part_class,
                                  register_architecture)

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o"}
DENSE_NAMES = {"up": "up", "down": "down"}


def build_ludelix(cfg: LudelixConfig) -> ModelSpec:
    norm_cls = part_class(NORMS, "rmsnorm_named", "norm")
    attn_cls = part_class(MIXERS, "attention", "mixer")
    memory_cls = part_class(MIXERS, "linear_memory", "mixer")
    pair_cls = part_class(MIXERS, "pair", "mixer")
    dense_cls = part_class(FEED_FORWARDS, "plain", "feed-forward")
    moe_cls = part_class(FEED_FORWARDS, "moe", "feed-forward")
    block_cls = part_class(BLOCKS, "pre_norm", "block")
    rotary_cls = part_class(POSITIONS, "rotary", "position encoding")
    w, eps = cfg.width, cfg.norm_eps
    rotaries: dict[LudelixRotary, object] = {}    # layers with equal rotations share the tables

    def rotary_of(rot: LudelixRotary | None):
        if rot is None:
            return None
        if rot not in rotaries:
            sc = rot.scaling
            if isinstance(sc, WavelengthScaling):
                sc = RopeScaling("llama3", sc.factor, sc.low, sc.high, sc.original)
            elif sc is not None:
                sc = YarnStretch(sc.factor, sc.original, sc.fast, sc.slow)
            rotaries[rot] = rotary_cls(rot.dims, rot.base, sc, interleaved=rot.pairs == "neighbours")
        return rotaries[rot]

    blocks = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        if layer.type == "gla":
            mixer = memory_cls(f"{p}.mix", w, m.heads, m.dim, m.vdim, eps, gate_tau=m.tau, gate_rank=m.rank,
                               q_scale=float(m.dim) ** -0.5, head_weight=True)
        elif layer.type == "attention":
            mixer = attn_cls(f"{p}.mix", w, m.heads, m.kv_heads, m.dim, rotary_of(m.rot), scale=m.scale,
                             window=m.window, value_dim=m.dim, names=ATTENTION_NAMES,
                             row_norm=("q.norm", "k.norm", eps),
                             bias=("q.b", "k.b"), values_are_keys=True, sink="sink")
        else:
            lt, rt = m.left, m.right
            left = attn_cls(f"{p}.mix.left", w, lt.heads, lt.kv_heads, lt.dim, rotary_of(lt.rot), scale=lt.scale,
                            value_dim=lt.vdim, names=ATTENTION_NAMES, chunk=lt.chunk, head_gate="g",
                            out_scale=m.left_scale)
            right = memory_cls(f"{p}.mix.right", w, rt.heads, rt.dim, rt.vdim, eps, head_decays=rt.decay,
                               rotary=rotary_of(rt.rot), k_scale=float(rt.dim) ** -0.5, head_weight=False,
                               out_scale=m.right_scale)
            mixer = pair_cls(left, right)
        ffn = ffn_norm = None
        if layer.mlp is not None:
            f = layer.mlp
            if f.kind == "dense":
                ffn = dense_cls(f"{p}.mlp", w, f.ff, "relu2", names=DENSE_NAMES)
            else:
                ffn = moe_cls(f"{p}.mlp", w, f.ff, f.experts, f.top, 0, f.shared_ff, table_vocab=cfg.vocab_size,
                              shared_gate=bool(f.shared_ff))
            ffn_norm = norm_cls(f"{p}.norm2", w, eps)
        blocks.append(block_cls(norm_cls(f"{p}.norm1", w, eps), mixer, ffn_norm, ffn))
    return ModelSpec(config=cfg, embedding=TokenEmbedding("", cfg.vocab_size, w, tensor="embed"),
                     blocks=blocks, final_norm=norm_cls("final.norm", w, eps),
                     head=LMHead("", cfg.vocab_size, w, tied_to="embed"),
                     positions=list(rotaries.values()))


register_architecture(LudelixConfig.NAME, LudelixConfig, build_ludelix)
