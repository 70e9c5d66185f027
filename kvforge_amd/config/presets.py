"""Named model shapes, each written exactly as its ``config.json`` would read.

The reference keeps ``PRESETS`` of ModelConfig objects (src/tokenvault/model_loader.py:17-39);
here a preset is the JSON dictionary itself, so a preset goes through the same
``from_dict`` path as a model folder and no size is held anywhere else.
"""

from __future__ import annotations

from typing import Any

_LLAMA3_32 = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
              "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
_LLAMA3_8 = dict(_LLAMA3_32, factor=8.0)


def _llama(**kw: Any) -> dict[str, Any]:
    base: dict[str, Any] = {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
        "attention_bias": False, "mlp_bias": False, "rope_scaling": None,
        "tie_word_embeddings": False, "bos_token_id": None, "eos_token_id": None,
    }
    base.update(kw)
    return base


PRESETS: dict[str, dict[str, Any]] = {
    "tiny-a": _llama(
        vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=16, intermediate_size=176,
        max_position_embeddings=128, rope_theta=10000.0, rms_norm_eps=1e-5,
        tie_word_embeddings=True),
    "tiny-b": _llama(
        vocab_size=384, hidden_size=96, num_hidden_layers=3, num_attention_heads=3,
        num_key_value_heads=1, head_dim=32, intermediate_size=256,
        max_position_embeddings=256, rope_theta=500000.0, rms_norm_eps=1e-6,
        rope_scaling={"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                      "high_freq_factor": 4.0, "original_max_position_embeddings": 64}),
    # the reference's unit-test and CPU-benchmark shapes (src/tokenvault/model_loader.py:19-27)
    "tiny": _llama(
        vocab_size=512, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=16, intermediate_size=172,
        max_position_embeddings=1024, rope_theta=10000.0, rms_norm_eps=1e-6),
    "small": _llama(
        vocab_size=8192, hidden_size=512, num_hidden_layers=6, num_attention_heads=8,
        num_key_value_heads=4, head_dim=64, intermediate_size=1408,
        max_position_embeddings=2048, rope_theta=10000.0, rms_norm_eps=1e-6),
    "llama-1b": _llama(
        vocab_size=128256, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32,
        num_key_value_heads=8, head_dim=64, intermediate_size=8192,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=_LLAMA3_32, tie_word_embeddings=True),
    "llama-3b": _llama(
        vocab_size=128256, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24,
        num_key_value_heads=8, head_dim=128, intermediate_size=8192,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=_LLAMA3_32, tie_word_embeddings=True),
    "llama-8b": _llama(
        vocab_size=128256, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
        num_key_value_heads=8, head_dim=128, intermediate_size=14336,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=_LLAMA3_8),
}


def fogorax(vocab: int, width: int, layers: int, heads: int, kv_heads: int, dim: int, ff: int,
            window: int, keep_first: int, side_dim: int, max_positions: int, vdim: int | None = None,
            share_every: int = 2, eps: float = 1e-5) -> dict[str, Any]:
    """A Fogorax config.json of ``layers`` equal layers; of every ``share_every`` layers the first
    projects keys and values and the others read its cache (1: every layer its own)."""
    out = []
    for i in range(layers):
        mixer: dict[str, Any] = {"dim": dim, "heads": heads, "kv_heads": kv_heads,
                                 "mask": {"keep_first": keep_first, "size": window},
                                 "scale": float(dim) ** -0.5, "vdim": vdim if vdim is not None else dim}
        if share_every > 1 and i % share_every:
            mixer["kv_from"] = i - i % share_every
        out.append({"mixer": mixer, "mlp": {"ff": ff, "kind": "dense"}, "type": "attention"})
    return {"architecture": "Fogorax", "layers": out, "max_positions": max_positions,
            "norm": {"eps": eps}, "token_side": {"dim": side_dim} if side_dim else None,
            "vocab": vocab, "width": width}


PRESETS["fogorax-tiny"] = fogorax(vocab=300, width=96, layers=4, heads=6, kv_heads=2, dim=16, ff=160,
                                  window=24, keep_first=2, side_dim=8, max_positions=512, vdim=32)
# the layer sizes of llama-1b in this design: what its kernels are measured at
PRESETS["fogorax-1b"] = fogorax(vocab=128256, width=2048, layers=16, heads=32, kv_heads=8, dim=64,
                                ff=8192, window=1024, keep_first=4, side_dim=64, max_positions=131072)


def rudorax(vocab: int, width: int, layers: list, loop: "tuple[int, int, int] | None" = None,
            embedding_scale: float = 1.0, logit_softcap: float | None = None, eps: float = 1e-6,
            max_positions: int | None = None) -> dict[str, Any]:
    """A Rudorax config.json.  ``layers``: one ``(type, mixer, mlp)`` per layer.  For
    ``"attention"`` the mixer holds ``heads kv_heads dim vdim window rot_dims scale scaling``
    (``scaling``: ``None`` or the YaRN numbers ``factor original fast slow``) and optionally
    ``base``; for ``"mlstm"`` it holds ``heads dim vdim gate_cap``.  ``mlp``: ``None`` or
    ``ff experts top identity shared_ff``.  ``loop``: ``(start, stop, times)``."""
    out = []
    for kind, m, f in layers:
        if kind == "attention":
            mixer: dict[str, Any] = {
                "dim": m["dim"], "heads": m["heads"], "kv_heads": m["kv_heads"], "mask": {"size": m["window"]},
                "rot": {"base": float(m.get("base", 10000.0)), "dims": m["rot_dims"], "scaling": m.get("scaling")},
                "scale": float(m["scale"]), "vdim": m["vdim"]}
        else:
            mixer = {"dim": m["dim"], "gate_cap": float(m["gate_cap"]), "heads": m["heads"], "vdim": m["vdim"]}
        mlp = None
        if f is not None:
            mlp = {"expert": {"ff": f["ff"]}, "kind": "moe",
                   "router": {"experts": f["experts"], "identity": f.get("identity", 0), "top": f["top"]},
                   "shared": {"ff": f["shared_ff"]} if f.get("shared_ff") else None}
        out.append({"mixer": mixer, "mlp": mlp, "type": kind})
    cfg: dict[str, Any] = {
        "architecture": "Rudorax", "embedding": {"scale": float(embedding_scale)}, "layers": out,
        "logit_softcap": logit_softcap,
        "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]} if loop else None,
        "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if max_positions is not None:
        cfg["max_positions"] = max_positions
    return cfg


def rudorax_stack(vocab: int, width: int, pairs: int, heads: int, kv_heads: int, dim: int, window: int,
                  lstm_heads: int, lstm_dim: int, lstm_vdim: int, ff: int, experts: int, top: int,
                  identity: int, shared_ff: int, max_positions: int = 131072) -> dict[str, Any]:
    """``pairs`` times an attention layer followed by a matrix-memory layer, all with routed
    experts; the whole head rotated with frequencies stretched eightfold."""
    att = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, window=window, rot_dims=dim,
               scale=float(dim) ** -0.5, base=500000.0,
               scaling={"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0})
    rec = dict(heads=lstm_heads, dim=lstm_dim, vdim=lstm_vdim, gate_cap=15.0)
    moe = dict(ff=ff, experts=experts, top=top, identity=identity, shared_ff=shared_ff)
    return rudorax(vocab, width, [("attention", att, moe), ("mlstm", rec, moe)] * pairs,
                   embedding_scale=float(width) ** 0.5, logit_softcap=30.0, max_positions=max_positions)


PRESETS["rudorax-tiny"] = rudorax(
    vocab=320, width=96,
    layers=[("attention", dict(heads=4, kv_heads=2, dim=32, vdim=32, window=48, rot_dims=16, scale=32 ** -0.5,
                               scaling={"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}),
             dict(ff=48, experts=6, top=2, identity=1, shared_ff=64)),
            ("mlstm", dict(heads=2, dim=24, vdim=48, gate_cap=10.0),
             dict(ff=48, experts=6, top=2, identity=1, shared_ff=64))],
    loop=(0, 2, 2), embedding_scale=96 ** 0.5, logit_softcap=25.0, max_positions=1024)
# layers of the width of llama-1b: what this design's kernels are measured at
PRESETS["rudorax-1b"] = rudorax_stack(vocab=128256, width=2048, pairs=8, heads=32, kv_heads=8, dim=64,
                                      window=1024, lstm_heads=8, lstm_dim=128, lstm_vdim=256, ff=1024,
                                      experts=32, top=4, identity=2, shared_ff=2048)


def buzinex(vocab: int, width: int, layers: list, embedding_scale: float = 1.0, logit_scale: float = 1.0,
            logit_softcap: float | None = None, eps: float = 1e-6,
            max_positions: int | None = None) -> dict[str, Any]:
    """A Buzinex config.json.  ``layers``: one ``(type, mixer, ff)`` per layer.  For
    ``"attention"`` the mixer holds ``heads kv_heads dim vdim scale`` and optionally ``softcap``,
    ``q_temp`` (``(coef, every)``) and ``window``; for ``"latent_attention"`` ``heads dim
    rot_dim vdim kv_rank scale`` and optionally ``window`` and ``base``; for ``"wkv"`` ``heads
    dim decay_rank``.  ``ff``: the feed-forward's width, or ``None`` for none."""
    out = []
    for kind, m, ff in layers:
        if kind == "attention":
            qt = m.get("q_temp")
            mixer: dict[str, Any] = {
                "dim": m["dim"], "heads": m["heads"], "kv_heads": m["kv_heads"],
                "q_temp": {"coef": float(qt[0]), "every": int(qt[1])} if qt else None,
                "scale": float(m["scale"]), "softcap": m.get("softcap"), "vdim": m["vdim"]}
            if m.get("window"):
                mixer["mask"] = {"size": m["window"]}
        elif kind == "latent_attention":
            mixer = {"dim": m["dim"], "heads": m["heads"], "kv_rank": m["kv_rank"],
                     "mask": {"size": m["window"]} if m.get("window") else None,
                     "rot": ({"base": float(m.get("base", 10000.0)), "dims": m.get("rot_dims", m["rot_dim"])}
                             if m["rot_dim"] else None),
                     "rot_dim": m["rot_dim"], "scale": float(m["scale"]), "vdim": m["vdim"]}
        else:
            mixer = {"decay_rank": m["decay_rank"], "dim": m["dim"], "heads": m["heads"]}
        out.append({"mixer": mixer, "mlp": {"ff": ff, "kind": "dense"} if ff else None, "type": kind})
    cfg: dict[str, Any] = {
        "architecture": "Buzinex", "embedding": {"scale": float(embedding_scale)}, "layers": out,
        "logit_scale": float(logit_scale), "logit_softcap": logit_softcap, "norm": {"eps": eps},
        "vocab": vocab, "width": width}
    if max_positions is not None:
        cfg["max_positions"] = max_positions
    return cfg


def buzinex_stack(vocab: int, width: int, groups: int, heads: int, kv_heads: int, dim: int, latent_dim: int,
                  rot_dim: int, kv_rank: int, window: int, wkv_heads: int, wkv_dim: int, ff: int,
                  max_positions: int = 131072) -> dict[str, Any]:
    """``groups`` times (capped attention, latent attention, wkv without a feed-forward, latent
    attention), the attention layers with dense feed-forwards."""
    att = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=float(dim) ** -0.5, softcap=50.0,
               q_temp=(0.1, 4096))
    lat = dict(heads=heads, dim=latent_dim, rot_dim=rot_dim, vdim=latent_dim, kv_rank=kv_rank,
               scale=float(latent_dim + rot_dim) ** -0.5, window=window, base=1000000.0)
    rec = dict(heads=wkv_heads, dim=wkv_dim, decay_rank=64)
    return buzinex(vocab, width, [("attention", att, ff), ("latent_attention", lat, ff), ("wkv", rec, None),
                                  ("latent_attention", lat, ff)] * groups,
                   embedding_scale=float(width) ** 0.5, logit_scale=float(width) ** -0.5, logit_softcap=30.0,
                   max_positions=max_positions)


PRESETS["buzinex-tiny"] = buzinex(
    vocab=320, width=96,
    layers=[("attention", dict(heads=4, kv_heads=2, dim=16, vdim=32, scale=0.25, softcap=20.0, q_temp=(0.3, 8)), 160),
            ("latent_attention", dict(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, scale=0.2, window=24), 160),
            ("wkv", dict(heads=2, dim=24, decay_rank=8), None)],
    embedding_scale=8.0, logit_scale=0.5, logit_softcap=20.0, max_positions=1024)
# layers of the width of llama-1b: what this design's kernels are measured at
PRESETS["buzinex-1b"] = buzinex_stack(vocab=128256, width=2048, groups=4, heads=32, kv_heads=8, dim=64,
                                      latent_dim=64, rot_dim=32, kv_rank=192, window=1024, wkv_heads=32,
                                      wkv_dim=64, ff=8192)


def ludelix(vocab: int, width: int, layers: list, eps: float = 1e-5,
            max_positions: int | None = None) -> dict[str, Any]:
    """A Ludelix config.json.  ``layers``: one ``(type, mixer, mlp)`` per layer.  For ``"gla"`` the
    mixer holds ``heads dim vdim tau`` and ``rank`` (of the gates' two matrices); for
    ``"attention"`` ``heads kv_heads dim scale`` and optionally ``window``, ``rot_dims``, ``base``
    and ``scaling`` (``(factor, low, high, original)``); for ``"parallel"`` ``left`` (``heads
    kv_heads dim vdim scale`` and optionally ``chunk``, ``rot_dims``, ``base``, ``scaling``:
    ``(factor, original, fast, slow)``), ``right`` (``heads dim vdim decay`` and optionally
    ``rot_dims``, ``base``), ``left_scale`` and ``right_scale``.  ``mlp``: ``None``, an ``int``
    (a dense feed-forward of that width) or ``(ff, experts, top, shared_ff)``."""
    def rot(m: dict, scaling) -> dict | None:
        if not m.get("rot_dims"):
            return None
        out: dict[str, Any] = {"base": float(m.get("base", 10000.0)), "dims": int(m["rot_dims"])}
        if scaling:
            out["scaling"] = scaling
        return out

    out = []
    for kind, m, mlp in layers:
        if kind == "gla":
            mixer: dict[str, Any] = {"dim": m["dim"], "heads": m["heads"], "rank": m["rank"], "tau": float(m["tau"]),
                                     "vdim": m["vdim"]}
        elif kind == "attention":
            sc = m.get("scaling")
            mixer = {"dim": m["dim"], "heads": m["heads"], "kv_heads": m["kv_heads"], "scale": float(m["scale"]),
                     "vdim": m["dim"]}
            if m.get("window"):
                mixer["mask"] = {"size": m["window"]}
            r = rot(m, {"factor": float(sc[0]), "low": float(sc[1]), "high": float(sc[2]), "original": int(sc[3])}
                    if sc else None)
            if r:
                mixer["rot"] = r
        else:
            lt, rt = m["left"], m["right"]
            sc = lt.get("scaling")
            left: dict[str, Any] = {"dim": lt["dim"], "heads": lt["heads"], "kv_heads": lt["kv_heads"],
                                    "scale": float(lt["scale"]), "vdim": lt["vdim"]}
            if lt.get("chunk"):
                left["mask"] = {"size": lt["chunk"]}
            r = rot(lt, {"factor": float(sc[0]), "original": int(sc[1]), "fast": float(sc[2]), "slow": float(sc[3])}
                    if sc else None)
            if r:
                left["rot"] = r
            right: dict[str, Any] = {"decay": [float(x) for x in rt["decay"]], "dim": rt["dim"], "heads": rt["heads"],
                                     "vdim": rt["vdim"]}
            r = rot(rt, None)
            if r:
                right["rot"] = r
            mixer = {"left": left, "left_scale": float(m.get("left_scale", 1.0)), "right": right,
                     "right_scale": float(m.get("right_scale", 1.0))}
        if mlp is None:
            ff: dict[str, Any] | None = None
        elif isinstance(mlp, int):
            ff = {"ff": mlp, "kind": "dense"}
        else:
            ff = {"expert": {"ff": mlp[0]}, "kind": "moe", "router": {"experts": mlp[1], "top": mlp[2]}}
            if mlp[3]:
                ff["shared"] = {"ff": mlp[3]}
        out.append({"mixer": mixer, "mlp": ff, "type": kind})
    cfg: dict[str, Any] = {"architecture": "Ludelix", "layers": out, "norm": {"eps": eps}, "vocab": vocab,
                           "width": width}
    if max_positions is not None:
        cfg["max_positions"] = max_positions
    return cfg


def retention_decays(heads: int) -> list[float]:
    """One decay per head, ``1 - 2^(-5 - h)``: the usual spread of memory lengths."""
    return [1.0 - 2.0 ** (-5.0 - h * 6.0 / max(heads - 1, 1)) for h in range(heads)]


def ludelix_stack(vocab: int, width: int, groups: int, heads: int, kv_heads: int, dim: int, window: int,
                  mem_heads: int, mem_dim: int, mem_vdim: int, ff: int, experts: int, top: int, shared_ff: int,
                  max_positions: int = 131072) -> dict[str, Any]:
    """``groups`` times (gated linear attention, attention whose values are its keys, chunked
    attention beside a retention, attention again), the first of each group with a dense
    feed-forward, the others with experts."""
    gla = dict(heads=mem_heads, dim=mem_dim, vdim=mem_vdim, tau=16.0, rank=16)
    att = dict(heads=heads, kv_heads=kv_heads, dim=dim, scale=float(dim) ** -0.5, window=window, rot_dims=dim // 2,
               base=500000.0, scaling=(8.0, 1.0, 4.0, 8192))
    par = dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=float(dim) ** -0.5, chunk=window,
                         rot_dims=dim, base=10000.0, scaling=(8.0, 4096, 32.0, 1.0)),
               right=dict(heads=mem_heads, dim=mem_dim, vdim=mem_vdim, decay=retention_decays(mem_heads),
                          rot_dims=mem_dim, base=10000.0), left_scale=1.0, right_scale=1.0)
    moe = (ff, experts, top, shared_ff)
    return ludelix(vocab, width, [("gla", gla, top * ff + shared_ff), ("attention", att, moe), ("parallel", par, moe),
                                  ("attention", att, moe)] * groups, max_positions=max_positions)


PRESETS["ludelix-tiny"] = ludelix(
    vocab=320, width=96,
    layers=[("gla", dict(heads=2, dim=16, vdim=24, tau=8.0, rank=4), 160),
            ("attention", dict(heads=4, kv_heads=2, dim=16, scale=0.25, window=24, rot_dims=8,
                               scaling=(4.0, 1.0, 4.0, 64)), (32, 6, 2, 64)),
            ("parallel", dict(left=dict(heads=2, kv_heads=1, dim=16, vdim=32, scale=0.25, chunk=20, rot_dims=16,
                                        scaling=(4.0, 64, 16.0, 1.0)),
                              right=dict(heads=2, dim=8, vdim=16, decay=[0.9, 0.98], rot_dims=8),
                              left_scale=1.25, right_scale=0.5), None)],
    max_positions=1024)
# layers of the width of llama-1b: what this design's kernels are measured at
PRESETS["ludelix-1b"] = ludelix_stack(vocab=128256, width=2048, groups=4, heads=32, kv_heads=8, dim=64, window=1024,
                                      mem_heads=16, mem_dim=64, mem_vdim=128, ff=1024, experts=32, top=4,
                                      shared_ff=2048)


def preset_dict(name: str) -> dict[str, Any]:
    try:
        return dict(PRESETS[name])
    except KeyError:
        raise KeyError(f"unknown preset {name!r}; known: {sorted(PRESETS)}") from None
