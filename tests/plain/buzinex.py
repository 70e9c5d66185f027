"""A plain, slow Buzinex decoder: whole sequences, no cache, no carried state, one function per
mechanism, torch on the CPU in 32-bit (or 64-bit, for a truth all but free of rounding).  It is
the oracle the engine's Buzinex model is held to and shares no code with ``kvforge_amd``: it
reads ``config.json`` dictionaries and ``{checkpoint name: tensor}`` dicts itself.

The design in this file's notation (``T`` tokens of one sequence, positions ``0..T-1``):

* stream ``x_t = embed[token_t] * c`` with ``c = embedding.scale``;
* a layer is a *sandwich*: ``x += Nb(mixer(Na(x)))`` and then, if it has a feed-forward,
  ``x += Nd(ff(Nc(x)))``, every ``N`` an RMS norm with a weight vector of its own;
* mixer ``attention``: grouped queries, q and k normalised per head, no rotation; the query of
  position ``p`` is stretched by ``1 + coef * ln(floor((p + 1) / every) + 1)``; scores are
  scaled by a constant and squashed by ``cap * tanh(s / cap)``; causal softmax;
* mixer ``latent_attention``: keys and values of all heads are read out of one small latent
  vector per token (the only thing a cache would keep, beside one rotated key part that all
  heads share); sliding window; the softmax's denominator holds one more term ``exp(sink_h)``;
* mixer ``wkv``: a matrix memory per head with a data-dependent decay per key channel, a bonus
  for the current token, token shift on all five inputs, a gate on the output;
* feed-forward: ``down(silu(gate h) * up h)``;
* logits ``= cap * tanh(s * embed @ N(x) / cap)`` with the unscaled embedding table.
"""

from __future__ import annotations

import math

import torch


def stored(x: torch.Tensor, store: torch.dtype | None) -> torch.Tensor:
    """``x`` after a trip through memory in type ``store`` (rounded and widened again), or
    unchanged for ``None``: ``forward(..., store=torch.bfloat16)`` rounds what an engine serving
    in bfloat16 may keep in 16 bits between two operations, and nothing that the design wants
    in 32 bits."""
    return x if store is None else x.to(store).to(x.dtype)


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x`` divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * w


def softmax_rows(scores: torch.Tensor, visible: torch.Tensor, sink: torch.Tensor | None = None
                 ) -> torch.Tensor:
    """Weights ``[H, T, T]`` of the visible keys; ``sink [H]`` adds ``exp(sink_h)`` to every
    row's denominator and nothing else."""
    s = scores.masked_fill(~visible[None], -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None, None] - m)
    return e / den


def visible_keys(queries: int, keys: int, window: int | None = None) -> torch.Tensor:
    """``[queries, keys]``: the queries are the last ``queries`` of ``keys`` positions; position
    ``i`` sees ``j <= i`` and, under a window, only ``i - j < window``."""
    i = torch.arange(keys - queries, keys)[:, None]
    j = torch.arange(keys)[None, :]
    seen = j <= i
    return seen & (i - j < int(window)) if window else seen


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, visible: torch.Tensor,
           cap: float | None = None, sink: torch.Tensor | None = None) -> torch.Tensor:
    """``q [Tq, H, d]``, ``k [Tk, H, d]``, ``v [Tk, H, dv]`` -> ``[Tq, H, dv]``: scores scaled,
    capped, masked, softmax (with a sink, if any), weighted sum."""
    s = capped(torch.einsum("thd,shd->hts", q, k) * float(scale), cap)
    return torch.einsum("hts,shd->thd", softmax_rows(s, visible, sink), v)


# ---------------------------------------------------------------------------------- attention
def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """``1 + coef * ln(floor((p + 1) / every) + 1)`` per position, in 32-bit."""
    steps = torch.div(positions.to(torch.int64) + 1, int(every), rounding_mode="floor")
    return 1.0 + float(coef) * torch.log(steps.to(torch.float32) + 1.0)


def capped(s: torch.Tensor, cap: float | None) -> torch.Tensor:
    return s if not cap else float(cap) * torch.tanh(s / float(cap))


def attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float,
              store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    G = int(m.get("kv_heads") or H)
    dv = int(m.get("vdim") or d)
    pos = torch.arange(T)
    q = stored(h @ w[p + "q"].T, store).view(T, H, d)
    k = stored(h @ w[p + "k"].T, store).view(T, G, d)
    v = stored(h @ w[p + "v"].T, store).view(T, G, dv)
    q = norm(q, w[p + "q.norm"], eps)
    k = norm(k, w[p + "k.norm"], eps)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(pos, qt["coef"], qt["every"]).to(q.dtype)[:, None, None]
    q, k = stored(q, store), stored(k, store)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    size = (m.get("mask") or {}).get("size")
    o = attend(q, k, v, m["scale"], visible_keys(T, T, size), m.get("softcap"))
    return stored(o.reshape(T, H * dv), store) @ w[p + "o"].T


# --------------------------------------------------------------------------- latent attention
def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """``x [T, heads, n]``: elements ``2i`` and ``2i+1`` (``i < dims/2``) are turned by the angle
    ``position * base^(-2i/dims)``; the rest passes.  Angles are formed in 32-bit."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = (float(base) ** (-2.0 * i / dims)).to(torch.float32)
    a = positions.to(torch.float32)[:, None] * f[None, :]
    cos, sin = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float,
                     store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, d, r = int(m["heads"]), int(m["dim"]), int(m["rot_dim"])
    dv, rank = int(m["vdim"]), int(m["kv_rank"])
    rot = m.get("rot")
    pos = torch.arange(T)
    q = stored(h @ w[p + "q"].T, store).view(T, H, d + r)
    down = stored(h @ w[p + "dkv"].T, store)
    c = stored(norm(down[:, :rank], w[p + "dkv.norm"], eps), store)
    k_rot = down[:, None, rank:rank + r]
    q_flat, q_rot = q[..., :d], q[..., d:]
    if rot:
        q_rot = rotate_pairs(q_rot, pos, int(rot["dims"]), rot["base"])
        k_rot = rotate_pairs(k_rot, pos, int(rot["dims"]), rot["base"])
    q_rot, k_rot = stored(q_rot, store), stored(k_rot, store)
    k_flat = stored(c @ w[p + "uk"].T, store).view(T, H, d)
    v = stored(c @ w[p + "uv"].T, store).view(T, H, dv)
    size = (m.get("mask") or {}).get("size")
    sink = w[p + "sink"].to(q.dtype) if (p + "sink") in w else None
    # a head's key: its own read-out of the latent, then the part that all heads share
    o = attend(torch.cat([q_flat, q_rot], -1), torch.cat([k_flat, k_rot.expand(T, H, r)], -1), v,
               m["scale"], visible_keys(T, T, size), None, sink)
    return stored(o.reshape(T, H * dv), store) @ w[p + "o"].T


# ------------------------------------------------------------------------------------- wkv
def shifted(h: torch.Tensor) -> torch.Tensor:
    """Every token's predecessor (zeros for the first)."""
    return torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)


def wkv_recurrence(r, k, v, decay, u):
    """``r, k, v, decay [T, H, d]``, ``u [H, d]``; per head a state ``S [d, d]`` (key channel
    by value channel) that starts at zero: ``o_t = (S + diag(u) k_t v_t^T)^T r_t`` and then
    ``S <- diag(decay_t) S + k_t v_t^T``."""
    T, H, d = r.shape
    S = torch.zeros(H, d, d, dtype=r.dtype)
    out = torch.zeros(T, H, d, dtype=r.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    return out


def wkv(h: torch.Tensor, w: dict, p: str, m: dict, eps: float,
        store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    before = shifted(h)

    def mix(s: str) -> torch.Tensor:
        return stored(h + (before - h) * w[p + "mu." + s], store)

    r = stored(mix("r") @ w[p + "r"].T, store).view(T, H, d)
    k = stored(mix("k") @ w[p + "k"].T, store).view(T, H, d)
    v = stored(mix("v") @ w[p + "v"].T, store).view(T, H, d)
    g = stored(mix("g") @ w[p + "g"].T, store)
    gate = g * torch.sigmoid(g)
    low = stored(torch.tanh(mix("w") @ w[p + "w1"].T), store)
    decay = torch.exp(-torch.exp(low @ w[p + "w2"].T + w[p + "w0"])).view(T, H, d)
    o = wkv_recurrence(r, k, v, decay, w[p + "u"].view(H, d))
    o = rms(o, eps).reshape(T, H * d) * w[p + "norm"] * gate
    return stored(o, store) @ w[p + "o"].T


# ------------------------------------------------------------------------------- feed-forward
def dense_ff(h: torch.Tensor, w: dict, p: str, store: torch.dtype | None = None) -> torch.Tensor:
    g = h @ w[p + "gate"].T
    a = stored(g * torch.sigmoid(g) * (h @ w[p + "up"].T), store)
    return a @ w[p + "down"].T


MIXERS = {"attention": attention, "latent_attention": latent_attention, "wkv": wkv}


# -------------------------------------------------------------------------------------- model
def forward(config: dict, weights: dict, tokens, dtype: torch.dtype = torch.float32,
            store: torch.dtype | None = None, layers_out: list | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence.  ``layers_out``, if given, receives the
    stream after every layer."""
    w = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in weights.items()}
    eps = float(config["norm"]["eps"])
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = w["embed"][ids] * float((config.get("embedding") or {}).get("scale", 1.0))
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = stored(norm(x, w[p + "norm1"], eps), store)
        y = MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps, store)
        x = x + norm(stored(y, store), w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = stored(norm(x, w[p + "norm2"], eps), store)
            y = dense_ff(h, w, p + "mlp.", store)
            x = x + norm(stored(y, store), w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    h = stored(norm(x, w["final.norm"], eps), store)
    logits = (h @ w["embed"].T) * float(config.get("logit_scale", 1.0))
    return capped(logits, config.get("logit_softcap")).to(torch.float32)


def greedy(config: dict, weights: dict, prompt, n: int) -> list[int]:
    """``n`` tokens by always taking the best one (the lowest index among equals)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, weights, toks)[-1].argmax()))
    return toks[len(prompt):]
