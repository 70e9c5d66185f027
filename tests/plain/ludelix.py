"""A plain, slow Ludelix decoder: whole sequences, no cache, no carried state, one function per
mechanism, torch on the CPU in 32-bit (or 64-bit, for a truth all but free of rounding).  It is
the oracle the engine's Ludelix model is held to and shares no code with ``kvforge_amd``: it
reads ``config.json`` dictionaries and ``{checkpoint name: tensor}`` dicts itself.

The design in this file's notation (``T`` tokens of one sequence, positions ``0..T-1``):

* stream ``x_t = embed[token_t]``;
* a layer: ``x += mixer(N1(x))``, then, where the layer has a feed-forward, ``x += ff(N2(x))``
  with ``N(x) = x / sqrt(mean(x^2) + eps) * w``;
* mixer ``gla``: per head a matrix memory ``S [dim, vdim]`` whose key rows decay by
  ``a_t = sigmoid(z_t)^(1/tau)``, ``z = A2 (A1 h) + b``: ``S_t = diag(a_t) S_(t-1) + k_t v_t^T``,
  ``o_t = S_t^T q_t`` with ``q`` scaled by ``dim^(-1/2)``; head norm with a weight, silu gate;
* mixer ``attention``: grouped queries; q and k carry biases and are normalised over the whole
  projected row (all heads at once); the values are the keys as they leave the projection;
  neighbouring pairs rotated with frequencies stretched by wavelength; sliding window; a sink
  in the softmax's denominator;
* mixer ``parallel``: ``left_scale * left(h) + right_scale * right(h)``: on the left grouped-query
  attention rotated half against half with YaRN-stretched frequencies, seeing only the keys of
  its own chunk of positions, with one sigmoid gate per head; on the right a retention, a matrix
  memory with one constant decay per head, rotated q and k, a head norm without weight and a
  silu gate;
* feed-forward ``dense``: ``W_down relu(W_up h)^2``; ``moe``: the experts a table names for the
  token's id, each with weight ``1/top``, plus a shared expert times ``sigmoid(w_sg . h)``;
* logits ``= embed @ N(x)``.
"""

from __future__ import annotations

import math

import torch


def stored(x: torch.Tensor, store: torch.dtype | None) -> torch.Tensor:
    """``x`` after a trip through memory in type ``store`` (rounded and widened again), or
    unchanged for ``None``."""
    return x if store is None else x.to(store).to(x.dtype)


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x`` divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * w


# ---------------------------------------------------------------------------------- rotations
def plain_frequencies(dims: int, base: float) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=torch.float64)
    return base ** (-2.0 * i / dims)


def wavelength_frequencies(dims: int, base: float, scaling: dict | None) -> torch.Tensor:
    """Frequencies stretched by wavelength: short waves stay, long ones are slowed by ``factor``,
    the ones between are blended."""
    f = plain_frequencies(dims, base)
    if not scaling:
        return f
    factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
    orig = float(scaling["original"])
    out = f.clone()
    for i in range(f.numel()):
        wave = 2.0 * math.pi / float(f[i])
        if wave < orig / high:
            continue
        if wave > orig / low:
            out[i] = f[i] / factor
        else:
            s = (orig / wave - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out


def yarn_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(frequency of every rotary pair in float64, factor on cos and sin)."""
    f = plain_frequencies(dims, base)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn(x: torch.Tensor, positions: torch.Tensor, f: torch.Tensor, mag: float, neighbours: bool) -> torch.Tensor:
    """``x [T, heads, dim]``: the first ``2 len(f)`` elements of every head are turned by the angle
    ``position * f_i``; pair ``i`` is elements ``(2i, 2i+1)`` (``neighbours``) or ``(i, i + len(f))``.
    Angles are formed in 32-bit."""
    n = f.numel()
    a = positions.to(torch.float32)[:, None] * f.to(torch.float32)[None, :]
    cos, sin = (a.cos() * mag).to(x.dtype)[:, None, :], (a.sin() * mag).to(x.dtype)[:, None, :]
    out = x.clone()
    if neighbours:
        u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = u * cos - v * sin
        out[..., 1:2 * n:2] = v * cos + u * sin
    else:
        u, v = x[..., :n], x[..., n:2 * n]
        out[..., :n] = u * cos - v * sin
        out[..., n:2 * n] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------------- attention
def window_mask(T: int, size: int) -> torch.Tensor:
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i - j < size)


def chunk_mask(T: int, size: int) -> torch.Tensor:
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask: torch.Tensor,
                      sink: torch.Tensor | None) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]``; head ``h`` reads key/value head
    ``h // (H / G)``.  ``sink [H]``: one more term ``exp(sink_h)`` in the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = q.new_zeros(T, H, v.shape[2])
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].expand_as(m))
        e = (s - m).exp()
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + (sink[h] - m).exp()
        out[:, h] = (e / den) @ v[:, g]
    return out


def sink_attention_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float,
                         store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    pos = torch.arange(T)
    q = stored(h @ w[p + "q"].T + w[p + "q.b"], store)
    k = stored(h @ w[p + "k"].T + w[p + "k.b"], store)
    v = k.view(T, G, d)
    qn = norm(q, w[p + "q.norm"], eps).view(T, H, d)
    kn = norm(k, w[p + "k.norm"], eps).view(T, G, d)
    rot = m.get("rot")
    if rot:
        f = wavelength_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        qn, kn = turn(qn, pos, f, 1.0, True), turn(kn, pos, f, 1.0, True)
    qn, kn = stored(qn, store), stored(kn, store)
    o = softmax_attention(qn, kn, v, float(m["scale"]), window_mask(T, int(m["mask"]["size"])),
                          w[p + "sink"].to(h.dtype))
    return stored(o, store).reshape(T, H * d) @ w[p + "o"].T


def chunk_attention_mixer(h: torch.Tensor, w: dict, p: str, m: dict, store: torch.dtype | None = None,
                          out_scale: float = 1.0) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = stored(h @ w[p + "q"].T, store).view(T, H, d)
    k = stored(h @ w[p + "k"].T, store).view(T, G, d)
    v = stored(h @ w[p + "v"].T, store).view(T, G, dv)
    gate = torch.sigmoid(stored(h @ w[p + "g"].T, store))            # [T, H]
    rot = m.get("rot")
    if rot:
        f, mag = yarn_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = stored(turn(q, pos, f, mag, False), store), stored(turn(k, pos, f, mag, False), store)
    o = softmax_attention(q, k, v, float(m["scale"]), chunk_mask(T, int(m["mask"]["size"])), None)
    o = o * gate[:, :, None] * out_scale
    return stored(o, store).reshape(T, H * dv) @ w[p + "o"].T


# ---------------------------------------------------------------------------------- memories
def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor) -> torch.Tensor:
    """``q, k [T, H, dk]``, ``v [T, H, dv]``, ``a [T, H, dk]`` (or ``[H, 1]`` for a constant per
    head): ``S_t = diag(a_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``, ``S_(-1) = 0``."""
    T, H, dk = q.shape
    S = q.new_zeros(H, dk, v.shape[2])
    out = q.new_zeros(T, H, v.shape[2])
    for t in range(T):
        at = a[t] if a.dim() == 3 else a
        S = at[:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def gla_decay(h: torch.Tensor, w: dict, p: str, tau: float, store: torch.dtype | None = None) -> torch.Tensor:
    low = stored(h @ w[p + "a1"].T, store)
    z = low @ w[p + "a2"].T + w[p + "a2.b"]
    return torch.exp(torch.nn.functional.logsigmoid(z) / tau)


def gla_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, dk, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = stored(h @ w[p + "q"].T, store).view(T, H, dk) * dk ** -0.5
    k = stored(h @ w[p + "k"].T, store).view(T, H, dk)
    v = stored(h @ w[p + "v"].T, store).view(T, H, dv)
    a = gla_decay(h, w, p, float(m["tau"]), store).view(T, H, dk)
    o = rms(decay_scan(q, k, v, a), eps) * w[p + "norm"]
    g = stored(h @ w[p + "g"].T, store)
    y = o.reshape(T, H * dv) * torch.nn.functional.silu(g)
    return stored(y, store) @ w[p + "o"].T


def retention_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, store: torch.dtype | None = None,
                    out_scale: float = 1.0) -> torch.Tensor:
    T = h.shape[0]
    H, dk, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = stored(h @ w[p + "q"].T, store).view(T, H, dk)
    k = stored(h @ w[p + "k"].T, store).view(T, H, dk)
    v = stored(h @ w[p + "v"].T, store).view(T, H, dv)
    rot = m.get("rot")
    if rot:
        f = plain_frequencies(int(rot["dims"]), float(rot["base"]))
        q, k = turn(q, pos, f, 1.0, False), turn(k, pos, f, 1.0, False)
    k = k * dk ** -0.5
    a = torch.tensor([float(x) for x in m["decay"]], dtype=h.dtype)[:, None]
    o = rms(decay_scan(q, k, v, a), eps)
    g = stored(h @ w[p + "g"].T, store)
    y = o.reshape(T, H * dv) * torch.nn.functional.silu(g) * out_scale
    return stored(y, store) @ w[p + "o"].T


def parallel_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, store: torch.dtype | None = None) -> torch.Tensor:
    left = chunk_attention_mixer(h, w, p + "left.", m["left"], store, float(m["left_scale"]))
    right = retention_mixer(h, w, p + "right.", m["right"], eps, store, float(m["right_scale"]))
    return left + right


# ---------------------------------------------------------------------------------- feed-forward
def dense_ff(h: torch.Tensor, w: dict, p: str, store: torch.dtype | None = None) -> torch.Tensor:
    a = torch.relu(stored(h @ w[p + "up"].T, store)) ** 2
    return stored(a, store) @ w[p + "down"].T


def expert(h: torch.Tensor, w: dict, p: str, store: torch.dtype | None = None, scale=None) -> torch.Tensor:
    g, u = stored(h @ w[p + "gate"].T, store), stored(h @ w[p + "up"].T, store)
    a = torch.nn.functional.silu(g) * u
    if scale is not None:
        a = a * scale
    return stored(a, store) @ w[p + "down"].T


def table_ff(h: torch.Tensor, tokens: torch.Tensor, w: dict, p: str, mlp: dict,
             store: torch.dtype | None = None) -> torch.Tensor:
    top = int(mlp["router"]["top"])
    table = w[p + "table"].long()
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in table[int(tokens[t])].tolist():
            out[t] += stored(expert(h[t:t + 1], w, f"{p}e{e}.", store)[0], store) / top
    if mlp.get("shared"):
        sg = torch.sigmoid(h @ w[p + "shared.sg"].T)                 # [T, 1]
        out = out + expert(h, w, p + "shared.", store, scale=sg)
    return out


# ---------------------------------------------------------------------------------- the model
def forward(config: dict, weights: dict, tokens, dtype: torch.dtype = torch.float32,
            store: torch.dtype | None = None, layers_out: list | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence.  ``dtype``: the arithmetic (float32 or
    float64); ``store``: what an engine may keep in 16 bits between operations is rounded to
    this.  ``layers_out``: a list that receives the stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tokens]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = stored(norm(x, w[p + "norm1"], eps), store)
        kind, m = layer["type"], layer["mixer"]
        if kind == "gla":
            x = x + gla_mixer(h, w, p + "mix.", m, eps, store)
        elif kind == "attention":
            x = x + sink_attention_mixer(h, w, p + "mix.", m, eps, store)
        elif kind == "parallel":
            x = x + parallel_mixer(h, w, p + "mix.", m, eps, store)
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        mlp = layer.get("mlp")
        if mlp:
            h = stored(norm(x, w[p + "norm2"], eps), store)
            if mlp["kind"] == "dense":
                x = x + dense_ff(h, w, p + "mlp.", store)
            elif mlp["kind"] == "moe":
                x = x + table_ff(h, tokens, w, p + "mlp.", mlp, store)
            else:
                raise ValueError(f"unknown feed-forward {mlp['kind']!r}")
        if layers_out is not None:
            layers_out.append(x.clone())
    h = stored(norm(x, w["final.norm"], eps), store)
    return h @ w["embed"].T


def greedy(config: dict, weights: dict, prompt, n: int, dtype: torch.dtype = torch.float32) -> list[int]:
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, weights, toks, dtype)[-1].argmax()))
    return toks[len(prompt):]
