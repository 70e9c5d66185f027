"""Python faces of the HIP kernels.  Each function checks on the host that shapes, dtypes,
devices and strides are what its kernel and launch grid assume, then launches on torch's
current stream (so launches made while a torch HIP-graph capture is active are captured).

There is no fallback: every function here runs a hand-written gfx950 kernel, or (``gemm`` for
bf16 with many rows, as the reference's engine does for its products) the library's matrix
product through ``csrc/gemm_library.hip``, or raises.  No torch operator computes anything
here.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import torch

from kvforge_amd.kernels import library

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32


class KernelError(RuntimeError):
    pass


def _tcode(dtype: torch.dtype) -> int:
    if dtype == F32:
        return 0
    if dtype == BF16:
        return 1
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}")


def _suffix(dtype: torch.dtype) -> str:
    return "f32" if _tcode(dtype) == 0 else "bf16"


# the raw handle of torch's current stream, without a Stream object built for every launch
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(t: torch.Tensor, name: str, dtype=None, shape=None, contiguous=True) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None:
        have = t.shape
        bad = len(have) != len(shape)
        if not bad:
            for want, got in zip(shape, have):   # a plain loop: this runs for every operand of every launch
                if want is not None and want != got:
                    bad = True
                    break
        if bad:
            raise KernelError(f"{name} must have shape {list(shape)}, got {list(have)}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


def _overlap(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Whether the memory spanned by two tensors' storage views intersects."""
    def span(t):
        if t.numel() == 0:
            return t.data_ptr(), t.data_ptr()
        last = sum((n - 1) * st for n, st in zip(t.shape, t.stride()))
        return t.data_ptr(), t.data_ptr() + (last + 1) * t.element_size()
    (a0, a1), (b0, b1) = span(a), span(b)
    return a0 < b1 and b0 < a1


def _ok(code: int, what: str) -> None:
    if code != 0:
        raise KernelError(f"{what} failed with HIP error {code}")


_fn_cache: dict[tuple[str, str], object] = {}


def _fn(module: str, name: str, argtypes: list):
    key = (module, name)
    f = _fn_cache.get(key)
    if f is None:
        lib = library.load(module)
        try:
            f = getattr(lib, name)
        except AttributeError:
            raise KernelError(f"kernel module {module!r} has no entry point {name!r}") from None
        f.argtypes = argtypes
        f.restype = c_int
        _fn_cache[key] = f
    return f


# ------------------------------------------------------------------------------ embedding
def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """``out[n] = table[ids[n]] * scale``, widened to fp32 first (the residual stream)."""
    n = ids.shape[0]
    _check(ids, "ids", I32, (n,))
    _check(table, "table", None, (None, None))
    vocab, h = table.shape
    _check(out, "out", F32, (n, h))
    f = _fn("elementwise", f"kvf_embed_{_suffix(table.dtype)}",
            [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p])
    _ok(f(ids.data_ptr(), table.data_ptr(), out.data_ptr(), n, h, vocab, float(scale), _stream()), "embed")


def softcap(x: torch.Tensor, cap: float | None, scale: float = 1.0) -> None:
    """``x = cap * tanh(x * scale / cap)`` in place over fp32 values (logits); without a cap
    (``None``) ``x = x * scale``."""
    _check(x, "x", F32)
    if cap is not None and not cap > 0.0:
        raise KernelError(f"softcap: the cap must be positive, got {cap}")
    f = _fn("elementwise", "kvf_softcap", [c_void_p, c_long, c_float, c_float, c_void_p])
    _ok(f(x.data_ptr(), x.numel(), float(cap or 0.0), float(scale), _stream()), "softcap")


# ------------------------------------------------------------------------------ RMS norm
def rmsnorm(x: torch.Tensor, weight: torch.Tensor | None, eps: float, out: torch.Tensor,
            rows: torch.Tensor | None = None, add: torch.Tensor | None = None) -> None:
    """``out[m] = y * rsqrt(mean(y^2) + eps) * weight`` with ``y = x[rows[m] or m]`` in fp32
    (``weight=None``: no weight, for a norm whose weight is folded into the next matrix).
    ``add`` (``[rows of x, h]``, dtype of ``out`` or fp32) is a sum still owed to ``x``: the norm
    is taken of ``x + add``, and without ``rows`` the sum is written back to ``x`` as well."""
    _check(x, "x", F32, (None, None))
    xr, h = x.shape
    m = out.shape[0]
    _check(out, "out", None, (m, h))
    if weight is not None:
        _check(weight, "weight", None, (h,))
        if weight.dtype not in (F32, out.dtype):
            raise KernelError(f"norm weight must be float32 or {out.dtype}, got {weight.dtype}")
    if rows is not None:
        _check(rows, "rows", I32, (m,))
    elif m > xr:
        raise KernelError("rmsnorm: more output rows than input rows")
    if add is not None:
        _check(add, "add", None, (xr, h))
        if add.dtype not in (F32, out.dtype):
            raise KernelError(f"rmsnorm: add must be float32 or {out.dtype}, got {add.dtype}")
    f = _fn("elementwise", f"kvf_rmsnorm_{_suffix(out.dtype)}",
            [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_int, c_int,
             c_int, c_void_p])
    _ok(f(x.data_ptr(), rows.data_ptr() if rows is not None else None,
          add.data_ptr() if add is not None else None,
          1 if add is not None and add.dtype == F32 else 0,
          weight.data_ptr() if weight is not None else None,
          1 if weight is not None and weight.dtype == F32 else 0, float(eps), out.data_ptr(),
          m, h, xr, _stream()), "rmsnorm")


def rmsnorm_pair(x: torch.Tensor, weight1: torch.Tensor, weight2: torch.Tensor, eps: float,
                 out1: torch.Tensor, out2: torch.Tensor, add: torch.Tensor | None = None) -> None:
    """Two RMS norms of the same rows in one pass: ``out1 = y * weight1`` and ``out2 = y * weight2``
    with ``y = v * rsqrt(mean(v^2) + eps)`` and ``v = x`` (``+ add``, a sum still owed to ``x``, which
    is then left in ``x``).  Weights fp32 ``[h]``; outputs of one type."""
    _check(x, "x", F32, (None, None))
    m, h = x.shape
    _check(weight1, "weight1", F32, (h,))
    _check(weight2, "weight2", F32, (h,))
    _check(out1, "out1", None, (m, h))
    _check(out2, "out2", out1.dtype, (m, h))
    if add is not None:
        _check(add, "add", None, (m, h))
        if add.dtype not in (F32, out1.dtype):
            raise KernelError(f"rmsnorm_pair: add must be float32 or {out1.dtype}, got {add.dtype}")
    f = _fn("elementwise", f"kvf_rmsnorm_pair_{_suffix(out1.dtype)}",
            [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), add.data_ptr() if add is not None else None,
          1 if add is not None and add.dtype == F32 else 0, weight1.data_ptr(), weight2.data_ptr(), float(eps),
          out1.data_ptr(), out2.data_ptr(), m, h, _stream()), "rmsnorm_pair")


def add_rows(x: torch.Tensor, delta: torch.Tensor) -> None:
    """``x += delta`` for the fp32 residual stream ``x`` and a product ``delta`` of equal shape."""
    _check(x, "x", F32, (None, None))
    _check(delta, "delta", None, tuple(x.shape))
    f = _fn("elementwise", f"kvf_add_rows_{_suffix(delta.dtype)}", [c_void_p, c_void_p, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), delta.data_ptr(), x.shape[0], x.shape[1], _stream()), "add_rows")


# ------------------------------------------------------------------------------ learned positions,
# norm + token shift, gated activations, output gate, per-token side input
def add_positions(x: torch.Tensor, table: torch.Tensor, positions: torch.Tensor) -> None:
    """``x[n] += table[positions[n]]`` for the fp32 stream ``x``: a learned vector per position."""
    _check(x, "x", F32, (None, None))
    n, h = x.shape
    _check(table, "table", None, (None, h))
    _check(positions, "positions", I32, (None,))
    if positions.shape[0] < n:
        raise KernelError("add_positions: positions shorter than the batch")
    f = _fn("elementwise", f"kvf_add_positions_{_suffix(table.dtype)}",
            [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), table.data_ptr(), positions.data_ptr(), n, h, table.shape[0], _stream()),
        "add_positions")


def norm_shift(x: torch.Tensor, weight: torch.Tensor, mu: torch.Tensor, state: torch.Tensor,
               slot_ids: torch.Tensor, seq_of_token: torch.Tensor, cu_q: torch.Tensor,
               positions: torch.Tensor, eps: float, plain: torch.Tensor, shifted: torch.Tensor) -> None:
    """RMS norm and token shift of the fp32 stream in one kernel.  With ``y = norm(x) * weight``:
    ``plain = y`` and ``shifted[t] = y[t] + (y[t-1] - y[t]) * mu``, where the token before the
    first one of a query run is read from the sequence's row of ``state`` (zeros at position 0)
    and the run's last ``y`` is left there.  ``weight``, ``mu``: fp32 ``[h]``; ``state``: fp32
    ``[slots, h]``; ``slot_ids``: a slot per sequence, negative for none."""
    _check(x, "x", F32, (None, None))
    n, h = x.shape
    _check(weight, "weight", F32, (h,))
    _check(mu, "mu", F32, (h,))
    _check(state, "state", F32, (None, h))
    for t, name in ((slot_ids, "slot_ids"), (seq_of_token, "seq_of_token"), (cu_q, "cu_q"),
                    (positions, "positions")):
        _check(t, name, I32, (None,))
    n_seqs = slot_ids.shape[0]
    if cu_q.shape[0] < n_seqs + 1 or seq_of_token.shape[0] < n or positions.shape[0] < n:
        raise KernelError("norm_shift: batch fields shorter than the batch")
    _check(plain, "plain", None, (n, h))
    _check(shifted, "shifted", plain.dtype, (n, h))
    f = _fn("elementwise", f"kvf_norm_shift_{_suffix(plain.dtype)}",
            [c_void_p] * 10 + [c_float] + [c_int] * 4 + [c_void_p])
    _ok(f(x.data_ptr(), weight.data_ptr(), mu.data_ptr(), state.data_ptr(), slot_ids.data_ptr(),
          seq_of_token.data_ptr(), cu_q.data_ptr(), positions.data_ptr(), plain.data_ptr(),
          shifted.data_ptr(), float(eps), n, h, n_seqs, state.shape[0], _stream()), "norm_shift")


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def gated_act(gate_up: torch.Tensor, out: torch.Tensor, activation: str, paired: bool = False,
              gate_bias: torch.Tensor | None = None, up_bias: torch.Tensor | None = None) -> None:
    """``out[:, i] = act(gate_i + gate_bias[i]) * (up_i + up_bias[i])``; the input row holds gate
    at ``i`` and up at ``I + i``, or with ``paired`` at ``2i`` and ``2i + 1``.  ``activation``:
    ``"silu"`` or ``"gelu_tanh"``; the biases are fp32 ``[I]`` or ``None``."""
    m, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("gated_act: input width must be even")
    if activation not in ACTIVATIONS:
        raise KernelError(f"gated_act: unknown activation {activation!r}; known: {sorted(ACTIVATIONS)}")
    _check(gate_up, "gate_up", None, (m, two_i))
    _check(out, "out", gate_up.dtype, (m, two_i // 2))
    for b, name in ((gate_bias, "gate_bias"), (up_bias, "up_bias")):
        if b is not None:
            _check(b, name, F32, (two_i // 2,))
    f = _fn("elementwise", f"kvf_gated_act_{_suffix(out.dtype)}",
            [c_void_p] * 4 + [c_int] * 4 + [c_void_p])
    _ok(f(gate_up.data_ptr(), gate_bias.data_ptr() if gate_bias is not None else None,
          up_bias.data_ptr() if up_bias is not None else None, out.data_ptr(), m, two_i // 2,
          1 if paired else 0, ACTIVATIONS[activation], _stream()), "gated_act")


def sigmoid_gate(y: torch.Tensor, gate: torch.Tensor) -> None:
    """``y *= sigmoid(gate)`` element by element; both ``[M, C]`` with dense rows (row strides may
    exceed C, so ``gate`` can be a block of columns of a wider product)."""
    m, c = y.shape
    _check(y, "y", None, (m, c), contiguous=False)
    _check(gate, "gate", y.dtype, (m, c), contiguous=False)
    if y.stride(1) != 1 or gate.stride(1) != 1:
        raise KernelError("sigmoid_gate: rows must be dense")
    f = _fn("elementwise", f"kvf_sigmoid_gate_{_suffix(y.dtype)}", [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p])
    _ok(f(y.data_ptr(), gate.data_ptr(), m, c, y.stride(0) if m > 1 else c,
          gate.stride(0) if m > 1 else c, _stream()), "sigmoid_gate")


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> None:
    """``x[m] += bias`` for every row of the fp32 stream."""
    _check(x, "x", F32, (None, None))
    _check(bias, "bias", F32, (x.shape[1],))
    f = _fn("elementwise", "kvf_add_bias", [c_void_p, c_void_p, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), bias.data_ptr(), x.shape[0], x.shape[1], _stream()), "add_bias")


TOKEN_SIDE_MAX_FLOATS = 16 * 1024   # the row and the gated vector live in 64 KB of LDS


def token_side(x: torch.Tensor, tokens: torch.Tensor, side: torch.Tensor, col0: int,
               gate: torch.Tensor, proj: torch.Tensor, weight: torch.Tensor, eps: float,
               bias: torch.Tensor | None = None, owed: torch.Tensor | None = None,
               proj_t: torch.Tensor | None = None) -> None:
    """A per-token input into the fp32 stream: with ``e = side[token, col0 : col0 + dim]``,
    ``y = proj @ (gelu_tanh(gate @ x[m]) * e)`` and ``x[m] += y * rsqrt(mean(y^2) + eps) * weight``.
    ``bias`` (fp32 ``[h]``) and ``owed`` (``[M, h]``, a product still owed to the stream) are added
    to ``x[m]`` first and stay in it.  ``gate [dim, h]``, ``proj [h, dim]`` and ``side`` share a
    type; ``weight`` is fp32.  ``proj_t``: ``proj`` transposed, ``[dim, h]`` contiguous; with it,
    rows of a multiple of 8 elements take a kernel of 1,024 threads with 16-byte loads."""
    _check(x, "x", F32, (None, None))
    n, h = x.shape
    _check(tokens, "tokens", I32, (None,))
    if tokens.shape[0] < n:
        raise KernelError("token_side: token ids shorter than the batch")
    _check(gate, "gate", None, (None, h))
    dim = gate.shape[0]
    _check(proj, "proj", gate.dtype, (h, dim))
    _check(side, "side", gate.dtype, (None, None))
    if not 0 <= col0 <= side.shape[1] - dim:
        raise KernelError(f"token_side: columns {col0}..{col0 + dim} outside the table's {side.shape[1]}")
    _check(weight, "weight", F32, (h,))
    if h + dim > TOKEN_SIDE_MAX_FLOATS:
        raise KernelError(f"token_side: a row of {h} + {dim} floats does not fit the kernel's LDS")
    if bias is not None:
        _check(bias, "bias", F32, (h,))
    if owed is not None:
        _check(owed, "owed", None, (n, h))
        if owed.dtype not in (F32, gate.dtype):
            raise KernelError(f"token_side: owed must be float32 or {gate.dtype}, got {owed.dtype}")
    if proj_t is not None:
        _check(proj_t, "proj_t", gate.dtype, (dim, h))
    f = _fn("elementwise", f"kvf_token_side_{_suffix(gate.dtype)}",
            [c_void_p, c_void_p, c_void_p, c_int] + [c_void_p] * 5 + [c_float] + [c_int] * 6 + [c_void_p, c_void_p])
    _ok(f(x.data_ptr(), bias.data_ptr() if bias is not None else None,
          owed.data_ptr() if owed is not None else None,
          1 if owed is not None and owed.dtype == F32 else 0, tokens.data_ptr(), side.data_ptr(),
          gate.data_ptr(), proj.data_ptr(), weight.data_ptr(), float(eps), n, h, dim, side.shape[0],
          side.shape[1], int(col0), proj_t.data_ptr() if proj_t is not None else None, _stream()),
        "token_side")


def settle_cast(x: torch.Tensor, bias: torch.Tensor | None = None, owed: torch.Tensor | None = None,
                copy: torch.Tensor | None = None) -> None:
    """``x[m] += bias + owed[m]`` for the fp32 stream (either may be ``None``), and, with
    ``copy`` (``[M, h]`` in fp32 or bf16), a copy of the rows as they then are."""
    _check(x, "x", F32, (None, None))
    m, h = x.shape
    if bias is not None:
        _check(bias, "bias", F32, (h,))
    kind = copy.dtype if copy is not None else (owed.dtype if owed is not None and owed.dtype == BF16 else F32)
    if owed is not None:
        _check(owed, "owed", None, (m, h))
        if owed.dtype not in (F32, kind):
            raise KernelError(f"settle_cast: owed must be float32 or {kind}, got {owed.dtype}")
    if copy is not None:
        _check(copy, "copy", None, (m, h))
    f = _fn("elementwise", f"kvf_settle_cast_{_suffix(kind)}",
            [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), bias.data_ptr() if bias is not None else None,
          owed.data_ptr() if owed is not None else None,
          1 if owed is not None and owed.dtype == F32 else 0,
          copy.data_ptr() if copy is not None else None, m, h, _stream()), "settle_cast")


def side_gate(a: torch.Tensor, tokens: torch.Tensor, side: torch.Tensor, col0: int, out: torch.Tensor) -> None:
    """``out[m, j] = gelu_tanh(a[m, j]) * side[tokens[m], col0 + j]`` (zeros for a token outside
    the table)."""
    m, dim = a.shape
    _check(a, "a", None, (m, dim))
    _check(out, "out", a.dtype, (m, dim))
    _check(side, "side", a.dtype, (None, None))
    _check(tokens, "tokens", I32, (None,))
    if tokens.shape[0] < m or not 0 <= col0 <= side.shape[1] - dim:
        raise KernelError("side_gate: token ids shorter than the batch, or columns outside the table")
    f = _fn("elementwise", f"kvf_side_gate_{_suffix(a.dtype)}", [c_void_p] * 4 + [c_int] * 5 + [c_void_p])
    _ok(f(a.data_ptr(), tokens.data_ptr(), side.data_ptr(), out.data_ptr(), m, dim, side.shape[0],
          side.shape[1], int(col0), _stream()), "side_gate")


def rms_add(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """``x[m] += y[m] * rsqrt(mean(y[m]^2) + eps) * weight``, all fp32."""
    _check(x, "x", F32, (None, None))
    _check(y, "y", F32, tuple(x.shape))
    _check(weight, "weight", F32, (x.shape[1],))
    f = _fn("elementwise", "kvf_rms_add", [c_void_p, c_void_p, c_void_p, c_float, c_int, c_int, c_void_p])
    _ok(f(x.data_ptr(), y.data_ptr(), weight.data_ptr(), float(eps), x.shape[0], x.shape[1], _stream()),
        "rms_add")


def rms_add_norm(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, weight2: torch.Tensor,
                 eps2: float, out: torch.Tensor) -> None:
    """``rms_add`` and the norm of the sum in one pass: ``x[m] += y[m] * rsqrt(mean(y[m]^2) + eps) *
    weight``, then ``out[m] = x[m] * rsqrt(mean(x[m]^2) + eps2) * weight2``; both weights fp32."""
    _check(x, "x", F32, (None, None))
    _check(y, "y", F32, tuple(x.shape))
    _check(weight, "weight", F32, (x.shape[1],))
    _check(weight2, "weight2", F32, (x.shape[1],))
    _check(out, "out", None, tuple(x.shape))
    f = _fn("elementwise", "kvf_rms_add_norm", [c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_float,
                                                c_void_p, c_int, c_int, c_void_p])
    _ok(f(_tcode(out.dtype), x.data_ptr(), y.data_ptr(), weight.data_ptr(), float(eps), weight2.data_ptr(),
          float(eps2), out.data_ptr(), x.shape[0], x.shape[1], _stream()), "rms_add_norm")


# ------------------------------------------------------------------------------ SwiGLU gate
def silu_mul(gate_up: torch.Tensor, out: torch.Tensor, paired: bool = False) -> None:
    """``out[:, i] = silu(gate_i) * up_i`` where the input row holds gate at ``i`` and up at
    ``I + i``, or, with ``paired``, gate at ``2i`` and up at ``2i + 1``."""
    m, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("silu_mul: input width must be even")
    _check(gate_up, "gate_up", None, (m, two_i))
    _check(out, "out", gate_up.dtype, (m, two_i // 2))
    f = _fn("elementwise", f"kvf_silu_mul_{_suffix(out.dtype)}",
            [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p])
    _ok(f(gate_up.data_ptr(), out.data_ptr(), m, two_i // 2, 1 if paired else 0, _stream()),
        "silu_mul")


# ------------------------------------------------------------------------------ rotary + cache
NO_TABLE_LEN = 2**31 - 1


def _rotary_tables(cos, sin, d: int, who: str):
    """(cos pointer, sin pointer, rotary width, positions the tables cover).  Without tables
    (both ``None``) nothing is rotated, the width is 0 and every position is covered."""
    if cos is None and sin is None:
        return None, None, 0, NO_TABLE_LEN
    _check(cos, "cos", F32, (None, None))
    _check(sin, "sin", F32, tuple(cos.shape))
    table_len, half = cos.shape
    if 2 * half > d or half <= 0:
        raise KernelError(f"{who}: rotary width {2 * half} does not fit head_dim {d}")
    return cos.data_ptr(), sin.data_ptr(), 2 * half, table_len


def rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                 cos: torch.Tensor | None, sin: torch.Tensor | None, block_table: torch.Tensor,
                 k_pages: torch.Tensor, v_pages: torch.Tensor, num_heads: int, num_kv_heads: int,
                 head_dim: int, write_kv: bool = True) -> None:
    """Rotate q (in place) and k by the cos/sin rows of each token's position; write rotated k
    and v into the pages named by the token's sequence row of ``block_table``.  Rotary pairs
    are neighbouring elements ``(2i, 2i + 1)`` of a head; without tables (``None``) q and k stay
    as they are and only the cache is written.  ``k_pages``:
    ``[num_blocks, KV, block_size, d]``; ``v_pages`` transposed: ``[num_blocks, KV, d, block_size]``.
    A row of ``qkv`` may hold further columns behind q, k and v (what else the same product made);
    they are left alone."""
    n = qkv.shape[0]
    H, KV, d = num_heads, num_kv_heads, head_dim
    _check(qkv, "qkv", None, (n, None))
    if qkv.shape[1] < (H + (2 * KV if write_kv else 0)) * d:
        raise KernelError(f"rope_kvwrite: rows of {qkv.shape[1]} elements do not hold q, k and v")
    _check(positions, "positions", I32, (None,))
    _check(seq_of_token, "seq_of_token", I32, (None,))
    if positions.shape[0] < n or seq_of_token.shape[0] < n:
        raise KernelError("rope_kvwrite: positions / seq_of_token shorter than the batch")
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, d, "rope_kvwrite")
    _check(block_table, "block_table", I32, (None, None))
    n_seqs, stride = block_table.shape
    _check(k_pages, "k_pages", qkv.dtype, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", qkv.dtype, (nb, KV, d, bs))
    f = _fn("elementwise", f"kvf_rope_kvwrite_{_suffix(qkv.dtype)}",
            [c_void_p] * 8 + [c_int] * 12 + [c_void_p])
    _ok(f(qkv.data_ptr(), positions.data_ptr(), seq_of_token.data_ptr(), cos_p,
          sin_p, block_table.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
          n, H, KV, d, rot, table_len, bs, stride, nb, 1 if write_kv else 0, n_seqs,
          qkv.shape[1], _stream()),
        "rope_kvwrite")


def qknorm_rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                        cos: torch.Tensor | None, sin: torch.Tensor | None, block_table: torch.Tensor,
                        k_pages: torch.Tensor, v_pages: torch.Tensor, num_heads: int,
                        num_kv_heads: int, head_dim: int, q_weight: torch.Tensor,
                        k_weight: torch.Tensor, norm_dim: int, eps: float, write_kv: bool = True,
                        q_temp: tuple[float, int] | None = None) -> None:
    """``rope_kvwrite`` with a norm per head in front of the rotation: every q and k head is
    divided by the root mean square of its first ``norm_dim`` elements (``eps`` inside the root)
    and multiplied by ``q_weight`` / ``k_weight`` (fp32 ``[norm_dim]``, shared by the heads), in
    fp32 from the projected row; elements ``norm_dim..head_dim-1`` (padding) stay zero.
    ``q_temp = (coef, every)``: the q heads of a token at position ``p`` are also multiplied by
    ``1 + coef * ln(floor((p + 1) / every) + 1)``."""
    n = qkv.shape[0]
    H, KV, d = num_heads, num_kv_heads, head_dim
    _check(qkv, "qkv", None, (n, None))
    if qkv.shape[1] < (H + 2 * KV) * d:
        raise KernelError(f"qknorm_rope_kvwrite: rows of {qkv.shape[1]} elements do not hold q, k and v")
    if not 0 < norm_dim <= d <= 256:
        raise KernelError(f"qknorm_rope_kvwrite: norm over {norm_dim} of {d} elements (at most 256)")
    _check(positions, "positions", I32, (None,))
    _check(seq_of_token, "seq_of_token", I32, (None,))
    if positions.shape[0] < n or seq_of_token.shape[0] < n:
        raise KernelError("qknorm_rope_kvwrite: positions / seq_of_token shorter than the batch")
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, d, "qknorm_rope_kvwrite")
    if rot > norm_dim:
        raise KernelError(f"qknorm_rope_kvwrite: rotary width {rot} beyond the head's {norm_dim} elements")
    _check(q_weight, "q_weight", F32, (norm_dim,))
    _check(k_weight, "k_weight", F32, (norm_dim,))
    _check(block_table, "block_table", I32, (None, None))
    n_seqs, stride = block_table.shape
    _check(k_pages, "k_pages", qkv.dtype, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", qkv.dtype, (nb, KV, d, bs))
    f = _fn("elementwise", f"kvf_qknorm_rope_kvwrite_{_suffix(qkv.dtype)}",
            [c_void_p] * 10 + [c_int, c_float, c_float, c_int] + [c_int] * 12 + [c_void_p])
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else (0.0, 0)
    if q_temp is not None and every < 1:
        raise KernelError(f"qknorm_rope_kvwrite: q_temp's step must be positive, got {every}")
    _ok(f(qkv.data_ptr(), positions.data_ptr(), seq_of_token.data_ptr(), cos_p, sin_p,
          block_table.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), q_weight.data_ptr(),
          k_weight.data_ptr(), int(norm_dim), float(eps), coef, every, n, H, KV, d, rot, table_len, bs, stride, nb,
          1 if write_kv else 0, n_seqs, qkv.shape[1], _stream()), "qknorm_rope_kvwrite")


def rownorm_rope_kvwrite(proj: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                         seq_of_token: torch.Tensor, cos: torch.Tensor | None, sin: torch.Tensor | None,
                         block_table: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                         num_heads: int, num_kv_heads: int, head_dim: int, q_weight: torch.Tensor,
                         k_weight: torch.Tensor, norm_dim: int, eps: float,
                         q_bias: torch.Tensor | None = None, k_bias: torch.Tensor | None = None,
                         values_are_keys: bool = False, write_kv: bool = True) -> None:
    """From projected rows in fp32 (``proj [n, >= (H + KV) d]``, or ``(H + 2 KV) d`` with values
    of their own): biases on q and k (fp32 over the heads' first ``norm_dim`` elements, or
    ``None``); q and k each divided by the root mean square over *all* their elements at once
    (every head, ``eps`` inside the root) and multiplied by ``q_weight [H * norm_dim]`` /
    ``k_weight [KV * norm_dim]``; the rotation of neighbouring pairs; q to ``q_out [n, H * d]``,
    k and the values to the pages.  ``values_are_keys``: a token's values are its keys as they
    stand after the bias, before norm and rotation."""
    n = proj.shape[0]
    H, KV, d = int(num_heads), int(num_kv_heads), int(head_dim)
    _check(proj, "proj", F32, (n, None))
    need = (H + (KV if values_are_keys else 2 * KV)) * d
    if proj.shape[1] < need:
        raise KernelError(f"rownorm_rope_kvwrite: rows of {proj.shape[1]} elements do not hold {need}")
    if not 0 < norm_dim <= d <= 256 or d % 2:
        raise KernelError(f"rownorm_rope_kvwrite: heads of {norm_dim} in {d} elements (even, at most 256)")
    _check(q_out, "q_out", None, (n, H * d), contiguous=False)
    if q_out.stride(1) != 1:
        raise KernelError("rownorm_rope_kvwrite: rows of q_out must be dense")
    _check(positions, "positions", I32, (None,))
    _check(seq_of_token, "seq_of_token", I32, (None,))
    if positions.shape[0] < n or seq_of_token.shape[0] < n:
        raise KernelError("rownorm_rope_kvwrite: positions / seq_of_token shorter than the batch")
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, d, "rownorm_rope_kvwrite")
    if rot > norm_dim:
        raise KernelError(f"rownorm_rope_kvwrite: rotary width {rot} beyond the head's {norm_dim} elements")
    _check(q_weight, "q_weight", F32, (H * norm_dim,))
    _check(k_weight, "k_weight", F32, (KV * norm_dim,))
    if q_bias is not None:
        _check(q_bias, "q_bias", F32, (H * norm_dim,))
    if k_bias is not None:
        _check(k_bias, "k_bias", F32, (KV * norm_dim,))
    _check(block_table, "block_table", I32, (None, None))
    n_seqs, stride = block_table.shape
    _check(k_pages, "k_pages", q_out.dtype, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", q_out.dtype, (nb, KV, d, bs))
    f = _fn("elementwise", "kvf_rownorm_rope_kvwrite",
            [c_int] + [c_void_p] * 11 + [c_int, c_void_p, c_void_p, c_int, c_float] + [c_int] * 13 + [c_void_p])
    _ok(f(_tcode(q_out.dtype), proj.data_ptr(), q_bias.data_ptr() if q_bias is not None else None,
          k_bias.data_ptr() if k_bias is not None else None, q_weight.data_ptr(), k_weight.data_ptr(),
          positions.data_ptr(), seq_of_token.data_ptr(), cos_p, sin_p, block_table.data_ptr(), q_out.data_ptr(),
          q_out.stride(0) if n > 1 else H * d, k_pages.data_ptr(), v_pages.data_ptr(), int(norm_dim), float(eps),
          1 if values_are_keys else 0, n, H, KV, d, rot, table_len, bs, stride, nb, 1 if write_kv else 0, n_seqs,
          proj.shape[1], _stream()), "rownorm_rope_kvwrite")


def head_gate(y: torch.Tensor, gate: torch.Tensor | None, heads: int, head_dim: int, scale: float = 1.0) -> None:
    """``y[m, h * d + e] *= sigmoid(gate[m, h]) * scale``: one gate number per head.  ``y [M, H * d]``
    with dense rows; ``gate`` fp32 ``[M, >= H]`` with dense rows (a block of columns of a wider
    product is fine), or ``None`` for the scale alone."""
    m = y.shape[0]
    H, d = int(heads), int(head_dim)
    _check(y, "y", None, (m, H * d), contiguous=False)
    if y.stride(1) != 1:
        raise KernelError("head_gate: rows of y must be dense")
    if gate is None:
        f = _fn("elementwise", "kvf_head_gate", [c_int, c_void_p, c_void_p] + [c_int] * 5 + [c_float, c_void_p])
        _ok(f(_tcode(y.dtype), y.data_ptr(), None, m, H, d, y.stride(0) if m > 1 else H * d, 0, float(scale),
              _stream()), "head_gate")
        return
    _check(gate, "gate", F32, (m, None), contiguous=False)
    if gate.shape[1] < H or gate.stride(1) != 1:
        raise KernelError("head_gate: a gate per head in dense rows")
    f = _fn("elementwise", "kvf_head_gate", [c_int, c_void_p, c_void_p] + [c_int] * 5 + [c_float, c_void_p])
    _ok(f(_tcode(y.dtype), y.data_ptr(), gate.data_ptr(), m, H, d, y.stride(0) if m > 1 else H * d,
          gate.stride(0) if m > 1 else gate.shape[1], float(scale), _stream()), "head_gate")


PLAIN_ACTIVATIONS = dict(ACTIVATIONS, relu2=2)


def plain_act(x: torch.Tensor, out: torch.Tensor, activation: str) -> None:
    """``out = act(x)`` element by element in fp32, rounded once (``out`` may be ``x``).
    ``activation``: ``"silu"``, ``"gelu_tanh"`` or ``"relu2"`` (the square of relu)."""
    if activation not in PLAIN_ACTIVATIONS:
        raise KernelError(f"plain_act: unknown activation {activation!r}; known: {sorted(PLAIN_ACTIVATIONS)}")
    _check(x, "x")
    _check(out, "out", x.dtype, tuple(x.shape))
    f = _fn("elementwise", "kvf_plain_act", [c_int, c_void_p, c_void_p, c_long, c_int, c_void_p])
    _ok(f(_tcode(x.dtype), x.data_ptr(), out.data_ptr(), x.numel(), PLAIN_ACTIVATIONS[activation], _stream()),
        "plain_act")


def gated_act_rowgate(gate_up: torch.Tensor, row_gate: torch.Tensor, out: torch.Tensor, activation: str) -> None:
    """``out[m, i] = act(gate_i) * up_i * sigmoid(row_gate[m])`` with (gate, up) at ``(2i, 2i + 1)``
    of the input row; ``row_gate`` fp32 ``[M, >= 1]`` (its first column counts)."""
    m, two_i = gate_up.shape
    if two_i % 2 or activation not in ACTIVATIONS:
        raise KernelError(f"gated_act_rowgate: an even width and one of {sorted(ACTIVATIONS)}")
    _check(gate_up, "gate_up", None, (m, two_i))
    _check(out, "out", gate_up.dtype, (m, two_i // 2))
    _check(row_gate, "row_gate", F32, (m, None), contiguous=False)
    f = _fn("elementwise", "kvf_gated_act_rowgate", [c_int, c_void_p, c_void_p, c_int, c_void_p] + [c_int] * 3 + [c_void_p])
    _ok(f(_tcode(out.dtype), gate_up.data_ptr(), row_gate.data_ptr(), row_gate.stride(0) if m > 1 else 1,
          out.data_ptr(), m, two_i // 2, ACTIVATIONS[activation], _stream()), "gated_act_rowgate")


# ------------------------------------------------------------------------------ matrix products
# Rows of the left operand up to which the weight-streaming MFMA kernel is used for bf16.  Over
# tiled weights it measured faster than the library's product up to 32 rows on the shapes of a
# 1B-parameter decoder (and it folds rotary, cache write, SwiGLU gate and residual sum into its
# store); with more rows the library wins, and the reference's engine uses a library product
# there as well.
SKINNY_MAX_M = 32
FUSED_NORM_MAX_M = 16
FUSED_EPILOGUE_MAX_M = 64
_GEMM_BF16_ARGS = ([c_void_p, c_int, c_void_p, c_int, c_void_p] + [c_int] * 6
                   + [c_float, c_void_p, c_void_p, c_void_p])
# A product that is added to a narrow fp32 stream (few output columns, long K) has too few
# workgroups to pull on the weights with all of the chip: with groups of 16 columns for at most
# half the compute units and from this K on it is cut into two halves of K
# (``k_halves_pay``).  The half that is left owed costs its consumers a second fp32 operand, so
# wider streams lose more there than the product gains (measured at 3072 columns: 7% of the step).
K_HALVES_MIN_K = 4096
_compute_units: dict[int, int] = {}


def compute_units(device) -> int:
    """Compute units of the device, asked of the device once."""
    index = torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if index not in _compute_units:
        _compute_units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _compute_units[index]


class StreamedWeight:
    """A bf16 weight matrix ``[N, K]`` kept twice: ``plain`` as the checkpoint has it (what the
    library product and the fp32 kernels read) and ``tiles``, ``[ceil(N/16), ceil(K/32), 64, 8]``,
    where tile ``(g, s)`` holds rows ``16g..16g+15``, columns ``32s..32s+31`` in the order the
    matrix-core instruction takes them (position ``16*c + r`` holds row ``r``, columns
    ``8c..8c+7``), zero-padded.  The weight-streaming kernel then loads 1 KB of consecutive bytes
    per operand fragment instead of 64 bytes from each of 16 rows, which is what lets it reach
    the memory's bandwidth.  Costs the matrix's size in memory a second time."""

    def __init__(self, plain: torch.Tensor) -> None:
        if plain.dim() != 2 or plain.dtype != BF16 or not plain.is_contiguous():
            raise KernelError("a streamed weight is a contiguous bf16 matrix")
        n, k = plain.shape
        n_pad, k_pad = -(-n // 16) * 16, -(-k // 32) * 32
        padded = plain
        if (n_pad, k_pad) != (n, k):
            padded = torch.zeros(n_pad, k_pad, dtype=BF16, device=plain.device)
            padded[:n, :k] = plain
        self.plain = plain
        self.tiles = (padded.view(n_pad // 16, 16, k_pad // 32, 4, 8).permute(0, 2, 3, 1, 4)
                      .contiguous().view(n_pad // 16, k_pad // 32, 64, 8))
        self.shape, self.dtype, self.device = plain.shape, plain.dtype, plain.device

    def dim(self) -> int:
        return 2


TILE_WEIGHTS = True  # parts keep the matrices they stream for few rows in tiles as well


def streamed(w: torch.Tensor):
    """``w`` ready for ``gemm`` and its fused forms: bf16 matrices on the GPU also in tiles."""
    if (TILE_WEIGHTS and w is not None and w.dtype == BF16 and w.is_cuda and w.dim() == 2
            and w.is_contiguous()):
        return StreamedWeight(w)
    return w


def plain_of(w) -> torch.Tensor:
    return w.plain if isinstance(w, StreamedWeight) else w


def copies_of(w) -> list[torch.Tensor]:
    """Every tensor that holds ``w``: the matrix itself, and its tiles if it is streamed."""
    if isinstance(w, StreamedWeight):
        return [w.plain, w.tiles]
    return [] if w is None else [w]


def _w_args(w) -> tuple[int, int]:
    """(pointer, tiled flag) of a weight for the weight-streaming kernel."""
    if isinstance(w, StreamedWeight):
        return w.tiles.data_ptr(), 1
    return w.data_ptr(), 0


def _gemm_operands(a, w, out, n_out):
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
        raise KernelError("gemm takes 2-D tensors")
    m, k = a.shape
    n, k2 = w.shape
    if k != k2 or tuple(out.shape) != (m, n_out(n)):
        raise KernelError(f"gemm shapes do not agree: a {list(a.shape)}, w {list(w.shape)}, "
                          f"out {list(out.shape)}")
    _check(a, "a", None, None, contiguous=False)
    _check(plain_of(w), "w")
    _check(out, "out", None, None, contiguous=False)
    if a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows of a and out must be dense")
    lda = a.stride(0) if m > 1 else k
    ldc = out.stride(0) if m > 1 else out.shape[1]
    return m, n, k, lda, ldc


def _rows_aligned(a: torch.Tensor, k: int, lda: int) -> bool:
    """Rows that the matrix-core kernels (and the library) read 16 bytes at a time: eight
    elements per step of K, every row and the first one at a multiple of 16 bytes."""
    return k % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0


def bf16_kernel_takes(a: torch.Tensor, w: torch.Tensor, rms: bool = False,
                      fused_epilogue: bool = False) -> bool:
    """Whether the MFMA weight-streaming kernel takes these operands: bf16 weights, bf16 rows
    (or, with ``rms``, fp32 rows), 16-byte aligned rows, at most ``SKINNY_MAX_M`` of them.
    Folding the norm in pays only while every workgroup converts one tile of rows
    (``FUSED_NORM_MAX_M``); beyond that a norm kernel of its own is cheaper.  Where the kernel's
    epilogue stands for a kernel of its own after the library's product (``fused_epilogue``:
    rotary and cache write, the SwiGLU gate) it pays up to ``FUSED_EPILOGUE_MAX_M`` rows."""
    m, k = a.shape
    lda = a.stride(0) if m > 1 else k
    limit = FUSED_NORM_MAX_M if rms else (FUSED_EPILOGUE_MAX_M if fused_epilogue else SKINNY_MAX_M)
    return (w.dtype == BF16 and a.dtype == (F32 if rms else BF16) and _rows_aligned(a, k, lda)
            and m <= limit)


def is_library_product(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm(a, w, ...)`` hands the product to the library: bf16 with more rows than the
    weight-streaming kernel takes; or more than one tile of rows over a deep and narrow weight
    (K >= 2 N), where that kernel has few workgroups and each re-reads every row of ``a`` along
    a long K (measured at [2048, 8192] and 32 rows: 19 us against the library's 15)."""
    m, k = a.shape
    n = w.shape[0]
    lda = a.stride(0) if m > 1 else k
    return (a.dtype == BF16 and w.dtype == BF16 and _rows_aligned(a, k, lda)
            and (m > SKINNY_MAX_M or (m > 16 and k >= 2 * n)))


def k_halves_pay(a: torch.Tensor, w) -> bool:
    """Whether ``gemm(a, w, out, accumulate=True, half_out=...)`` is worth asking for: one tile of
    bf16 rows over a deep weight with few columns (the down projection of a small model)."""
    m, k = a.shape
    return (not is_library_product(a, w) and a.dtype == BF16 and plain_of(w).dtype == BF16
            and k % 8 == 0 and m <= 16 and k >= K_HALVES_MIN_K
            and -(-w.shape[0] // 16) <= compute_units(a.device) // 2)


# The library's product is called through an entry point of our own: torch.mm costs 17 us of
# host time a call, which is what bounds a step that is launched kernel by kernel (a portion of a
# prompt) at a few hundred rows.
LIBRARY_WORKSPACE_BYTES = 76 << 20
_library_ready: dict[int, bool] = {}
_LIBRARY_ARGS = [c_void_p, c_void_p, c_void_p] + [c_int] * 7 + [c_void_p]


def library_ready(device) -> None:
    """Set the library product up on ``device`` (its workspace is allocated here, once): to be
    called outside any stream capture, which ``gemm`` does by itself on its first library
    product."""
    dev = torch.device(device).index
    if dev is None:
        dev = torch.cuda.current_device()
    if _library_ready.get(dev):
        return
    if torch.cuda.is_current_stream_capturing():
        raise KernelError("the library product has to be set up before a stream is captured: "
                          "run the step once (or call ops.library_ready) outside the capture")
    init = _fn("gemm_library", "kvf_gemm_library_init", [c_long])
    with torch.cuda.device(dev):
        _ok(init(LIBRARY_WORKSPACE_BYTES), "gemm_library_init")
    _library_ready[dev] = True


def _library_product(a, w, out, accumulate, m, n, k, lda, ldc) -> None:
    """``out = a @ w.T`` (or ``+=``, in fp32) by hipBLASLt, with fp32 sums stored as ``out`` has
    them.  Raises where the library names no algorithm for the shape."""
    if out.dtype not in (F32, BF16) or (accumulate and out.dtype != F32):
        raise KernelError(f"library product: output must be float32 or bfloat16, got {out.dtype}")
    library_ready(a.device)
    f = _fn("gemm_library", "kvf_gemm_library_bf16", _LIBRARY_ARGS)
    code = f(a.data_ptr(), w.data_ptr(), out.data_ptr(), 1 if out.dtype == F32 else 0,
             1 if accumulate else 0, m, n, k, lda, ldc, _stream())
    if code == -1:
        raise KernelError(f"the library has no bf16 product for {m} x {n} x {k} "
                          f"(row strides {lda} / {ldc})")
    _ok(code, "gemm_library")


def gemm(a: torch.Tensor, w, out: torch.Tensor, accumulate: bool = False,
         owed: torch.Tensor | None = None, half_out: torch.Tensor | None = None) -> None:
    """``out = a @ w.T`` (``accumulate``: ``out += a @ w.T`` with ``out`` fp32).

    ``a: [M, K]`` (row stride may exceed K), ``w: [N, K]`` contiguous or a ``StreamedWeight``,
    ``out: [M, N]``.
    bf16 x bf16 runs on MFMA with fp32 accumulation; any operand in fp32 runs the fp32
    vector-ALU kernel (true 32-bit multiply and accumulate).
    With ``accumulate``: ``owed`` (bf16, shape and row stride of ``out``) is a sum still owed to
    ``out`` and is added on the way; ``half_out`` (bf16, likewise, only where ``k_halves_pay``)
    receives the product over the second half of K *instead of* ``out``, which the caller then
    owes to ``out``: twice the workgroups pull on ``w``."""
    m, n, k, lda, ldc = _gemm_operands(a, w, out, lambda n: n)
    if accumulate and out.dtype != F32:
        raise KernelError("gemm: accumulation needs an fp32 output")
    for t, name in ((owed, "owed"), (half_out, "half_out")):
        if t is None:
            continue
        if not accumulate:
            raise KernelError(f"gemm: {name} goes with accumulate")
        _check(t, name, BF16, (m, n), contiguous=False)
        if t.stride(1) != 1 or (m > 1 and t.stride(0) != ldc):
            raise KernelError(f"gemm: {name} must have the row stride of out")
    if half_out is not None and not k_halves_pay(a, w):
        raise KernelError("gemm: half_out only where k_halves_pay(a, w)")
    if half_out is not None:
        # the workgroups of one half of K read owed and out while those of the other write half_out
        for t, name in ((owed, "owed"), (out, "out")):
            if t is not None and _overlap(t, half_out):
                raise KernelError(f"gemm: half_out must not share memory with {name}")
    if m == 0:
        return
    out_kind = 2 if accumulate else (0 if out.dtype == F32 else 1)
    if not accumulate:
        _tcode(out.dtype)
    if a.dtype == BF16 and w.dtype == BF16 and _rows_aligned(a, k, lda):
        if not is_library_product(a, w):
            f = _fn("gemm_bf16", "kvf_gemm_bf16", _GEMM_BF16_ARGS)
            wp, tiled = _w_args(w)
            _ok(f(a.data_ptr(), 0, wp, tiled, out.data_ptr(), out_kind, m, n, k, lda, ldc, 0.0,
                  owed.data_ptr() if owed is not None else None,
                  half_out.data_ptr() if half_out is not None else None, _stream()), "gemm_bf16")
            return
        if owed is not None:
            add_rows(out, owed)
        _library_product(a, plain_of(w), out, accumulate, m, n, k, lda, ldc)
        return
    if owed is not None:
        add_rows(out, owed)
    w = plain_of(w)
    f = _fn("gemm_generic", "kvf_gemm_generic",
            [c_void_p, c_int, c_void_p, c_int, c_void_p] + [c_int] * 6 + [c_void_p])
    _ok(f(a.data_ptr(), _tcode(a.dtype), w.data_ptr(), _tcode(w.dtype), out.data_ptr(), out_kind,
          m, n, k, lda, ldc, _stream()), "gemm_generic")


def gemm_generic_vector_alus_only(on: bool) -> bool:
    """For tests: keep 32-bit products of many rows on the vector ALUs (the kernel of 64 x 64
    tiles that the matrix-core kernel replaced) or let them go to the matrix cores again.
    Returns the setting before."""
    f = _fn("gemm_generic", "kvf_gemm_generic_vector_alus_only", [c_int])
    return bool(f(1 if on else 0))


def gemm_gated(a: torch.Tensor, w, out: torch.Tensor, activation: str = "silu",
               gate_bias: torch.Tensor | None = None, up_bias: torch.Tensor | None = None,
               rms_eps: float | None = None) -> None:
    """The MFMA weight-streaming product over (gate, up) row pairs of ``w`` with the gate folded
    into its store: ``out[:, j] = act(c[2j] + gate_bias[j]) * (c[2j+1] + up_bias[j])``,
    ``out: [M, N/2]`` bf16.  ``activation``: ``"silu"`` or ``"gelu_tanh"``; biases fp32 ``[N/2]`` or
    ``None``; ``rms_eps`` as in ``gemm_fused``.  Callers check ``bf16_kernel_takes`` first."""
    rms = rms_eps is not None
    m, n, k, lda, ldc = _gemm_operands(a, w, out, lambda n: n // 2)
    if not bf16_kernel_takes(a, w, rms, True):
        raise KernelError("gemm_gated: operands do not fit the MFMA kernel")
    if n % 4 or out.dtype != BF16:
        raise KernelError("gemm_gated: pairs need N in steps of 4 and a bf16 output")
    if activation not in ACTIVATIONS:
        raise KernelError(f"gemm_gated: unknown activation {activation!r}; known: {sorted(ACTIVATIONS)}")
    for b, name in ((gate_bias, "gate_bias"), (up_bias, "up_bias")):
        if b is not None:
            _check(b, name, F32, (n // 2,))
    if m == 0:
        return
    f = _fn("gemm_bf16", "kvf_gemm_bf16_gated",
            [c_void_p, c_int, c_void_p, c_int, c_void_p] + [c_int] * 5 + [c_float, c_int, c_void_p, c_void_p,
                                                                        c_void_p])
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), 1 if rms else 0, wp, tiled, out.data_ptr(), m, n, k, lda, ldc, float(rms_eps or 0.0),
          ACTIVATIONS[activation], gate_bias.data_ptr() if gate_bias is not None else None,
          up_bias.data_ptr() if up_bias is not None else None, _stream()), "gemm_gated")


def gemm_fused(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rms_eps: float | None = None,
               silu_pairs: bool = False, accumulate: bool = False) -> None:
    """The MFMA weight-streaming product with work folded in at both ends.

    ``rms_eps``: ``a`` is the fp32 residual stream and each row is scaled by
    ``rsqrt(mean(a^2) + eps)`` (the norm's weight is already folded into ``w``).
    ``silu_pairs``: columns are (gate, up) pairs and ``out[:, j] = silu(c[2j]) * c[2j+1]``,
    ``out: [M, N/2]`` bf16.  Callers check ``bf16_kernel_takes`` first."""
    rms = rms_eps is not None
    m, n, k, lda, ldc = _gemm_operands(a, w, out, (lambda n: n // 2) if silu_pairs else (lambda n: n))
    if not bf16_kernel_takes(a, w, rms, silu_pairs):
        raise KernelError("gemm_fused: operands do not fit the MFMA kernel")
    if silu_pairs:
        if n % 4 or out.dtype != BF16 or accumulate:
            raise KernelError("gemm_fused: SwiGLU pairs need N in steps of 4 and a bf16 output")
        epi = 3
    elif accumulate:
        if out.dtype != F32:
            raise KernelError("gemm_fused: accumulation needs an fp32 output")
        epi = 2
    else:
        epi = 0 if out.dtype == F32 else 1
        _tcode(out.dtype)
    if m == 0:
        return
    f = _fn("gemm_bf16", "kvf_gemm_bf16", _GEMM_BF16_ARGS)
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), 1 if rms else 0, wp, tiled, out.data_ptr(), epi, m, n, k, lda, ldc,
          float(rms_eps or 0.0), None, None, _stream()), "gemm_bf16")


def gemm_qkv_rope(a: torch.Tensor, w: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                  seq_of_token: torch.Tensor, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  block_table: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, write_kv: bool = True,
                  rms_eps: float | None = None, a_owed: torch.Tensor | None = None,
                  extra_cols: int = 0) -> None:
    """Fused q/k/v projection: ``a @ w.T`` with rotary applied to q and k (neighbouring columns
    are pairs), rotated q stored to ``q_out [M, H*d]`` and rotated k and v written into the
    pages; without tables (``None``) nothing is rotated.  ``rms_eps`` as in ``gemm_fused``.  ``a_owed`` (with ``rms_eps``; bf16, shape and
    strides, counted in elements, of ``a``): a sum still owed to ``a``; the projection is taken of ``a + a_owed``, and
    ``a`` itself is left as it is.  ``extra_cols``: so many further rows of ``w`` behind q, k and v
    (an output gate, say), whose columns of the product are stored behind q, ``q_out [M, H*d +
    extra_cols]``; ``num_kv_heads`` may then be 0 for a projection without keys and values."""
    H, KV, d = num_heads, num_kv_heads, head_dim
    extra = int(extra_cols)
    if extra < 0 or extra % 4:
        raise KernelError(f"gemm_qkv_rope: extra_cols must be a non-negative multiple of 4, got {extra}")
    rms = rms_eps is not None
    m, k = a.shape
    _check(a, "a", None, (m, k), contiguous=False)
    _check(plain_of(w), "w", BF16, ((H + 2 * KV) * d + extra, k))
    if not bf16_kernel_takes(a, w, rms, True) or a.stride(1) != 1:
        raise KernelError("gemm_qkv_rope: operands do not fit the MFMA kernel")
    if a_owed is not None:
        if not rms or m > FUSED_NORM_MAX_M:
            raise KernelError("gemm_qkv_rope: a_owed goes with rms_eps (fp32 rows, one tile of them)")
        _check(a_owed, "a_owed", BF16, (m, k), contiguous=False)
        if a_owed.stride() != a.stride():
            raise KernelError("gemm_qkv_rope: a_owed must have the strides of a")
    _check(q_out, "q_out", BF16, (m, H * d + extra))
    _check(positions, "positions", I32, (None,))
    _check(seq_of_token, "seq_of_token", I32, (None,))
    if positions.shape[0] < m or seq_of_token.shape[0] < m:
        raise KernelError("gemm_qkv_rope: positions / seq_of_token shorter than the batch")
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, d, "gemm_qkv_rope")
    if d % 4:
        raise KernelError(f"gemm_qkv_rope: head_dim {d} not supported")
    _check(block_table, "block_table", I32, (None, None))
    if KV == 0 and write_kv:
        raise KernelError("gemm_qkv_rope: a projection without keys and values writes no cache")
    _check(k_pages, "k_pages", BF16, (None, KV if KV else None, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", BF16, (nb, k_pages.shape[1], d, bs))
    if m == 0:
        return
    f = _fn("gemm_bf16", "kvf_gemm_bf16_qkv_rope",
            [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float]
            + [c_void_p] * 8 + [c_int] * 11 + [c_void_p])
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), 1 if rms else 0, wp, tiled, q_out.data_ptr(), m, k,
          a.stride(0) if m > 1 else k, q_out.stride(0) if m > 1 else H * d + extra, float(rms_eps or 0.0),
          a_owed.data_ptr() if a_owed is not None else None, positions.data_ptr(), seq_of_token.data_ptr(), cos_p, sin_p,
          block_table.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), H, KV, d, rot,
          table_len, bs, block_table.shape[1], nb, 1 if write_kv else 0, block_table.shape[0],
          extra, _stream()), "gemm_qkv_rope")


def pick_workspace(rows: int, n: int, device) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Scratch of ``gemm_pick`` for ``rows`` rows over ``n`` columns: the workgroups' best values
    and columns, and the ticket (one int, zero between launches)."""
    pick_groups = _fn("gemm_bf16", "kvf_gemm_bf16_pick_groups", [c_int, c_int])
    # few rows take fewer columns per workgroup, hence more workgroups: room for any count up to rows
    groups = max(int(pick_groups(m, int(n))) for m in range(1, int(rows) + 1))
    tickets = int(_fn("gemm_bf16", "kvf_gemm_bf16_pick_ticket_ints", [])())
    return (torch.empty(16 * groups + 16 * 64, dtype=F32, device=device),
            torch.empty(16 * groups + 16 * 64, dtype=I32, device=device),
            torch.zeros(tickets, dtype=I32, device=device))


def gemm_pick(a: torch.Tensor, w, residual: torch.Tensor, tokens: torch.Tensor,
              token_ids: torch.Tensor, positions: torch.Tensor, ctx_lens: torch.Tensor,
              ring: torch.Tensor, run_counter: torch.Tensor, embed: torch.Tensor, work: tuple) -> None:
    """The output head of a decode step with everything after it folded in: ``a`` (the
    normalised rows, bf16, at most 16, one per sequence) is multiplied by ``w``, the largest
    logit of every row is picked without the logits being stored (lowest column among equal
    ones), and the picked token becomes its sequence's next input exactly as ``decode_advance``
    does it; the tokens' rows of ``embed`` are then written into ``residual`` (fp32, a row per
    sequence) as the next step's residual stream.  ``work``: from ``pick_workspace``; launches
    that share it must not overlap."""
    m, k = a.shape
    _check(a, "a", BF16, (m, k), contiguous=False)
    if a.stride(1) != 1 or m > FUSED_NORM_MAX_M or m == 0:
        raise KernelError(f"gemm_pick takes 1 to {FUSED_NORM_MAX_M} dense bf16 rows")
    _check(plain_of(w), "w", BF16, (None, k))
    n = w.shape[0]
    if not bf16_kernel_takes(a, w):
        raise KernelError("gemm_pick: operands do not fit the MFMA kernel")
    _check(residual, "residual", F32, (m, k), contiguous=False)
    if residual.stride(1) != 1 or (m > 1 and residual.stride(0) % 4):
        raise KernelError("gemm_pick: rows of the residual stream must be dense and start on 16 bytes")
    for t, name in ((tokens, "tokens"), (token_ids, "token_ids"), (positions, "positions"),
                    (ctx_lens, "ctx_lens")):
        _check(t, name, I32, (None,))
        if t.shape[0] < m:
            raise KernelError(f"gemm_pick: {name} is shorter than the batch")
    _check(ring, "ring", I32, (None, None))
    _check(run_counter, "run_counter", I32, (1,))
    if ring.shape[1] < m:
        raise KernelError("gemm_pick: rows of the ring are shorter than the batch")
    _check(embed, "embed", BF16, (None, k))
    if embed.shape[0] < n or k % 8:
        raise KernelError("gemm_pick: the embedding table must hold a row of K elements (a multiple "
                          "of 8) for every column of w")
    part_val, part_idx, ticket = work
    groups = int(_fn("gemm_bf16", "kvf_gemm_bf16_pick_groups", [c_int, c_int])(m, n))
    _check(part_val, "work[0]", F32, (None,))
    _check(part_idx, "work[1]", I32, (None,))
    _check(ticket, "work[2]", I32, (int(_fn("gemm_bf16", "kvf_gemm_bf16_pick_ticket_ints", [])()),))
    if part_val.shape[0] < 16 * groups + 16 * 64 or part_idx.shape[0] < 16 * groups + 16 * 64:
        raise KernelError("gemm_pick: workspace too small for these rows and columns")
    f = _fn("gemm_bf16", "kvf_gemm_bf16_pick",
            [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int] + [c_void_p] * 9
            + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p])
    wp, tiled = _w_args(w)
    _ok(f(a.data_ptr(), wp, tiled, m, n, k, a.stride(0) if m > 1 else k, part_val.data_ptr(),
          part_idx.data_ptr(), ticket.data_ptr(), tokens.data_ptr(), token_ids.data_ptr(),
          positions.data_ptr(), ctx_lens.data_ptr(), ring.data_ptr(), run_counter.data_ptr(),
          ring.shape[1], ring.shape[0], embed.data_ptr(), residual.data_ptr(), k,
          residual.stride(0) if m > 1 else k, _stream()), "gemm_pick")


def set_gemm_waves(waves: int, rows: int = 0) -> None:
    """Measurement aid: force the waves per workgroup and the rows of W per workgroup of the
    MFMA kernel (0 = by shape)."""
    lib = library.load("gemm_bf16")
    for fn, v in ((lib.kvf_gemm_bf16_set_waves, waves), (lib.kvf_gemm_bf16_set_rows, rows)):
        fn.argtypes = [c_int]
        fn.restype = None
        fn(int(v))


# ------------------------------------------------------------------------------ attention
def _attn_common(q, k_pages, v_pages, block_table, cu_q, ctx_lens, out, H, KV, d):
    if d % 16 or d > 256 or d <= 0:
        raise KernelError(f"attention kernels take head sizes in steps of 16 up to 256, got {d}")
    if H % KV:
        raise KernelError(f"query heads ({H}) must be a multiple of kv heads ({KV})")
    _check(q, "q", None, (None, None), contiguous=False)
    if q.stride(1) != 1 or q.shape[1] < H * d:
        raise KernelError("attention: q rows must be dense and hold all query heads")
    _check(k_pages, "k_pages", q.dtype, (None, KV, None, d))
    nb, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", q.dtype, (nb, KV, d, bs))
    _check(block_table, "block_table", I32, (None, None))
    n_seqs = block_table.shape[0]
    _check(cu_q, "cu_q", I32, (None,))
    _check(ctx_lens, "ctx_lens", I32, (None,))
    if cu_q.shape[0] < n_seqs + 1 or ctx_lens.shape[0] < n_seqs:
        raise KernelError("attention: cu_q / ctx_lens shorter than the block table")
    _check(out, "out", q.dtype, (None, H * d))
    if out.shape[0] < q.shape[0]:
        raise KernelError("attention: out has fewer rows than q")
    return n_seqs


def _slopes_ptr(slopes, H: int, like: torch.Tensor):
    """Pointer to the per-head slopes of a bias by distance, or ``None`` for attention without."""
    if slopes is None:
        return None
    _check(slopes, "slopes", F32, (H,))
    if slopes.device != like.device:
        raise KernelError("attention: slopes live on another device than q")
    return slopes.data_ptr()


def _sinks_ptr(sinks, H: int, like: torch.Tensor):
    """Pointer to the per-head sink scores (fp32 ``[H]``), or ``None`` for a softmax without."""
    if sinks is None:
        return None
    _check(sinks, "sinks", F32, (H,))
    if sinks.device != like.device:
        raise KernelError("attention: sinks live on another device than q")
    return sinks.data_ptr()


def _no_sinks_with_slopes(sinks, slopes, on_matrix_cores: bool) -> None:
    if sinks is not None and slopes is not None and on_matrix_cores:
        raise KernelError("attention: the matrix-core kernels take sinks or slopes, not both")


def _score_cap(cap, sinks, slopes, on_matrix_cores: bool) -> float:
    """The cap on scaled scores as the kernels take it (0: none)."""
    if cap is None:
        return 0.0
    if not cap > 0.0:
        raise KernelError(f"attention: the score cap must be positive, got {cap}")
    if on_matrix_cores and (sinks is not None or slopes is not None):
        raise KernelError("attention: the matrix-core kernels cap scores without sinks and slopes only")
    return float(cap)


def _keep_first(window: int, keep_first: int) -> int:
    """Keys kept visible behind a window; without a window every key is visible anyway."""
    keep = int(keep_first)
    if keep < 0:
        raise KernelError(f"attention: keep_first must not be negative, got {keep}")
    return keep if int(window) > 0 else 0


def _mask_arg(window: int, chunk: int) -> int:
    """What the attention kernels take as their mask: a window ``w`` as ``w``, chunks of ``c``
    positions as ``-c``, neither as 0."""
    window, chunk = int(window or 0), int(chunk or 0)
    if window < 0 or chunk < 0 or (window and chunk):
        raise KernelError(f"attention: a window ({window}) or chunks ({chunk}), not negative and not both")
    return -chunk if chunk else window


def _gate_args(gate, q: torch.Tensor, cols: int):
    """(pointer, row stride) of an output gate, or (None, 0)."""
    if gate is None:
        return None, 0
    _check(gate, "gate", q.dtype, (None, cols), contiguous=False)
    if gate.shape[0] < q.shape[0] or gate.stride(1) != 1 or gate.stride(0) % 4 or gate.data_ptr() % 8:
        raise KernelError("attention: the gate needs a row per token, dense rows that start on 8 bytes")
    return gate.data_ptr(), gate.stride(0)


def attention_on_matrix_cores(dtype: torch.dtype, block_size: int) -> bool:
    """The MFMA attention kernels take bf16 and pages of a multiple of 8 tokens; everything else
    (the true 32-bit path above all) runs the vector-ALU kernel."""
    return dtype == BF16 and block_size % 8 == 0


def prefill_rows_per_item(dtype: torch.dtype, head_dim: int, block_size: int, row_tiles: int = 1) -> int:
    """Rows of (query token, head in group) that one entry of a prefill work list covers.
    ``row_tiles``: 1 or 2 tiles of 16 rows per wave of the matrix-core kernel (two where the head
    size allows them; they pay when the work fills the chip anyway, see ``attn_mfma.hip``)."""
    if attention_on_matrix_cores(dtype, block_size):
        return int(_fn("attn_mfma", "kvf_attn_mfma_rows_per_item", [c_int, c_int])(int(head_dim), int(row_tiles)))
    return int(_fn("attn_generic", "kvf_attn_generic_rows_per_item", [])())


_blocks_per_cu: dict[tuple, int] = {}


def prefill_blocks_per_cu(dtype: torch.dtype, head_dim: int, block_size: int, row_tiles: int = 1) -> int:
    """Workgroups of the kernel for query runs that one compute unit holds at a time (by its
    registers and LDS, asked of the runtime once): what fills the chip is this many times the
    compute units."""
    key = (dtype, int(head_dim), int(block_size) % 8 == 0, int(row_tiles))
    if key not in _blocks_per_cu:
        n = 4
        if attention_on_matrix_cores(dtype, block_size):
            n = int(_fn("attn_mfma", "kvf_attn_mfma_prefill_blocks_per_cu", [c_int, c_int])(int(head_dim), int(row_tiles)))
        _blocks_per_cu[key] = max(1, n)
    return _blocks_per_cu[key]


def attn_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                 block_table: torch.Tensor, cu_q: torch.Tensor, ctx_lens: torch.Tensor,
                 work: torch.Tensor, out: torch.Tensor, num_heads: int, num_kv_heads: int,
                 head_dim: int, scale: float, window: int = 0,
                 slopes: torch.Tensor | None = None, rows_per_item: int | None = None,
                 keep_first: int = 0, gate: torch.Tensor | None = None,
                 sinks: torch.Tensor | None = None, score_cap: float | None = None,
                 chunk: int = 0) -> None:
    """Causal attention of query runs over the paged cache.  ``work``: ``[num_work, 3]`` rows
    (sequence row, item, item or -1) where a sequence has ``query_len * H/KV`` rows per kv head,
    an item covers ``rows_per_item`` of them (what ``prefill_rows_per_item`` gave when the rows
    were made; by default its answer for one row tile), and the items of one row are taken by
    one workgroup in turn; rows start in the order given (the longest walks first).  ``v_pages`` are transposed:
    ``[num_blocks, KV, head_dim, block_size]``.  ``slopes``: fp32 ``[H]``; the score of key ``j``
    for a query at position ``p`` of head ``h`` then is ``scale * q.k + slopes[h] * (j - p)``.
    ``keep_first``: with a window, the first so many keys of a sequence stay visible behind it.
    ``gate`` (``[tokens, H*d]``, dense rows, type of ``q``): an output gate; what is stored is the
    attention output times ``sigmoid(gate)``, element by element, in the matrix-core kernels'
    store (the 32-bit kernels take no gate: their caller runs ``sigmoid_gate`` behind them).
    ``sinks``: fp32 ``[H]``; the softmax's denominator of head ``h`` then holds one more term
    ``exp(sinks[h])``, a key without a value whose score is not scaled.
    ``score_cap``: the scaled score ``s`` becomes ``score_cap * tanh(s / score_cap)`` (the
    matrix-core kernels have it without sinks and slopes only).
    ``chunk``: positions are cut into chunks of so many, counted from position 0 of the sequence,
    and a query sees only the keys of its own chunk (instead of a window, not beside one)."""
    H, KV, d = num_heads, num_kv_heads, head_dim
    window = _mask_arg(window, chunk)
    n_seqs = _attn_common(q, k_pages, v_pages, block_table, cu_q, ctx_lens, out, H, KV, d)
    cap = _score_cap(score_cap, sinks, slopes, attention_on_matrix_cores(q.dtype, k_pages.shape[2]))
    _check(work, "work", I32, (None, 3))
    keep = _keep_first(window, keep_first)
    gp, gs = _gate_args(gate, q, H * d)
    sl = _slopes_ptr(slopes, H, q)
    sk = _sinks_ptr(sinks, H, q)
    nb, _, bs, _ = k_pages.shape
    if rows_per_item is None:
        rows_per_item = prefill_rows_per_item(q.dtype, d, bs)
    _no_sinks_with_slopes(sinks, slopes, attention_on_matrix_cores(q.dtype, bs))
    if attention_on_matrix_cores(q.dtype, bs):
        if window < 0 and (sinks is not None or slopes is not None or cap > 0.0):
            raise KernelError("attn_prefill: the matrix-core kernel has chunks of positions with plain scores "
                              "only (no sinks, slopes or score cap beside them)")
        f = _fn("attn_mfma", "kvf_attn_mfma_prefill",
                [c_void_p] * 7 + [c_int, c_int] + [c_void_p] + [c_int] * 11 + [c_float, c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p])
        _ok(f(q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(),
              cu_q.data_ptr(), ctx_lens.data_ptr(), work.data_ptr(), work.shape[0], int(rows_per_item), out.data_ptr(),
              H, KV, d, bs, nb, block_table.shape[1], q.stride(0), out.stride(0), int(window), keep,
              n_seqs, float(scale), sl, gp, gs, sk, cap, _stream()), "attn_mfma_prefill")
        return
    if gate is not None:
        raise KernelError("attn_prefill: the 32-bit kernel takes no gate; gate its rows afterwards")
    if rows_per_item != prefill_rows_per_item(q.dtype, d, bs):
        raise KernelError(f"attn_prefill: the 32-bit kernel takes items of "
                          f"{prefill_rows_per_item(q.dtype, d, bs)} rows, got {rows_per_item}")
    if q.stride(0) % 4 or out.stride(0) % 4:
        raise KernelError("attn_prefill: rows of q and out must start on 16 bytes")
    f = _fn("attn_generic", "kvf_attn_generic",
            [c_int] + [c_void_p] * 7 + [c_int] + [c_void_p] + [c_int] * 11
            + [c_float, c_void_p, c_void_p, c_float, c_void_p])
    _ok(f(_tcode(q.dtype), q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
          block_table.data_ptr(), cu_q.data_ptr(), ctx_lens.data_ptr(), work.data_ptr(),
          work.shape[0], out.data_ptr(), H, KV, d, bs, nb, block_table.shape[1], q.stride(0),
          out.stride(0), int(window), keep, n_seqs, float(scale), sl, sk, cap, _stream()), "attn_generic")


def attn_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                block_table: torch.Tensor, seq_ids: torch.Tensor | None, num_seqs: int,
                cu_q: torch.Tensor, ctx_lens: torch.Tensor, out: torch.Tensor, num_heads: int,
                num_kv_heads: int, head_dim: int, scale: float, window: int = 0, splits: int = 1,
                workspace: tuple[torch.Tensor, torch.Tensor] | None = None,
                token_is_seq: bool = False, slopes: torch.Tensor | None = None,
                keep_first: int = 0, gate: torch.Tensor | None = None,
                sinks: torch.Tensor | None = None, score_cap: float | None = None,
                chunk: int = 0) -> None:
    """Attention of one-token queries: sequence rows ``seq_ids[:num_seqs]`` (or ``0..num_seqs-1``)
    each attend from their token ``cu_q[seq]`` over ``ctx_lens[seq]`` cached keys.  The key
    range may be cut into ``splits`` runs; ``workspace`` then holds fp32 partial accumulators
    (``num_seqs * H * splits * d``) and fp32 (max, sum) pairs (``num_seqs * H * splits * 2``).
    ``token_is_seq``: the caller vouches that ``cu_q[i] == i`` for every sequence (a batch of
    single tokens), which spares the matrix-core kernel a dependent load.  ``slopes``: as in
    ``attn_prefill``; ``keep_first`` and ``gate`` likewise (the matrix-core kernels only: the
    32-bit path is given no gate, its caller gates the rows afterwards); ``sinks`` likewise (all
    kernels; with cuts the term joins the sum where the cuts are merged); ``score_cap`` and
    ``chunk`` likewise."""
    H, KV, d = num_heads, num_kv_heads, head_dim
    window = _mask_arg(window, chunk)
    n_seqs = _attn_common(q, k_pages, v_pages, block_table, cu_q, ctx_lens, out, H, KV, d)
    cap = _score_cap(score_cap, sinks, slopes, attention_on_matrix_cores(q.dtype, k_pages.shape[2]))
    sl = _slopes_ptr(slopes, H, q)
    sk = _sinks_ptr(sinks, H, q)
    keep = _keep_first(window, keep_first)
    gp, gs = _gate_args(gate, q, H * d)
    if token_is_seq and seq_ids is not None:
        raise KernelError("attn_decode: token_is_seq is for batches where every sequence decodes")
    if seq_ids is not None:
        _check(seq_ids, "seq_ids", I32, (None,))
        if seq_ids.shape[0] < num_seqs:
            raise KernelError("attn_decode: seq_ids shorter than num_seqs")
    elif num_seqs > n_seqs:
        raise KernelError("attn_decode: more sequences than block-table rows")
    nb, _, bs, _ = k_pages.shape
    if not 1 <= splits <= 64:
        raise KernelError(f"attn_decode: 1 to 64 cuts of the key range, got {splits}")
    pa = pm = None
    if splits > 1:
        if workspace is None:
            raise KernelError("attn_decode: splits > 1 need a workspace")
        pa, pm = workspace[0], workspace[1]
        _check(pa, "workspace[0]", F32)
        _check(pm, "workspace[1]", F32)
        if pa.numel() < num_seqs * H * splits * d or pm.numel() < num_seqs * H * splits * 2:
            raise KernelError("attn_decode: workspace too small")
    _no_sinks_with_slopes(sinks, slopes, attention_on_matrix_cores(q.dtype, bs))
    if not attention_on_matrix_cores(q.dtype, bs):
        if gate is not None:
            raise KernelError("attn_decode: the 32-bit kernel takes no gate; gate its rows afterwards")
        f = _fn("attn_generic", "kvf_attn_generic_decode",
                [c_int] + [c_void_p] * 10 + [c_int] * 13 + [c_float, c_void_p, c_void_p, c_float, c_void_p])
        _ok(f(_tcode(q.dtype), q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
              block_table.data_ptr(), seq_ids.data_ptr() if seq_ids is not None else None,
              None if token_is_seq else cu_q.data_ptr(), ctx_lens.data_ptr(), out.data_ptr(),
              pa.data_ptr() if pa is not None else None, pm.data_ptr() if pm is not None else None,
              num_seqs, H, KV, d, bs, nb, block_table.shape[1], q.stride(0), out.stride(0),
              int(window), keep, n_seqs, int(splits), float(scale), sl, sk, cap, _stream()), "attn_generic_decode")
        return
    f = _fn("attn_mfma", "kvf_attn_mfma_decode",
            [c_void_p] * 10 + [c_int] * 13 + [c_float, c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p])
    _ok(f(q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(),
          seq_ids.data_ptr() if seq_ids is not None else None,
          None if token_is_seq else cu_q.data_ptr(),
          ctx_lens.data_ptr(), out.data_ptr(), pa.data_ptr() if pa is not None else None,
          pm.data_ptr() if pm is not None else None, num_seqs, H, KV, d, bs, nb,
          block_table.shape[1], q.stride(0), out.stride(0), int(window), keep, n_seqs, int(splits),
          float(scale), sl, gp, gs, sk, cap, _stream()), "attn_mfma_decode")


# ------------------------------------------------------------------------------ matrix-memory recurrence
MLSTM_CHUNK_FROM = 8     # runs of at least so many tokens go chunk by chunk on the matrix cores
MLSTM_MULTI_FROM = 192   # and runs of at least so many through the passes that take all chunks at once


def mlstm_chunk_len(key_dim: int) -> int:
    """Tokens of a chunk of the matrix-core kernels for heads of this key size."""
    return 64 if key_dim <= 128 else 32


def mlstm_multi_plan(q_lens, key_dim: int, multi_from: int = MLSTM_MULTI_FROM) -> tuple[list[int], list[int]]:
    """For the runs of at least ``multi_from`` tokens among ``q_lens`` (a step's runs in sequence
    order): the flat rows ``(sequence, first token, tokens, 0)`` of their chunks and
    ``(sequence, first chunk, chunks)`` of the runs, as ``mlstm_scan(multi=...)`` wants them."""
    cl = mlstm_chunk_len(key_dim)
    chunks: list[int] = []
    runs: list[int] = []
    start = 0
    for seq, q in enumerate(q_lens):
        if q >= multi_from:
            first = len(chunks) // 4
            for t in range(0, q, cl):
                chunks += [seq, start + t, min(cl, q - t), 0]
            runs += [seq, first, len(chunks) // 4 - first]
        start += q
    return chunks, runs


def mlstm_multi_scratch(n_tokens: int, n_chunks: int, heads: int, key_dim: int, value_dim: int) -> dict[str, tuple]:
    """(shape, dtype) of the scratch tensors the passes over all chunks need, by name."""
    H, dk, dv = int(heads), int(key_dim), int(value_dim)
    return {"li": ((n_tokens, H), F32), "mt": ((n_tokens, H), F32), "bc": ((n_tokens, H), torch.float64),
            "mc": ((n_chunks, H), F32), "gl": ((n_chunks, H), F32), "W": ((n_chunks, H, dk, dv), F32),
            "un": ((n_chunks, H, dk), F32)}


def mlstm_state_floats(heads: int, key_dim: int, value_dim: int) -> int:
    """fp32 numbers of one request's state: per head the matrix ``[key_dim, value_dim]``, the
    normaliser ``[key_dim]`` and the running maximum."""
    return heads * (key_dim * value_dim + key_dim + 1)


def mlstm_scan(rows: torch.Tensor, gates: torch.Tensor, gate_bias: torch.Tensor, cu_q: torch.Tensor,
               positions: torch.Tensor, slot_ids: torch.Tensor, state: torch.Tensor, out: torch.Tensor,
               num_seqs: int, heads: int, key_dim: int, value_dim: int, q_off: int, k_off: int,
               v_off: int, cap: float, q_scale: float, chunk_from: int = MLSTM_CHUNK_FROM,
               short_runs: bool = True, long_runs: bool = True, multi_from: int | None = None,
               multi: dict | None = None) -> None:
    """The matrix-memory recurrence over every sequence's tokens of this step, from and into the
    sequences' state slots.  ``rows [N, >= ...]``: projected rows holding q (``heads * key_dim``
    elements from column ``q_off``), k (from ``k_off``) and v (``heads * value_dim`` from
    ``v_off``); ``gates [N, 2 heads]`` fp32: input-gate then forget-gate pre-activations, to
    (rows may be longer) which ``gate_bias [2 heads]`` is added before the cap ``cap * tanh(z / cap)``; the forget
    gate's log is ``logsigmoid`` of its capped value.  ``state [slots, mlstm_state_floats]``
    fp32; a sequence whose first token of the step sits at position 0 starts from zeros whatever
    its slot holds; a negative slot skips the sequence.  ``out [N, heads * value_dim]`` fp32: the
    heads' outputs ``S^T q / (max(|n . q|, exp(-m)) + 1e-6)`` with ``q`` times ``q_scale``.
    Two kernels share the work: runs of fewer than ``chunk_from`` tokens are walked token by
    token, longer ones a chunk at a time on the matrix cores (in fp32); ``short_runs`` /
    ``long_runs`` say which of the two are launched (a caller that knows its runs' lengths
    spares the other launch).  ``multi``: for runs of at least ``multi_from`` tokens, whose chunks
    are then taken all at once by four passes (gates, every chunk's own contribution, the
    carry over a run's chunks, the outputs): ``chunks`` ``[n, 4]`` and ``runs`` ``[r, 3]`` (int32,
    from ``mlstm_multi_plan``) and the scratch tensors of ``mlstm_multi_scratch``; without it no
    run is that long for the kernels (``multi_from`` is then ignored)."""
    n = rows.shape[0]
    H, dk, dv = int(heads), int(key_dim), int(value_dim)
    _check(rows, "rows", None, (n, None), contiguous=False)
    if rows.stride(1) != 1:
        raise KernelError("mlstm_scan: rows must be dense")
    for off, size, name in ((q_off, H * dk, "q"), (k_off, H * dk, "k"), (v_off, H * dv, "v")):
        if off < 0 or off + size > rows.shape[1]:
            raise KernelError(f"mlstm_scan: {name} at columns {off}..{off + size} lies outside rows of {rows.shape[1]}")
    if not 0 < dk <= 256:
        raise KernelError(f"mlstm_scan: key sizes up to 256, got {dk}")
    _check(gates, "gates", F32, (n, None))
    if gates.shape[1] < 2 * H:
        raise KernelError(f"mlstm_scan: gate rows of {gates.shape[1]} numbers do not hold {2 * H} gates")
    _check(gate_bias, "gate_bias", F32, (2 * H,))
    _check(cu_q, "cu_q", I32, (None,))
    _check(positions, "positions", I32, (None,))
    _check(slot_ids, "slot_ids", I32, (None,))
    if cu_q.shape[0] < num_seqs + 1 or slot_ids.shape[0] < num_seqs or positions.shape[0] < n:
        raise KernelError("mlstm_scan: cu_q / slot_ids / positions shorter than the batch")
    _check(state, "state", F32, (None, mlstm_state_floats(H, dk, dv)))
    _check(out, "out", F32, (n, H * dv))
    if chunk_from < 1:
        raise KernelError(f"mlstm_scan: chunk_from must be positive, got {chunk_from}")
    n_chunks = n_runs = 0
    extra = [None] * 9
    big = 2**31 - 1
    if multi is not None:
        multi_from = MLSTM_MULTI_FROM if multi_from is None else int(multi_from)
        if multi_from < chunk_from:
            raise KernelError("mlstm_scan: multi_from must not be below chunk_from")
        _check(multi["chunks"], "chunks", I32, (None, 4))
        _check(multi["runs"], "runs", I32, (None, 3))
        n_chunks, n_runs = multi["chunks"].shape[0], multi["runs"].shape[0]
        for name, (shape, dtype) in mlstm_multi_scratch(n, n_chunks, H, dk, dv).items():
            _check(multi[name], name, dtype, shape)
        extra = [multi[k].data_ptr() for k in ("chunks", "runs", "li", "mt", "bc", "mc", "gl", "W", "un")]
    f = _fn("mlstm", "kvf_mlstm_scan", [c_int] + [c_void_p] * 8 + [c_int] * 10 + [c_float, c_float] + [c_int] * 6
            + [c_void_p] * 9 + [c_void_p])
    _ok(f(_tcode(rows.dtype), rows.data_ptr(), gates.data_ptr(), gate_bias.data_ptr(), cu_q.data_ptr(),
          positions.data_ptr(), slot_ids.data_ptr(), state.data_ptr(), out.data_ptr(), int(num_seqs),
          H, dk, dv, rows.stride(0) if n > 1 else rows.shape[1], int(q_off), int(k_off), int(v_off),
          state.shape[0], gates.shape[1], float(cap), float(q_scale), int(chunk_from), 1 if short_runs else 0,
          1 if long_runs else 0, multi_from if multi is not None else big, n_chunks, n_runs, *extra,
          _stream()), "mlstm_scan")


def mlstm_out(heads_raw: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float,
              out: torch.Tensor, heads: int, value_dim: int) -> None:
    """``out[n, h, :] = o / rms(o) * weight[h, :] * sigmoid(gate[n, h, :])`` for the raw heads
    ``o = heads_raw[n, h, :]`` (fp32): the root mean square is taken per head over its
    ``value_dim`` elements, ``eps`` inside the root.  ``gate``: dense rows of ``out``'s type (a
    view of wider rows is fine)."""
    n = heads_raw.shape[0]
    H, dv = int(heads), int(value_dim)
    _check(heads_raw, "heads_raw", F32, (n, H * dv))
    _check(weight, "weight", F32, (H * dv,))
    _check(out, "out", None, (n, H * dv))
    _check(gate, "gate", out.dtype, (n, H * dv), contiguous=False)
    if gate.stride(1) != 1:
        raise KernelError("mlstm_out: gate rows must be dense")
    f = _fn("mlstm", "kvf_mlstm_out", [c_int, c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p] + [c_int] * 3 + [c_void_p])
    _ok(f(_tcode(out.dtype), heads_raw.data_ptr(), gate.data_ptr(), gate.stride(0) if n > 1 else H * dv,
          weight.data_ptr(), float(eps), out.data_ptr(), n, H, dv, _stream()), "mlstm_out")


# ------------------------------------------------------------------------------ latent attention
def latent_split(proj: torch.Tensor, qkv: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                 heads: int, dim: int, rot: int, rank: int, head_dim: int) -> None:
    """A projected row ``[heads x (dim | rot) | latent (rank) | shared key part (rot)]`` becomes
    the attention kernels' row ``[heads + 2, head_dim]``: q head ``h`` gets its ``rot`` part in
    front (columns ``rot..rot+rank-1`` are left for ``head_product`` to fill, the rest is
    zero), the one k head is ``[key part | norm(latent) | 0]`` and the one v head
    ``[0 | norm(latent) | 0]``, the norm being ``x / sqrt(mean(x^2) + eps) * norm_weight`` in
    fp32 with one rounding."""
    n = proj.shape[0]
    H, d = int(heads), int(head_dim)
    _check(proj, "proj", None, (n, None), contiguous=False)
    _check(qkv, "qkv", proj.dtype, (n, (H + 2) * d))
    _check(norm_weight, "norm_weight", F32, (rank,))
    if proj.stride(1) != 1 or proj.shape[1] < H * (dim + rot) + rank + rot or d < rot + rank:
        raise KernelError(f"latent_split: rows of {proj.shape[1]} elements / heads of {d} do not hold "
                          f"{H} x ({dim} + {rot}) + {rank} + {rot}")
    f = _fn("latent", "kvf_latent_split", [c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_float]
            + [c_int] * 6 + [c_void_p])
    _ok(f(_tcode(proj.dtype), proj.data_ptr(), proj.stride(0) if n > 1 else proj.shape[1], qkv.data_ptr(),
          qkv.shape[1], norm_weight.data_ptr(), float(eps), n, H, int(dim), int(rot), int(rank), d,
          _stream()), "latent_split")


def head_product(x: torch.Tensor, in_head: int, w: torch.Tensor, out: torch.Tensor, out_head: int) -> None:
    """``out[n, h * out_head + o] = sum_i w[h, o, i] * x[n, h * in_head + i]`` for per-head
    matrices ``w [H, O, I]``: ``x`` and ``out`` are rows (views of wider rows are fine) in which
    head ``h`` starts ``h * in_head`` / ``h * out_head`` elements in.  fp32 multiply and add."""
    n = x.shape[0]
    _check(w, "w", None, (None, None, None))
    H, O, I = w.shape
    _check(x, "x", None, (n, None), contiguous=False)
    _check(out, "out", x.dtype, (n, None), contiguous=False)
    if x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("head_product: rows must be dense")
    if (H - 1) * in_head + I > x.shape[1] or (H - 1) * out_head + O > out.shape[1] or in_head < 0 or out_head < 0:
        raise KernelError(f"head_product: {H} heads of {I} / {O} elements do not fit rows of "
                          f"{x.shape[1]} / {out.shape[1]}")
    if _overlap(x, out):
        raise KernelError("head_product: out must not share memory with x")
    f = _fn("latent", "kvf_head_product", [c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p]
            + [c_int] * 6 + [c_void_p])
    _ok(f(_tcode(x.dtype), _tcode(w.dtype), x.data_ptr(), x.stride(0) if n > 1 else x.shape[1], int(in_head),
          w.data_ptr(), out.data_ptr(), out.stride(0) if n > 1 else out.shape[1], int(out_head), n, H, O, I,
          _stream()), "head_product")


# ------------------------------------------------------------------------------ decaying matrix memory
def wkv_state_floats(heads: int, dim: int, width: int) -> int:
    """fp32 numbers of a request's slot: every head's ``S [dim, dim]``, then the last input row."""
    return heads * dim * dim + width


def wkv_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, prev_off: int, slot_ids: torch.Tensor,
            seq_of_token: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor, out: torch.Tensor,
            n_seqs: int) -> None:
    """``out[m, t] = h[t] + (h_prev[t] - h[t]) * mu[m]`` for ``mu [M, width]`` (fp32): ``h_prev``
    is the row before ``t`` in its query run, for a run's first token the row kept at
    ``prev_off`` in the sequence's state slot (zeros at position 0 or without a slot); the last
    row of every run is left in its slot."""
    n, width = h.shape
    _check(h, "h", None, (n, width))
    _check(mu, "mu", F32, (None, width))
    M = mu.shape[0]
    _check(out, "out", h.dtype, (M, n, width))
    _check(state, "state", F32, (None, None))
    for t, name in ((slot_ids, "slot_ids"), (seq_of_token, "seq_of_token"), (cu_q, "cu_q"), (positions, "positions")):
        _check(t, name, I32, (None,))
    if seq_of_token.shape[0] < n or positions.shape[0] < n or cu_q.shape[0] < n_seqs + 1 or slot_ids.shape[0] < n_seqs:
        raise KernelError("wkv_mix: batch arrays shorter than the batch")
    if prev_off < 0 or prev_off + width > state.shape[1]:
        raise KernelError("wkv_mix: the kept row does not fit the slot")
    f = _fn("wkv", "kvf_wkv_mix", [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int] + [c_void_p] * 5
            + [c_int] * 5 + [c_void_p])
    _ok(f(_tcode(h.dtype), h.data_ptr(), mu.data_ptr(), state.data_ptr(), state.shape[1], int(prev_off),
          slot_ids.data_ptr(), seq_of_token.data_ptr(), cu_q.data_ptr(), positions.data_ptr(), out.data_ptr(),
          width, M, int(n_seqs), state.shape[0], n, _stream()), "wkv_mix")


def tanh_cast(x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = tanh(x)`` for fp32 ``x``, rounded once to ``out``'s type."""
    _check(x, "x", F32)
    _check(out, "out", None, tuple(x.shape))
    f = _fn("wkv", "kvf_wkv_tanh", [c_int, c_void_p, c_void_p, c_long, c_void_p])
    _ok(f(_tcode(out.dtype), x.data_ptr(), out.data_ptr(), x.numel(), _stream()), "tanh_cast")


# Runs of at least WKV_MULTI_FROM tokens are cut into chunks of WKV_CHUNK tokens that go side by
# side (three passes); shorter runs go token by token in one workgroup per head.
WKV_CHUNK = 16
WKV_MULTI_FROM = 64


def wkv_multi_plan(q_lens, multi_from: int = WKV_MULTI_FROM) -> tuple[list[int], list[int]]:
    """For the runs of at least ``multi_from`` tokens among ``q_lens`` (a step's runs in sequence
    order): the flat rows ``(sequence, first token, tokens, 0)`` of their chunks and
    ``(sequence, first chunk, chunks)`` of the runs, as ``wkv_scan(multi=...)`` wants them."""
    chunks: list[int] = []
    runs: list[int] = []
    start = 0
    for seq, q in enumerate(q_lens):
        if q >= multi_from:
            first = len(chunks) // 4
            for t in range(0, q, WKV_CHUNK):
                chunks += [seq, start + t, min(WKV_CHUNK, q - t), 0]
            runs += [seq, first, len(chunks) // 4 - first]
        start += q
    return chunks, runs


def wkv_multi_scratch(n_chunks: int, heads: int, dim: int) -> dict[str, tuple]:
    """(shape, dtype) of the scratch tensors the passes over all chunks need, by name."""
    return {"G": ((n_chunks, int(heads), int(dim), int(dim)), F32), "D": ((n_chunks, int(heads), int(dim)), F32)}


def wkv_scan(rows: torch.Tensor, r_off: int, k_off: int, v_off: int, z: torch.Tensor, w0: torch.Tensor,
             u: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor,
             state: torch.Tensor, out: torch.Tensor, n_seqs: int, heads: int, dim: int,
             multi: dict | None = None, short_runs: bool = True) -> None:
    """The recurrence ``o_j = sum_i r_i (S_ij + u_i k_i v_j)``, ``S_ij <- w_i S_ij + k_i v_j`` with
    ``w = exp(-exp(z + w0))`` over every query run, in fp32, from and to the sequences' state
    slots (a run at position 0 starts from zeros whatever its slot holds; a sequence without a
    slot starts from zeros and keeps nothing).  ``rows``: r, k, v of a token ``[heads * dim]``
    each at the given offsets of its row; ``z`` fp32 ``[n, >= heads * dim]``; ``w0``, ``u`` fp32
    ``[heads * dim]``; ``out`` fp32 ``[n, heads * dim]``.  ``multi``: ``chunks`` and ``runs``
    (int32 device tensors of ``wkv_multi_plan``'s rows) and the scratch ``G``, ``D``: those runs
    go chunk by chunk side by side and the token-by-token kernel leaves them alone; it is not
    launched at all with ``short_runs=False`` (the caller knows that no other run is there)."""
    n = rows.shape[0]
    H, dk = int(heads), int(dim)
    _check(rows, "rows", None, (n, None))
    if max(r_off, k_off, v_off) + H * dk > rows.shape[1] or min(r_off, k_off, v_off) < 0:
        raise KernelError("wkv_scan: r, k, v do not fit the rows")
    _check(z, "z", F32, (n, None))
    if z.shape[1] < H * dk:
        raise KernelError("wkv_scan: decay rows too short")
    _check(w0, "w0", F32, (H * dk,))
    _check(u, "u", F32, (H * dk,))
    _check(out, "out", F32, (n, H * dk))
    _check(state, "state", F32, (None, None))
    if state.shape[1] < H * dk * dk or not 0 < dk <= 256:
        raise KernelError(f"wkv_scan: heads of {dk} (at most 256) need slots of {H * dk * dk} floats")
    for t, name in ((cu_q, "cu_q"), (positions, "positions"), (slot_ids, "slot_ids")):
        _check(t, name, I32, (None,))
    if cu_q.shape[0] < n_seqs + 1 or slot_ids.shape[0] < n_seqs or positions.shape[0] < n:
        raise KernelError("wkv_scan: batch arrays shorter than the batch")
    common = (_tcode(rows.dtype), rows.data_ptr(), z.data_ptr(), w0.data_ptr(), u.data_ptr(), cu_q.data_ptr(),
              positions.data_ptr(), slot_ids.data_ptr(), state.data_ptr(), out.data_ptr())
    shape = (int(n_seqs), H, dk, state.shape[0], state.shape[1], rows.shape[1], int(r_off), int(k_off), int(v_off),
             z.shape[1])
    if short_runs or multi is None:
        f = _fn("wkv", "kvf_wkv_scan", [c_int] + [c_void_p] * 9 + [c_int] * 11 + [c_void_p])
        _ok(f(*common, *shape, WKV_MULTI_FROM if multi is not None else 0, _stream()), "wkv_scan")
    if multi is None:
        return
    chunks, runs, G, D = multi["chunks"], multi["runs"], multi["G"], multi["D"]
    _check(chunks, "chunks", I32, (None, 4))
    _check(runs, "runs", I32, (None, 3))
    nc = chunks.shape[0]
    _check(G, "G", F32, (None, H, dk, dk))
    _check(D, "D", F32, (None, H, dk))
    if G.shape[0] < nc or D.shape[0] < nc:
        raise KernelError("wkv_scan: scratch for fewer chunks than the plan has")
    f = _fn("wkv", "kvf_wkv_chunks", [c_int] + [c_void_p] * 10 + [c_int, c_void_p, c_int, c_void_p, c_void_p]
            + [c_int] * 10 + [c_void_p])
    _ok(f(*common, chunks.data_ptr(), nc, runs.data_ptr(), runs.shape[0], G.data_ptr(), D.data_ptr(), *shape,
          _stream()), "wkv_chunks")


def wkv_out(heads_raw: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float,
            out: torch.Tensor, heads: int, dim: int) -> None:
    """``out[n, h, :] = o / rms(o) * weight[h, :] * silu(gate[n, h, :])`` for the raw heads
    ``o = heads_raw[n, h, :]`` (fp32), the root mean square per head with ``eps`` inside the
    root.  ``gate``: dense rows of ``out``'s type (a view of wider rows is fine)."""
    n = heads_raw.shape[0]
    H, dk = int(heads), int(dim)
    _check(heads_raw, "heads_raw", F32, (n, H * dk))
    _check(weight, "weight", F32, (H * dk,))
    _check(out, "out", None, (n, H * dk))
    _check(gate, "gate", out.dtype, (n, H * dk), contiguous=False)
    if gate.stride(1) != 1:
        raise KernelError("wkv_out: gate rows must be dense")
    f = _fn("wkv", "kvf_wkv_out", [c_int, c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p] + [c_int] * 3 + [c_void_p])
    _ok(f(_tcode(out.dtype), heads_raw.data_ptr(), gate.data_ptr(), gate.stride(0) if n > 1 else H * dk,
          weight.data_ptr(), float(eps), out.data_ptr(), n, H, dk, _stream()), "wkv_out")


# ------------------------------------------------------------------------------ routed experts
MOE_MAX_ROUTER_OUTPUTS = 512
MOE_MAX_TOP = 16


def moe_topk(logits: torch.Tensor, correction: torch.Tensor, chosen: torch.Tensor,
             weights: torch.Tensor) -> None:
    """The router's choice per token from its fp32 ``logits [N, R]``: ``s = softmax(logits)``, the
    ``top`` outputs with the largest ``s + correction`` (the lowest index among equals) go to
    ``chosen [N, top]`` (int32) and their ``s``, divided by the sum of the chosen ``s`` (+ 1e-20),
    to ``weights [N, top]`` (fp32)."""
    n, R = logits.shape
    _check(logits, "logits", F32, (n, R), contiguous=False)
    if logits.stride(1) != 1:
        raise KernelError("moe_topk: logits rows must be dense")
    _check(correction, "correction", F32, (R,))
    top = chosen.shape[1]
    _check(chosen, "chosen", I32, (n, top))
    _check(weights, "weights", F32, (n, top))
    if R > MOE_MAX_ROUTER_OUTPUTS or not 0 < top <= min(MOE_MAX_TOP, R):
        raise KernelError(f"moe_topk: up to {MOE_MAX_ROUTER_OUTPUTS} router outputs and {MOE_MAX_TOP} choices, got {R} / {top}")
    f = _fn("moe", "kvf_moe_topk", [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p])
    _ok(f(logits.data_ptr(), logits.stride(0) if n > 1 else R, correction.data_ptr(), chosen.data_ptr(),
          weights.data_ptr(), n, R, top, _stream()), "moe_topk")


def moe_dense_act(gate_up: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor, out: torch.Tensor,
                  experts: int, ff: int) -> None:
    """``gate_up [N, 2 experts ff]`` holds every expert's (gate, up) pairs as neighbouring columns;
    ``out[n, e ff + j] = weight(n, e) * silu(gate) * up`` where token ``n`` chose expert ``e`` and an
    exact zero elsewhere."""
    n = gate_up.shape[0]
    E, top = int(experts), chosen.shape[1]
    _check(gate_up, "gate_up", None, (n, 2 * E * ff))
    _check(out, "out", gate_up.dtype, (n, E * ff))
    _check(chosen, "chosen", I32, (n, top))
    _check(weights, "weights", F32, (n, top))
    f = _fn("moe", "kvf_moe_dense_act", [c_int] + [c_void_p] * 4 + [c_int] * 4 + [c_void_p])
    _ok(f(_tcode(gate_up.dtype), gate_up.data_ptr(), chosen.data_ptr(), weights.data_ptr(), out.data_ptr(),
          n, E, int(ff), top, _stream()), "moe_dense_act")


def moe_identity(x: torch.Tensor, h: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
                 first: int) -> None:
    """``x[n] += w * h[n]`` with ``w`` the sum of the weights of token ``n``'s choices that are
    ``>= first`` (router outputs that pass the input on); ``x`` is the fp32 stream."""
    n, width = x.shape
    _check(x, "x", F32, (n, width))
    _check(h, "h", None, (n, width))
    top = chosen.shape[1]
    _check(chosen, "chosen", I32, (n, top))
    _check(weights, "weights", F32, (n, top))
    f = _fn("moe", "kvf_moe_identity", [c_int] + [c_void_p] * 4 + [c_int] * 4 + [c_void_p])
    _ok(f(_tcode(h.dtype), x.data_ptr(), h.data_ptr(), chosen.data_ptr(), weights.data_ptr(), n, width,
          top, int(first), _stream()), "moe_identity")


def moe_grouped_takes(x: torch.Tensor, w_gate_up, w_down, experts: int, ff: int) -> bool:
    """Whether ``moe_grouped`` takes these operands: bf16 rows that start on 16 bytes, both
    weights kept in tiles, a width that is a multiple of 8 and experts whose width is a
    multiple of 32."""
    n, k = x.shape
    return (x.dtype == BF16 and isinstance(w_gate_up, StreamedWeight) and isinstance(w_down, StreamedWeight)
            and _rows_aligned(x, k, x.stride(0) if n > 1 else k) and ff % 32 == 0 and 0 < experts <= 512)


def moe_grouped_tiles(rows: int, top: int, experts: int) -> int:
    """Tiles of 16 rows that the (token, choice) pairs of ``rows`` tokens can make at most."""
    return -(-rows * top // 16) + experts


def moe_grouped(x: torch.Tensor, w_gate_up: "StreamedWeight", w_down: "StreamedWeight", chosen: torch.Tensor,
                weights: torch.Tensor, residual: torch.Tensor, experts: int, ff: int,
                scratch: dict[str, torch.Tensor]) -> None:
    """``residual[n] += sum_k weights[n, k] * expert_{chosen[n, k]}(x[n])`` (a choice ``>= experts``
    stands for ``x[n]`` itself) with every expert's products taken over only the rows that chose
    it: the pairs are grouped by expert on the device, tiles of 16 rows go through the
    matrix cores against the expert's tiles of ``w_gate_up`` (``[experts * 2 ff, K]``, gate and
    up rows interleaved) and ``w_down`` (``[K, experts * ff]``), an expert's output row is stored
    in bf16 and the weighted sum over a token's choices is taken in fp32 in their order.
    ``scratch``: ``where order [n top]``, ``tiles [3 moe_grouped_tiles]``, ``num_tiles [1]`` (int32),
    ``act [n top, ff]``, ``y [n top, K]`` (bf16)."""
    n, k = x.shape
    top = chosen.shape[1]
    if not moe_grouped_takes(x, w_gate_up, w_down, experts, ff):
        raise KernelError("moe_grouped: operands it does not take (see moe_grouped_takes)")
    if tuple(w_gate_up.shape) != (experts * 2 * ff, k) or tuple(w_down.shape) != (k, experts * ff):
        raise KernelError(f"moe_grouped: weights {list(w_gate_up.shape)} / {list(w_down.shape)} do not fit "
                          f"{experts} experts of width {ff} over rows of {k}")
    _check(chosen, "chosen", I32, (n, top))
    _check(weights, "weights", F32, (n, top))
    _check(residual, "residual", F32, (n, k))
    pairs, max_tiles = n * top, moe_grouped_tiles(n, top, experts)
    for name, dtype, shape in (("where", I32, (pairs,)), ("order", I32, (pairs,)), ("tiles", I32, (3 * max_tiles,)),
                               ("num_tiles", I32, (1,)), ("act", BF16, (pairs, ff)), ("y", BF16, (pairs, k))):
        _check(scratch[name], name, dtype, shape)
    f = _fn("moe", "kvf_moe_grouped", [c_void_p, c_int, c_void_p] + [c_int] * 5 + [c_void_p] * 8 + [c_int]
            + [c_void_p] * 4)
    _ok(f(x.data_ptr(), x.stride(0) if n > 1 else k, x.data_ptr(), n, k, int(experts), int(ff), top,
          w_gate_up.tiles.data_ptr(), w_down.tiles.data_ptr(), chosen.data_ptr(), weights.data_ptr(),
          scratch["where"].data_ptr(), scratch["order"].data_ptr(), scratch["tiles"].data_ptr(),
          scratch["num_tiles"].data_ptr(), max_tiles, scratch["act"].data_ptr(), scratch["y"].data_ptr(),
          residual.data_ptr(), _stream()), "moe_grouped")



def moe_table(tokens: torch.Tensor, table: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
              experts: int) -> None:
    """A choice made by a table: token id ``t`` uses the experts ``table[t]`` (int32
    ``[vocab, top]``), each with weight ``1 / top``; ``chosen [N, top]`` (int32) and
    ``weights [N, top]`` (fp32) as ``moe_topk`` leaves them."""
    n, top = chosen.shape
    _check(tokens, "tokens", I32, (None,))
    if tokens.shape[0] < n:
        raise KernelError("moe_table: fewer token ids than rows")
    _check(table, "table", I32, (None, top))
    _check(chosen, "chosen", I32, (n, top))
    _check(weights, "weights", F32, (n, top))
    if not 0 < top <= MOE_MAX_TOP:
        raise KernelError(f"moe_table: up to {MOE_MAX_TOP} choices, got {top}")
    f = _fn("moe", "kvf_moe_table", [c_void_p] * 4 + [c_int] * 4 + [c_void_p])
    _ok(f(tokens.data_ptr(), table.data_ptr(), chosen.data_ptr(), weights.data_ptr(), n, table.shape[0], top,
          int(experts), _stream()), "moe_table")


# ------------------------------------------------------------------------------ linear-attention memory
# Runs of at least LINMEM_MULTI_FROM tokens are cut into chunks of LINMEM_CHUNK tokens that go side
# by side (three passes); shorter runs go token by token in one workgroup per head and slice.
LINMEM_CHUNK = 16
LINMEM_MULTI_FROM = 64


def linmem_state_floats(heads: int, key_dim: int, value_dim: int) -> int:
    """fp32 numbers of a request's slot: every head's ``S [key_dim, value_dim]``."""
    return int(heads) * int(key_dim) * int(value_dim)


def linmem_multi_plan(q_lens, multi_from: int = LINMEM_MULTI_FROM) -> tuple[list[int], list[int]]:
    """For the runs of at least ``multi_from`` tokens among ``q_lens`` (a step's runs in sequence
    order): the flat rows ``(sequence, first token, tokens, 0)`` of their chunks and
    ``(sequence, first chunk, chunks)`` of the runs, as ``linmem_scan(multi=...)`` wants them."""
    chunks: list[int] = []
    runs: list[int] = []
    start = 0
    for seq, q in enumerate(q_lens):
        if q >= multi_from:
            first = len(chunks) // 4
            for t in range(0, q, LINMEM_CHUNK):
                chunks += [seq, start + t, min(LINMEM_CHUNK, q - t), 0]
            runs += [seq, first, len(chunks) // 4 - first]
        start += q
    return chunks, runs


def linmem_multi_scratch(n_chunks: int, heads: int, key_dim: int, value_dim: int) -> dict[str, tuple]:
    """(shape, dtype) of the scratch tensors the passes over all chunks need, by name."""
    return {"G": ((n_chunks, int(heads), int(key_dim), int(value_dim)), F32),
            "D": ((n_chunks, int(heads), int(key_dim)), F32)}


def linmem_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor,
                cu_q: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor, state: torch.Tensor,
                out: torch.Tensor, n_seqs: int, heads: int, key_dim: int, value_dim: int,
                gate_bias: torch.Tensor | None = None, tau: float | None = None, q_scale: float = 1.0,
                k_scale: float = 1.0, multi: dict | None = None, short_runs: bool = True,
                cos: torch.Tensor | None = None, sin: torch.Tensor | None = None) -> None:
    """The recurrence ``S_ij <- a_i S_ij + k_i v_j``, ``o_j = sum_i q_i S_ij`` (the output sees
    its own token) over every query run, in fp32, from and to the sequences' state slots (a run
    at position 0 starts from zeros whatever its slot holds; a sequence without a slot starts
    from zeros and keeps nothing).  ``q, k [n, heads * key_dim]`` and ``v [n, heads * value_dim]``
    are dense rows (views of wider rows are fine).  With ``cos`` / ``sin`` (fp32 tables by
    position) the first elements of every q and k head are rotated in neighbouring pairs first, in
    fp32; then q and k are multiplied by ``q_scale`` / ``k_scale`` in fp32.  The decays: with ``tau`` given, ``decay`` is fp32 ``[n, >= heads *
    key_dim]`` pre-activations and ``a = sigmoid(decay + gate_bias)^(1/tau)``; otherwise
    ``decay`` is fp32 ``[heads * key_dim]``, constants.  ``out`` fp32 ``[n, heads * value_dim]``.
    ``multi``: ``chunks`` and ``runs`` (int32 device tensors of ``linmem_multi_plan``'s rows) and
    the scratch ``G``, ``D``: those runs go chunk by chunk side by side and the token-by-token
    kernel leaves them alone; it is not launched at all with ``short_runs=False``."""
    n = q.shape[0]
    H, dk, dv = int(heads), int(key_dim), int(value_dim)
    for t, name, w in ((q, "q", H * dk), (k, "k", H * dk), (v, "v", H * dv)):
        _check(t, name, q.dtype, (n, w), contiguous=False)
        if t.stride(1) != 1:
            raise KernelError(f"linmem_scan: rows of {name} must be dense")
    gated = tau is not None
    if gated:
        _check(decay, "decay", F32, (n, None), contiguous=False)
        if decay.shape[1] < H * dk or decay.stride(1) != 1 or not tau > 0:
            raise KernelError("linmem_scan: gate rows too short, not dense, or tau not positive")
        if gate_bias is not None:
            _check(gate_bias, "gate_bias", F32, (H * dk,))
    else:
        _check(decay, "decay", F32, (H * dk,))
        if gate_bias is not None:
            raise KernelError("linmem_scan: a gate bias goes with gates (tau)")
    _check(out, "out", F32, (n, H * dv))
    _check(state, "state", F32, (None, None))
    if state.shape[1] < H * dk * dv or not 0 < dk <= 256 or dv <= 0:
        raise KernelError(f"linmem_scan: heads of {dk} x {dv} (key size at most 256) need slots of {H * dk * dv} floats")
    for t, name in ((cu_q, "cu_q"), (positions, "positions"), (slot_ids, "slot_ids")):
        _check(t, name, I32, (None,))
    if cu_q.shape[0] < n_seqs + 1 or slot_ids.shape[0] < n_seqs or positions.shape[0] < n:
        raise KernelError("linmem_scan: batch arrays shorter than the batch")
    stride = lambda t, w: t.stride(0) if n > 1 else w  # noqa: E731
    cos_p, sin_p, rot, table_len = _rotary_tables(cos, sin, dk, "linmem_scan")
    common = (_tcode(q.dtype), q.data_ptr(), k.data_ptr(), v.data_ptr(), decay.data_ptr(),
              gate_bias.data_ptr() if gate_bias is not None else None, cos_p, sin_p, rot, table_len,
              cu_q.data_ptr(), positions.data_ptr(),
              slot_ids.data_ptr(), state.data_ptr(), out.data_ptr(), int(n_seqs), H, dk, dv, state.shape[0],
              state.shape[1], stride(q, H * dk), stride(k, H * dk), stride(v, H * dv), 1 if gated else 0,
              (decay.stride(0) if n > 1 else decay.shape[1]) if gated else 0,
              1.0 / float(tau) if gated else 1.0, float(q_scale), float(k_scale))
    types = [c_int] + [c_void_p] * 7 + [c_int] * 2 + [c_void_p] * 5 + [c_int] * 11 + [c_float] * 3
    if short_runs or multi is None:
        f = _fn("linmem", "kvf_linmem_scan", types + [c_int, c_void_p])
        _ok(f(*common, LINMEM_MULTI_FROM if multi is not None else 0, _stream()), "linmem_scan")
    if multi is None:
        return
    chunks, runs, G, D = multi["chunks"], multi["runs"], multi["G"], multi["D"]
    _check(chunks, "chunks", I32, (None, 4))
    _check(runs, "runs", I32, (None, 3))
    nc = chunks.shape[0]
    _check(G, "G", F32, (None, H, dk, dv))
    _check(D, "D", F32, (None, H, dk))
    if G.shape[0] < nc or D.shape[0] < nc:
        raise KernelError("linmem_scan: scratch for fewer chunks than the plan has")
    f = _fn("linmem", "kvf_linmem_chunks", types + [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p])
    _ok(f(*common, chunks.data_ptr(), nc, runs.data_ptr(), runs.shape[0], G.data_ptr(), D.data_ptr(), _stream()),
        "linmem_chunks")


def linmem_out(heads_raw: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor | None, eps: float,
               out: torch.Tensor, heads: int, value_dim: int, scale: float = 1.0) -> None:
    """``out[n, h, :] = o / rms(o) * weight * silu(gate[n, h, :]) * scale`` for the raw heads
    ``o = heads_raw[n, h, :]`` (fp32), the root mean square per head with ``eps`` inside the
    root; ``weight`` fp32 ``[value_dim]`` shared by the heads, or ``None`` for none.  ``gate``:
    dense rows of ``out``'s type (a view of wider rows is fine)."""
    n = heads_raw.shape[0]
    H, dv = int(heads), int(value_dim)
    _check(heads_raw, "heads_raw", F32, (n, H * dv))
    if weight is not None:
        _check(weight, "weight", F32, (dv,))
    _check(out, "out", None, (n, H * dv))
    _check(gate, "gate", out.dtype, (n, H * dv), contiguous=False)
    if gate.stride(1) != 1:
        raise KernelError("linmem_out: gate rows must be dense")
    f = _fn("linmem", "kvf_linmem_out", [c_int, c_void_p, c_void_p, c_int, c_void_p, c_float, c_float, c_void_p]
            + [c_int] * 3 + [c_void_p])
    _ok(f(_tcode(out.dtype), heads_raw.data_ptr(), gate.data_ptr(), gate.stride(0) if n > 1 else H * dv,
          weight.data_ptr() if weight is not None else None, float(eps), float(scale), out.data_ptr(), n, H, dv,
          _stream()), "linmem_out")


# ------------------------------------------------------------------------------ sampling
GREEDY_SPLIT_MAX = 16


def sample_work_size(rows: int) -> int:
    """int32 elements of the ``work`` tensor that lets ``sample`` read greedy rows with several
    workgroups each: tickets, then the best value and index of every chunk."""
    return rows * (1 + 2 * GREEDY_SPLIT_MAX)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor | None,
           top_p: torch.Tensor | None, u: torch.Tensor, tokens: torch.Tensor,
           u_step: torch.Tensor | None = None, work: torch.Tensor | None = None) -> None:
    """One token per row of fp32 ``logits``: argmax where ``temperature == 0``, otherwise the
    inverse CDF of the processed distribution at ``u``.  With ``u_step`` (one int32 on the
    device) ``u`` holds several rows of numbers, ``[steps, row stride]``, and row ``u_step[0]``
    is used: a captured launch then serves several decode steps.  ``work`` (int32,
    ``sample_work_size(rows)`` elements, zero when first handed over, not shared with a launch
    that may overlap): greedy rows are then read by several workgroups each, about as many as
    fill the chip; the result is the same."""
    _check(logits, "logits", F32, (None, None), contiguous=False)
    if logits.stride(1) != 1:
        raise KernelError("sample: logits rows must be dense")
    r, v = logits.shape
    _check(temperature, "temperature", F32, (r,))
    stride = 0
    if u_step is None:
        _check(u, "u", F32, (r,))
    else:
        _check(u_step, "u_step", I32, (1,))
        _check(u, "u", F32, (None, None))
        stride = u.shape[1]
        if stride < r:
            raise KernelError("sample: rows of u are shorter than the batch")
    _check(tokens, "tokens", I32, (r,))
    if top_k is not None:
        _check(top_k, "top_k", I32, (r,))
    if top_p is not None:
        _check(top_p, "top_p", F32, (r,))
    splits = 1
    if work is not None:
        _check(work, "work", I32, (None,))
        if work.shape[0] < sample_work_size(r):
            raise KernelError("sample: work is smaller than sample_work_size(rows)")
        # about one workgroup per compute unit, each with at least 4096 logits
        splits = max(1, min(GREEDY_SPLIT_MAX, compute_units(logits.device) // r, v // 4096))
    f = _fn("sampling", "kvf_sample",
            [c_void_p, c_int, c_int, c_int] + [c_void_p] * 5 + [c_int, c_void_p, c_void_p, c_int,
                                                                c_void_p])
    _ok(f(logits.data_ptr(), logits.stride(0) if r > 1 else v, r, v, temperature.data_ptr(),
          top_k.data_ptr() if top_k is not None else None,
          top_p.data_ptr() if top_p is not None else None, u.data_ptr(),
          u_step.data_ptr() if u_step is not None else None, stride, tokens.data_ptr(),
          work.data_ptr() if work is not None else None, splits, _stream()), "sample")


def decode_advance(sampled: torch.Tensor, token_ids: torch.Tensor, positions: torch.Tensor,
                   ctx_lens: torch.Tensor, ring: torch.Tensor, counter: torch.Tensor) -> None:
    """After a step of single tokens: ``ring[counter[0]] = sampled``; for every sequence with a
    context, the sampled token becomes the next input (``token_ids``), ``positions`` and
    ``ctx_lens`` move on by one; ``counter[0] += 1``.  All on the device, in stream order."""
    r = sampled.shape[0]
    for t, name in ((sampled, "sampled"), (token_ids, "token_ids"), (positions, "positions"),
                    (ctx_lens, "ctx_lens")):
        _check(t, name, I32, (r,))
    _check(ring, "ring", I32, (None, None))
    _check(counter, "counter", I32, (1,))
    if ring.shape[1] < r:
        raise KernelError("decode_advance: rows of the ring are shorter than the batch")
    f = _fn("sampling", "kvf_decode_advance", [c_void_p] * 6 + [c_int] * 3 + [c_void_p])
    _ok(f(sampled.data_ptr(), token_ids.data_ptr(), positions.data_ptr(), ctx_lens.data_ptr(),
          ring.data_ptr(), counter.data_ptr(), r, ring.shape[1], ring.shape[0], _stream()),
        "decode_advance")
