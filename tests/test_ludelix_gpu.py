"""Ludelix on the GPU: each mechanism's kernels alone against the plain functions, then whole
models (other sizes in every test than anywhere else) through the engine's runner, cache and
state slots: whole prompts, the stream after every layer, token-by-token decoding, portions down
to two tokens, unequal requests in one batch, pages and slots that come back, marked keys on
either side of a window's and a chunk's edge, a memory that carries a token for hundreds of
steps, a sink that takes the weight, models drawn at random, and greedy generation through the
engine and its scheduler."""

from __future__ import annotations

import math
import os
import random

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import kvforge_amd
from kvforge_amd.config.presets import ludelix as make_config
from kvforge_amd.engine.batch import StepEntry
from tests import replay_util as ru
from tests.plain import ludelix as plain
from tests.test_fogorax_gpu import in_portions, make_runner, prompts_for, replay, replay_all
from tests.test_kernels_gpu import Paged, prefill_work
from tests.test_rudorax_gpu import close_to_truth, jittered

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]
NAME = {torch.float32: "float32", torch.bfloat16: "bfloat16"}


def ops():
    from kvforge_amd.kernels import ops as o
    return o


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


# ======================================================================= mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("v_from_k", [True, False])
@pytest.mark.parametrize("H,KV,dk,d,rot", [(4, 2, 16, 16, 8), (3, 1, 24, 32, 24), (8, 1, 64, 64, 0), (5, 5, 6, 16, 2),
                                           (2, 1, 256, 256, 64), (6, 3, 40, 48, 12)])
def test_biases_a_norm_over_whole_rows_rotation_and_values_that_are_keys(dtype, v_from_k, H, KV, dk, d, rot):
    """q and k get their biases, each is divided by the root mean square of the *whole* row (all
    heads at once) and weighted element by element, the first ``rot`` elements of every head are
    rotated in neighbouring pairs; the values that reach the pages are the keys before norm and
    rotation, or columns of their own."""
    n, bs, eps = 10, 8, 1e-4
    heads = H + KV + (0 if v_from_k else KV)
    proj = rand(n, heads * d + 5, seed=dk, scale=1.5)
    view = proj[:, :heads * d].view(n, heads, d)
    view[:, :H + KV, dk:] = 0.0
    pos = torch.tensor([0, 1, 2, 3, 5, 6, 7, 13, 62, 63], dtype=torch.int32)
    qw, kw = 1.0 + rand(H * dk, seed=1, scale=0.2), 1.0 + rand(KV * dk, seed=2, scale=0.2)
    qb, kb = rand(H * dk, seed=3, scale=0.7), rand(KV * dk, seed=4, scale=0.7)
    table = i32([[7, 2, 5, 0, 3, 1, 6, 4]])
    kp = torch.full((8, KV, bs, d), 9.0, dtype=dtype, device=DEV)
    vp = torch.full((8, KV, d, bs), 9.0, dtype=dtype, device=DEV)
    q_out = torch.full((n, H * d), 9.0, dtype=dtype, device=DEV)
    f = plain.plain_frequencies(rot, 100.0) if rot else None
    cos = sin = None
    if rot:
        ang = torch.arange(64, dtype=torch.float32)[:, None] * f.float()[None, :]
        cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    ops().rownorm_rope_kvwrite(proj.to(DEV), q_out, pos.to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
                               cos, sin, table, kp, vp, H, KV, d, qw.to(DEV), kw.to(DEV), dk, eps,
                               q_bias=qb.to(DEV), k_bias=kb.to(DEV), values_are_keys=v_from_k)
    q = view[:, :H, :dk].reshape(n, H * dk) + qb
    k = view[:, H:H + KV, :dk].reshape(n, KV * dk) + kb
    v = k.view(n, KV, dk) if v_from_k else view[:, H + KV:, :]
    qn, kn = plain.norm(q, qw, eps).view(n, H, dk), plain.norm(k, kw, eps).view(n, KV, dk)
    if rot:
        qn, kn = plain.turn(qn, pos, f, 1.0, True), plain.turn(kn, pos, f, 1.0, True)
    got = q_out.float().cpu().view(n, H, d)
    torch.testing.assert_close(got[..., :dk], qn, **tol(dtype))
    assert float(got[..., dk:].abs().max() if d > dk else 0.0) == 0.0
    for t, p in enumerate(pos.tolist()):
        page, off = int(table[0, p // bs]), p % bs
        torch.testing.assert_close(kp[page, :, off, :dk].float().cpu(), kn[t], **tol(dtype))
        torch.testing.assert_close(vp[page, :, :v.shape[2], off].float().cpu(), v[t], **tol(dtype))


def chunk_reference(paged, q, seq_lens, q_lens, scale, chunk, window, sink, G):
    outs, off = [], 0
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        k = paged.keys[s].float()
        v = paged.values[s].float()
        mask = plain.chunk_mask(n, chunk) if chunk else plain.window_mask(n, window or n)
        outs.append(plain.softmax_attention(q[off:off + ql].float(), k, v, scale, mask[n - ql:], sink))
        off += ql
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (8, 1, 64, 16), (3, 1, 48, 8), (6, 2, 128, 16), (4, 4, 64, 16)])
@pytest.mark.parametrize("chunk", [1, 7, 32, 50, 1000])
def test_attention_within_chunks_of_positions(dtype, H, KV, d, bs, chunk):
    """Query runs and single tokens (one cut and several): a query sees the keys of its own chunk
    alone, chunks counted from position 0 whatever the run's first position is."""
    scale = 1 / math.sqrt(d)
    for seq_lens, q_lens in (([90, 33, 70, 5], [40, 33, 2, 5]), ([7, 90, 1, 300, 50, 51], [1, 1, 1, 1, 1, 1])):
        paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + chunk)
        n = sum(q_lens)
        buf = rand(n, H * d, seed=d + 1, scale=1.5).to(dtype)
        cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
        ctx = torch.tensor(seq_lens, dtype=torch.int32)
        want = chunk_reference(paged, buf.view(n, H, d), seq_lens, q_lens, scale, chunk, None, None, H // KV)
        want = want.reshape(n, H * d)
        if chunk < 50:
            free = chunk_reference(paged, buf.view(n, H, d), seq_lens, q_lens, scale, None, None, None, H // KV)
            assert float((want - free.reshape(n, H * d)).abs().max()) > 0.05       # the chunks matter here
        args = (buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV))
        if max(q_lens) > 1:
            out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
            ops().attn_prefill(*args, cu.to(DEV), ctx.to(DEV), prefill_work(q_lens, H // KV, dtype, d, bs).to(DEV),
                               out, H, KV, d, scale, 0, chunk=chunk)
            torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
            continue
        for splits in (1, 3):
            out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
            ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV))
            ops().attn_decode(*args, None, n, cu.to(DEV), ctx.to(DEV), out, H, KV, d, scale, 0, splits, ws,
                              chunk=chunk)
            torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


def test_a_window_and_chunks_exclude_each_other():
    paged = Paged([8], 1, 16, 4, torch.float32)
    q = torch.zeros(1, 16, device=DEV)
    with pytest.raises(ops().KernelError):
        ops().attn_decode(q, paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, 1, i32([0, 1]), i32([8]),
                          torch.zeros_like(q), 1, 1, 16, 1.0, 4, chunk=4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d", [(1, 16), (5, 24), (8, 64), (3, 10), (2, 36)])
def test_one_gate_per_head_and_a_constant(dtype, H, d):
    y = rand(9, H * d + 8, seed=H).to(dtype)
    g = rand(9, 16, seed=d, scale=2.0)
    dev = y.clone().to(DEV)
    ops().head_gate(dev[:, :H * d], g.to(DEV), H, d, 1.2)
    want = y.float()[:, :H * d].view(9, H, d) * torch.sigmoid(g[:, :H])[:, :, None] * 1.2
    torch.testing.assert_close(dev.float().cpu()[:, :H * d], want.reshape(9, H * d), **tol(dtype))
    torch.testing.assert_close(dev.cpu()[:, H * d:], y[:, H * d:], atol=0, rtol=0)
    ops().head_gate(dev[:, :H * d], None, H, d, 0.5)
    torch.testing.assert_close(dev.float().cpu()[:, :H * d], want.reshape(9, H * d) * 0.5, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_squared_relu_and_a_gate_per_row(dtype):
    x = rand(7, 50, seed=1, scale=2.0).to(dtype)
    dev = x.clone().to(DEV)
    ops().plain_act(dev, dev, "relu2")
    torch.testing.assert_close(dev.float().cpu(), torch.relu(x.float()) ** 2, **tol(dtype))
    for inter in (30, 32, 1024):              # one pair a thread, and four
        gu, rg = rand(7, 2 * inter, seed=2).to(dtype), rand(7, 16, seed=3, scale=2.0)
        out = torch.zeros(7, inter, dtype=dtype, device=DEV)
        ops().gated_act_rowgate(gu.to(DEV), rg.to(DEV), out, "silu")
        g, u = gu.float()[:, 0::2], gu.float()[:, 1::2]
        want = torch.nn.functional.silu(g) * u * torch.sigmoid(rg[:, :1])
        torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    wide = rand(5, 4096, seed=4, scale=2.0).to(dtype).to(DEV)      # eight elements a thread
    into = torch.zeros_like(wide)
    ops().plain_act(wide, into, "relu2")
    torch.testing.assert_close(into.float().cpu(), torch.relu(wide.float().cpu()) ** 2, **tol(dtype))


def test_a_table_chooses_the_experts():
    table = torch.tensor([[3, 1], [0, 2], [5, 4], [1, 0], [9, 2]], dtype=torch.int32)     # 9 names no expert
    tokens = i32([2, 0, 4, 7, 1, 3])                                                    # 7 lies outside the table
    chosen = torch.full((6, 2), -5, dtype=torch.int32, device=DEV)
    weights = torch.full((6, 2), -5.0, device=DEV)
    ops().moe_table(tokens, table.to(DEV), chosen, weights, 6)
    assert chosen.cpu().tolist() == [[5, 4], [3, 1], [0, 2], [0, 0], [0, 2], [1, 0]]
    assert weights.cpu().tolist() == [[0.5, 0.5], [0.5, 0.5], [0.0, 0.5], [0.0, 0.0], [0.5, 0.5], [0.5, 0.5]]


def run_memory(dtype, q, k, v, a, runs, state, slots, positions, H, dk, dv, **kw):
    """The kernels over the runs of one step.  ``a``: gates' pre-activations ``[n, H * dk]`` (with
    ``tau`` among ``kw``) or constants ``[H * dk]``."""
    o = ops()
    n = q.shape[0]
    rows = torch.cat([q, k, v], dim=1).to(dtype).to(DEV)
    Q = H * dk
    cu = i32([0] + list(np.cumsum(runs)))
    chunks, rr = o.linmem_multi_plan(runs)
    multi = None
    if chunks:
        multi = {"chunks": i32(chunks).view(-1, 4), "runs": i32(rr).view(-1, 3)}
        for name, (shape, dt) in o.linmem_multi_scratch(len(chunks) // 4, H, dk, dv).items():
            multi[name] = torch.full(shape, 7.0, dtype=dt, device=DEV)
    out = torch.full((n, H * dv), 7.0, device=DEV)
    o.linmem_scan(rows[:, :Q], rows[:, Q:2 * Q], rows[:, 2 * Q:], a.to(DEV), cu, i32(positions), i32(slots), state, out,
                  len(runs), H, dk, dv, multi=multi, short_runs=any(r < o.LINMEM_MULTI_FROM for r in runs), **kw)
    return out.cpu()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(2, 16, 16), (3, 24, 40), (1, 64, 128), (2, 100, 72), (1, 256, 64), (4, 8, 200)])
@pytest.mark.parametrize("gated", [True, False])
def test_the_memory_over_runs_steps_and_slots(dtype, H, dk, dv, gated):
    """Three sequences in one step, one token by token, one chunk by chunk (long enough), one a
    single token; then each goes on from what the step left in its slot, the long one token by
    token and the short ones in runs; a slot that held another's memory starts from zeros at
    position 0; a sequence without a slot starts from zeros and keeps nothing."""
    lens = [9, 150, 1]
    more = [70, 3, 20]
    g = torch.Generator().manual_seed(dk + dv)
    total = [a + b for a, b in zip(lens, more)]
    seqs = []
    for n in total:
        q, k = torch.randn(n, H, dk, generator=g), torch.randn(n, H, dk, generator=g) * 0.5
        v = torch.randn(n, H, dv, generator=g)
        z = torch.randn(n, H, dk, generator=g) * 2.0 + 2.0
        if dtype == torch.bfloat16:
            q, k, v = q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float()
        seqs.append((q, k, v, z))
    tau, bias = 4.0, rand(H * dk, seed=5)
    consts = torch.rand(H, generator=g) * 0.1 + 0.9
    def decays(z):
        if gated:
            return torch.exp(torch.nn.functional.logsigmoid(z + bias.view(H, dk)) / tau)
        return consts[:, None]
    want = [plain.decay_scan(q * 0.3, k * 1.7, v, decays(z)) for q, k, v, z in seqs]
    state = torch.full((4, H * dk * dv + 3), 5.0, device=DEV)          # leftovers of others in every slot
    slots = [2, 0, 3]
    kw = dict(q_scale=0.3, k_scale=1.7)
    if gated:
        kw.update(tau=tau, gate_bias=bias.to(DEV))
    def step(parts):
        cat = lambda i: torch.cat([seqs[s][i][a:b].reshape(b - a, -1) for s, a, b in parts])
        a = cat(3) if gated else consts[:, None].expand(H, dk).reshape(-1).contiguous()
        pos = [p for s, lo, hi in parts for p in range(lo, hi)]
        return run_memory(dtype, cat(0), cat(1), cat(2), a, [hi - lo for _, lo, hi in parts], state,
                          [slots[s] for s, _, _ in parts], pos, H, dk, dv, **kw)
    first = step([(s, 0, lens[s]) for s in range(3)])
    off = 0
    for s in range(3):
        torch.testing.assert_close(first[off:off + lens[s]].view(-1, H, dv), want[s][:lens[s]], atol=2e-4, rtol=2e-4)
        off += lens[s]
    second = step([(s, lens[s], total[s]) for s in range(3)])
    off = 0
    for s in range(3):
        torch.testing.assert_close(second[off:off + more[s]].view(-1, H, dv), want[s][lens[s]:], atol=2e-4, rtol=2e-4)
        off += more[s]
    # token by token from the middle of the long one's memory
    again = step([(1, 0, total[1] - 5)])
    torch.testing.assert_close(again.view(-1, H, dv), want[1][:total[1] - 5], atol=2e-4, rtol=2e-4)
    third = torch.cat([step([(1, t, t + 1)]) for t in range(total[1] - 5, total[1])])
    torch.testing.assert_close(third.view(-1, H, dv), want[1][total[1] - 5:], atol=2e-4, rtol=2e-4)
    # without a slot
    slots[0] = -1
    before = state.clone()
    alone = step([(0, 0, 30)])
    torch.testing.assert_close(alone.view(-1, H, dv), want[0][:30], atol=2e-4, rtol=2e-4)
    assert torch.equal(before, state)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_memorys_queries_and_keys_are_rotated_in_32_bit(dtype):
    H, dk, dv, rot, n = 2, 16, 24, 12, 90
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(n, H, d, generator=g).to(dtype).float() for d in (dk, dk, dv))
    f = plain.plain_frequencies(rot, 1000.0)
    ang = torch.arange(256, dtype=torch.float32)[:, None] * f.float()[None, :]
    pos = torch.arange(100, 100 + n)
    a = torch.tensor([0.97, 0.999])
    want = plain.decay_scan(plain.turn(q, pos, f, 1.0, True), plain.turn(k, pos, f, 1.0, True) * 0.25, v, a[:, None])
    state = torch.zeros(1, H * dk * dv, device=DEV)
    got = run_memory(dtype, q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1),
                     a[:, None].expand(H, dk).reshape(-1).contiguous(), [n], state, [-1], pos.tolist(), H, dk, dv,
                     k_scale=0.25, cos=ang.cos().to(DEV), sin=ang.sin().to(DEV))
    torch.testing.assert_close(got.view(n, H, dv), want, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("weight", [True, False])
def test_head_norm_gate_and_constant(dtype, weight):
    H, dv, n = 3, 40, 6
    o, g = rand(n, H * dv, seed=1, scale=3.0), rand(n, H * dv + 8, seed=2).to(dtype)
    o[2] = 0.0
    w = 1.0 + rand(dv, seed=3, scale=0.3) if weight else None
    out = torch.zeros(n, H * dv, dtype=dtype, device=DEV)
    ops().linmem_out(o.to(DEV), g.to(DEV)[:, 8:], w.to(DEV) if weight else None, 1e-3, out, H, dv, 0.5)
    want = plain.rms(o.view(n, H, dv), 1e-3) * (w if weight else 1.0)
    want = want.reshape(n, H * dv) * torch.nn.functional.silu(g.float()[:, 8:]) * 0.5
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


# ======================================================================= whole models
def shape_a():
    """All mixers and both feed-forwards; sizes that no kernel's tiles divide."""
    return make_config(vocab=211, width=72, layers=[
        ("gla", dict(heads=3, dim=24, vdim=40, tau=6.0, rank=5), 100),
        ("attention", dict(heads=6, kv_heads=2, dim=24, scale=0.3, window=21, rot_dims=10, base=5000.0,
                           scaling=(3.0, 1.0, 3.0, 40)), (24, 5, 2, 56)),
        ("parallel", dict(left=dict(heads=4, kv_heads=2, dim=20, vdim=28, scale=0.2, chunk=17, rot_dims=12,
                                    base=2000.0, scaling=(5.0, 50, 8.0, 0.5)),
                          right=dict(heads=3, dim=12, vdim=20, decay=[0.9, 0.97, 0.995], rot_dims=8, base=100.0),
                          left_scale=0.8, right_scale=1.7), (40, 7, 3, 0)),
        ("gla", dict(heads=1, dim=72, vdim=16, tau=2.0, rank=20), None)], eps=1e-5, max_positions=2048)


def shape_b():
    """What a model may make equal or one: one head everywhere, kv heads = heads, one expert
    chosen of one, windows and chunks of one key and longer than any prompt, whole heads rotated
    and none, no scaling, scales of 1, tau 1, a decay of 1 and of 0."""
    return make_config(vocab=64, width=32, layers=[
        ("attention", dict(heads=1, kv_heads=1, dim=16, scale=1.0, window=1, rot_dims=16), (16, 1, 1, 16)),
        ("parallel", dict(left=dict(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.25, chunk=1),
                          right=dict(heads=2, dim=16, vdim=16, decay=[1.0, 0.0]), left_scale=1.0, right_scale=1.0), 32),
        ("gla", dict(heads=1, dim=16, vdim=16, tau=1.0, rank=1), None),
        ("attention", dict(heads=2, kv_heads=2, dim=16, scale=0.25, window=4000), 48),
        ("parallel", dict(left=dict(heads=1, kv_heads=1, dim=32, vdim=16, scale=0.2, chunk=5000, rot_dims=32),
                          right=dict(heads=1, dim=32, vdim=48, decay=[0.99], rot_dims=32), left_scale=2.0,
                          right_scale=0.25), (16, 3, 3, 0))], eps=1e-6, max_positions=512)


def shape_c():
    """Layers wide enough for the kernels that serving a real model takes: heads of 64 on the
    matrix cores, memories wider than a wave's rows, experts on the grouped kernels, a
    feed-forward deep enough for a down projection cut in two halves of K, a vocabulary that ends
    inside a group of 16 columns."""
    return make_config(vocab=1000, width=384, layers=[
        ("attention", dict(heads=6, kv_heads=2, dim=64, scale=0.125, window=50, rot_dims=32, base=100000.0,
                           scaling=(8.0, 1.0, 4.0, 64)), (128, 8, 2, 256)),
        ("gla", dict(heads=3, dim=128, vdim=128, tau=16.0, rank=16), 4096),
        ("parallel", dict(left=dict(heads=6, kv_heads=1, dim=64, vdim=64, scale=0.125, chunk=64, rot_dims=64,
                                    scaling=(8.0, 128, 32.0, 1.0)),
                          right=dict(heads=3, dim=64, vdim=128, decay=[0.97, 0.99, 0.999], rot_dims=64),
                          left_scale=1.2, right_scale=0.5), (64, 8, 1, 128))], eps=1e-5, max_positions=2048)


SHAPE = {"a": shape_a, "b": shape_b, "c": shape_c}


def liven(folder: str) -> None:
    """Random weights of std 0.02 give flat attention and memories that hardly turn.  Scaled so
    that attention is peaked, sinks and gates matter, decays swing with the tokens, and the
    layers outweigh the embedding."""
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        f = 1.0
        if k.endswith(("q.norm", "k.norm")):
            f = 2.0
        elif k.endswith((".q", ".k", ".g")) and ".mix" in k:
            f = 6.0
        elif k.endswith((".v", ".o")) and ".mix" in k:
            f = 5.0
        elif k.endswith((".a1", ".a2")):
            f = 12.0
        elif k.endswith((".down", ".sg")):
            f = 8.0
        elif k.endswith((".up", ".gate")):
            f = 4.0
        if f != 1.0:
            w[k] = (w[k].float() * f).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})


_MODELS: dict = {}


def model_folder(tmp_path_factory, name: str, dtype):
    key = (name, dtype)
    if key not in _MODELS:
        folder = str(tmp_path_factory.mktemp(f"ludelix_{name}_{NAME[dtype]}"))
        cfg = SHAPE[name]()
        kvforge_amd.write_random_model(folder, cfg, seed=len(name) + 17, dtype=NAME[dtype])
        liven(folder)
        _MODELS[key] = (folder, cfg, load_file(os.path.join(folder, "model.safetensors")))
    return _MODELS[key]


_WANT: dict = {}


def plain_logits(cfg, w, toks, dtype):
    """(the truth, plain runs with the roundings of ``dtype``): the plain model in 64-bit, and in
    32-bit (for a 32-bit engine) or in 32-bit with every trip through memory that a bfloat16
    engine may make rounded to bfloat16: as the weights are, and four times with them moved by
    half a bfloat16 step, which shows the rows where the design multiplies rounding (a memory
    head is divided by its own size, so a head whose query all but misses its memory is rounding
    through and through)."""
    key = (id(w), tuple(toks), dtype)
    if key not in _WANT:
        truth = plain.forward(cfg, w, toks, dtype=torch.float64).float()
        if dtype == torch.bfloat16:
            runs = [plain.forward(cfg, w, toks, store=torch.bfloat16)]
            runs += [plain.forward(cfg, jittered(w, s), toks, store=torch.bfloat16) for s in range(1, 5)]
        else:
            runs = [plain.forward(cfg, w, toks)]
        _WANT[key] = (truth, runs)
    return _WANT[key]


def check(got, cfg, w, toks, dtype, what=""):
    truth, plain_runs = plain_logits(cfg, w, toks, dtype)
    close_to_truth(got, truth, plain_runs, dtype, what)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(SHAPE))
def test_whole_prompts_and_their_first_tokens(tmp_path_factory, name, dtype):
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    runner = make_runner(folder, dtype)
    seqs = prompts_for(cfg, [1, 2, 3, 70, 150], 1)
    got = replay(runner, seqs, [[(r, 0, len(t))] for r, t in seqs.items()])
    for r, t in seqs.items():
        check(got[r], cfg, w, t, dtype, f"{name} {r}")
    assert runner.cache.num_free_blocks == 64 and runner.cache.slots.num_free == 4


@pytest.mark.parametrize("name", sorted(SHAPE))
def test_the_stream_after_every_layer(tmp_path_factory, name):
    """In 32-bit, so that a fault names its layer."""
    folder, cfg, w = model_folder(tmp_path_factory, name, torch.float32)
    runner = make_runner(folder, torch.float32)
    toks = prompts_for(cfg, [60], 2)["r0"]
    want, truth = [], []
    plain.forward(cfg, w, toks, layers_out=want)
    plain.forward(cfg, w, toks, dtype=torch.float64, layers_out=truth)
    runner.cache.allocate("x", 0)
    runner.cache.append_slots("x", len(toks), 0)
    step, _ = runner.build_step([StepEntry("x", toks, 0, "all")])
    model = runner.model
    assert len(model.order) == len(want) == len(cfg["layers"])
    with torch.inference_mode():
        residual = model.embed(step)
        for i, (call, ls) in enumerate(zip(model.order, model.layer_states)):
            model.spec.blocks[call.layer].forward(residual, step, ls)
            step.settle()
            own = float((want[i].double() - truth[i]).abs().max())
            torch.testing.assert_close(residual.cpu().double(), truth[i], atol=max(3e-4, 8.0 * own), rtol=3e-4,
                                       msg=lambda m: f"layer {i} ({cfg['layers'][i]['type']}): {m}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(SHAPE))
def test_decoding_token_by_token_equals_the_prompt_read_at_once(tmp_path_factory, name, dtype):
    """From the first token on, and from a prompt's end for 119 tokens, past every window and
    over several chunks' edges."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    runner = make_runner(folder, dtype)
    seqs = prompts_for(cfg, [90, 160], 3)
    plan = [[("r0", i, i + 1)] for i in range(90)]
    plan += [[("r1", 0, 41)]] + [[("r1", i, i + 1)] for i in range(41, 160)]
    got = replay(runner, seqs, plan)
    for r, t in seqs.items():
        check(got[r], cfg, w, t, dtype, f"{name} {r}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(SHAPE))
@pytest.mark.parametrize("sizes", [(2,), (7, 2, 5, 3, 2, 11), (13, 1, 8, 40, 3), (64, 9)])
def test_prompts_in_portions(tmp_path_factory, name, dtype, sizes):
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    runner = make_runner(folder, dtype)
    seqs = prompts_for(cfg, [101], 4)
    got = replay(runner, seqs, in_portions("r0", 101, sizes))
    check(got["r0"], cfg, w, seqs["r0"], dtype, f"{name} {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(SHAPE))
def test_unequal_requests_in_one_batch_against_each_alone(tmp_path_factory, name, dtype):
    """Portions of some requests beside single tokens of others; four slots and so few pages
    that both are used again by later requests; a request left out of a step goes on later."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    seqs = prompts_for(cfg, [83, 40, 7, 120, 33, 58], 5)
    plan = [
        [("r0", 0, 30), ("r1", 0, 1)],
        [("r0", 30, 31), ("r1", 1, 40), ("r2", 0, 2)],
        [("r2", 2, 7), ("r0", 31, 64), ("r3", 0, 50)],
        [("r3", 50, 51), ("r4", 0, 9)],                        # r0 is left out here
        [("r0", 64, 83), ("r3", 51, 52), ("r4", 9, 10), ("r5", 0, 16)],
        [("r3", 52, 118), ("r4", 10, 33), ("r5", 16, 17)],
        [("r3", 118, 119), ("r5", 17, 58)],
        [("r3", 119, 120)],
    ]
    # shape b keeps every key of its wide window and chunk: 83 + 52 + 10 + 16 tokens live at the most
    runner = make_runner(folder, dtype, block_size=8, num_blocks=52, seqs=4)
    together = replay(runner, seqs, plan)
    assert runner.cache.num_free_blocks == 52 and runner.cache.slots.num_free == 4
    for r, t in seqs.items():
        check(together[r], cfg, w, t, dtype, f"{name} {r} in the batch")
        alone = replay(runner, {r: t}, [[(r, 0, len(t))]])[r]
        check(alone, cfg, w, t, dtype, f"{name} {r} alone")
        truth, plain_runs = plain_logits(cfg, w, t, dtype)
        close_to_truth(together[r], alone, [p + (alone - truth) for p in plain_runs], dtype,
                       f"{name} {r} against itself alone")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_a_prompt_of_a_thousand_tokens(tmp_path_factory, name, dtype):
    """Dozens of chunks of the memories side by side, window and chunks over many pages: whole,
    in large and small portions, and its last tokens one by one."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    runner = make_runner(folder, dtype, block_size=16, num_blocks=80, tokens=1200)
    toks = prompts_for(cfg, [1100], 11)["r0"]
    for plan in ([[("r0", 0, 1100)]], in_portions("r0", 1100, (300, 64, 65, 7, 129, 2)),
                 [[("r0", 0, 1050)]] + [[("r0", i, i + 1)] for i in range(1050, 1100)]):
        got = replay(runner, {"r0": toks}, plan)["r0"]
        check(got, cfg, w, toks, dtype, f"{name}, {len(plan)} steps")


def marked_model(tmp_path, dtype, kind, size):
    """A one-layer model in which token 1 is marked: its embedding lies along one axis that no
    other token uses, the keys read that axis, every query has a constant that meets it, the
    values carry it on.  So the marked token's key scores far above all others for every query.
    ``kind``: ``"attention"`` (a window of ``size``, values that are the keys) or ``"parallel"``
    (chunks of ``size`` beside a retention that forgets at once)."""
    V, W = 50, 32
    if kind == "attention":
        layer = ("attention", dict(heads=2, kv_heads=1, dim=16, scale=1.0, window=size), None)
    else:
        layer = ("parallel", dict(left=dict(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, chunk=size),
                                  right=dict(heads=1, dim=16, vdim=16, decay=[0.0]), left_scale=1.0,
                                  right_scale=0.01), None)
    cfg = make_config(vocab=V, width=W, layers=[layer], eps=1e-6, max_positions=1024)
    folder = str(tmp_path / f"m_{kind}")
    kvforge_amd.write_random_model(folder, cfg, seed=5, dtype=NAME[dtype])
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    e = rand(V, W, seed=1, scale=0.3)
    e[:, 0] = 0.0
    e[:, 1] = 1.0                       # a constant every token has: the queries' handle
    e[1] = 0.0
    e[1, 0] = 6.0
    new = {"embed": e, "l0.norm1": torch.ones(W)}
    wq, wk = torch.zeros(32, W), rand(16, W, seed=2, scale=0.05)
    wq[15, 1] = wq[31, 1] = 1.0
    wk[:, 0] = 0.0
    wk[15, 0] = 1.0
    if kind == "attention":
        # the values are the keys: what the marked key carries on is its own element 15
        new.update({"l0.mix.q": wq, "l0.mix.k": wk, "l0.mix.q.norm": torch.full((32,), 1.0),
                    "l0.mix.k.norm": torch.full((16,), 2.0), "l0.mix.q.b": torch.zeros(32),
                    "l0.mix.k.b": torch.zeros(16), "l0.mix.sink": torch.tensor([0.5, -2.0]),
                    "l0.mix.o": rand(W, 32, seed=4, scale=0.5)})
    else:
        wv = rand(16, W, seed=2, scale=0.05)
        wv[:, 0] = rand(16, seed=3, scale=2.0)
        new.update({"l0.mix.left.q": wq * 2.0, "l0.mix.left.k": wk * 2.0, "l0.mix.left.v": wv,
                    "l0.mix.left.o": rand(W, 32, seed=4, scale=0.5), "l0.mix.left.g": rand(2, W, seed=6, scale=0.1)})
    for k, t in new.items():
        assert w[k].shape == t.shape, k
        w[k] = t.to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})
    return folder, cfg, load_file(path)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bs", [8, 16])
def test_one_key_among_hundreds_on_either_side_of_the_window(tmp_path, dtype, bs):
    """The logits follow whether the marked token is just inside the window (a query and the
    ``size - 1`` before it) or just outside, at page borders and in the middle of pages, read
    whole, in portions and token by token."""
    window = 37
    folder, cfg, w = marked_model(tmp_path, dtype, "attention", window)
    runner = make_runner(folder, dtype, block_size=bs, num_blocks=-(-700 // bs), tokens=512)
    g = torch.Generator().manual_seed(bs)
    for at in (0, 7, bs - 1, bs, 3 * bs - 1, 100):
        n = at + window + 1                       # the last position is the first that no longer sees `at`
        toks = (torch.randint(2, 50, (n + 20,), generator=g)).tolist()
        toks[at] = 1
        want = plain.forward(cfg, w, toks)
        blind = plain.forward(cfg, w, [t if i != at else 2 for i, t in enumerate(toks)])
        spread = float(want.std())
        assert float((want[n - 2] - blind[n - 2]).abs().max()) > 0.3 * spread      # seen from the window's last place
        assert float((want[n - 1] - blind[n - 1]).abs().max()) < 1e-4 * spread     # and not from the next
        for plan in ([[("x", 0, len(toks))]], in_portions("x", len(toks), (5, 2, 11)),
                     [[("x", 0, at + 1)]] + [[("x", i, i + 1)] for i in range(at + 1, len(toks))]):
            got = replay(runner, {"x": toks}, plan)["x"]
            check(got, cfg, w, toks, dtype, f"marked at {at}, pages of {bs}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bs", [8, 16])
def test_one_key_among_hundreds_on_either_side_of_a_chunks_edge(tmp_path, dtype, bs):
    """The marked token is seen from every later position of its own chunk and from none of the
    next, whether it is a chunk's first, a middle or its last position; prompts are cut inside
    chunks, at their edges, and read token by token."""
    chunk = 29
    folder, cfg, w = marked_model(tmp_path, dtype, "parallel", chunk)
    runner = make_runner(folder, dtype, block_size=bs, num_blocks=-(-700 // bs), tokens=512)
    g = torch.Generator().manual_seed(bs + 1)
    for at in (0, chunk - 1, chunk, 2 * chunk + 11, 5 * chunk - 2):
        end = (at // chunk + 1) * chunk              # the first position of the next chunk
        toks = (torch.randint(2, 50, (end + 20,), generator=g)).tolist()
        toks[at] = 1
        want = plain.forward(cfg, w, toks)
        blind = plain.forward(cfg, w, [t if i != at else 2 for i, t in enumerate(toks)])
        spread = float(want.std())
        if at < end - 1:
            assert float((want[end - 1] - blind[end - 1]).abs().max()) > 0.3 * spread   # from its chunk's last place
        assert float((want[end] - blind[end]).abs().max()) < 1e-4 * spread               # not from the next chunk
        for plan in ([[("x", 0, len(toks))]], in_portions("x", len(toks), (5, 2, 11)), in_portions("x", len(toks), (chunk,)),
                     [[("x", 0, at + 1)]] + [[("x", i, i + 1)] for i in range(at + 1, len(toks))]):
            got = replay(runner, {"x": toks}, plan)["x"]
            check(got, cfg, w, toks, dtype, f"marked at {at}, pages of {bs}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_takes_weight_from_the_keys(tmp_path, dtype):
    """With a large sink the attention layer's output all but vanishes; left out, the logits move."""
    folder, cfg, w = marked_model(tmp_path, dtype, "attention", 64)
    path = os.path.join(folder, "model.safetensors")
    w["l0.mix.sink"] = torch.tensor([9.0, 7.0]).to(w["l0.mix.sink"].dtype)
    save_file(w, path, metadata={"format": "pt"})
    w = load_file(path)
    toks = prompts_for(cfg, [80], 3)["r0"]
    none = dict(w)
    none["l0.mix.sink"] = torch.full((2,), -60.0)
    a, b = plain.forward(cfg, w, toks), plain.forward(cfg, none, toks)
    assert float((a - b).abs().max()) > 0.3 * float(b.std())
    runner = make_runner(folder, dtype, block_size=8, num_blocks=40, tokens=256)
    for plan in ([[("x", 0, 80)]], [[("x", 0, 40)]] + [[("x", i, i + 1)] for i in range(40, 80)]):
        check(replay(runner, {"x": toks}, plan)["x"], cfg, w, toks, dtype, "sink")


def test_pages_behind_window_and_chunk_come_back_while_a_request_lives(tmp_path):
    att = dict(heads=3, kv_heads=1, dim=24, scale=0.15, window=19, rot_dims=12, base=5000.0)
    par = dict(left=dict(heads=2, kv_heads=2, dim=16, vdim=24, scale=0.2, chunk=19, rot_dims=8),
               right=dict(heads=2, dim=8, vdim=8, decay=[0.9, 0.99]), left_scale=1.0, right_scale=1.0)
    cfg = make_config(vocab=120, width=48, layers=[("attention", att, 40), ("parallel", par, None)], eps=1e-5,
                      max_positions=512)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=8, dtype="float32")
    liven(folder)
    w = load_file(os.path.join(folder, "model.safetensors"))
    runner = make_runner(folder, torch.float32, block_size=8, num_blocks=6)
    toks = prompts_for(cfg, [200], 6)["r0"]       # 25 pages if all were kept; 19 keys need 4 at most
    got = replay(runner, {"r0": toks}, in_portions("r0", 200, (24, 1, 9)))
    check(got["r0"], cfg, w, toks, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["gla", "retention"])
def test_memory_carries_a_token_from_the_far_past(tmp_path, dtype, kind):
    """A model of memories whose decays are held near one: what token 0 was still shows in the
    logits hundreds of tokens later, through portions and single tokens and through a slot that
    others have used."""
    if kind == "gla":
        layers = [("gla", dict(heads=2, dim=16, vdim=16, tau=64.0, rank=4), None),
                  ("gla", dict(heads=2, dim=16, vdim=16, tau=64.0, rank=4), 24)]
    else:
        par = dict(left=dict(heads=1, kv_heads=1, dim=16, vdim=16, scale=0.25, chunk=3),
                   right=dict(heads=2, dim=16, vdim=16, decay=[0.9999, 1.0], rot_dims=16), left_scale=0.01,
                   right_scale=1.0)
        layers = [("parallel", par, None), ("parallel", par, 24)]
    cfg = make_config(vocab=40, width=32, layers=layers, eps=1e-6, max_positions=512)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=6, dtype=NAME[dtype])
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        if k.endswith(".a2.b"):
            w[k] = torch.full_like(w[k], 6.0)          # sigmoid(6)^(1/64): nothing fades
        elif k.endswith((".q", ".k", ".v", ".g")) and ".mix" in k:
            w[k] = (w[k].float() * 8.0).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})
    w = load_file(path)
    runner = make_runner(folder, dtype, block_size=8, num_blocks=16, seqs=2, tokens=512)
    assert len(runner.model.state_specs) == 2
    toks = prompts_for(cfg, [400], 7)["r0"]
    other = [(toks[0] + 1) % 40] + toks[1:]
    a, b = plain.forward(cfg, w, toks), plain.forward(cfg, w, other)
    assert float((a[-1] - b[-1]).abs().max()) > 0.05 * float(a.std())     # the first token still matters
    plan = in_portions("x", 300, (64, 3, 2, 50)) + [[("x", i, i + 1)] for i in range(300, 400)]
    for seq in (toks, other):
        got = replay(runner, {"x": seq}, plan)["x"]
        check(got, cfg, w, seq, dtype, "far past")


def random_shape(seed: int) -> dict:
    """A model whose every size, count, constant and layer order is drawn."""
    rng = random.Random(seed)
    width = rng.choice([24, 40, 56, 64, 88, 104, 128])

    def rot(dim, even_only=2):
        r = rng.choice([0, 2, 4, 8, 12, 16, 32, 64])
        return min(r, dim - dim % 2)

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return rng.choice([8, 24, 40, 64, 136])
        experts = rng.choice([1, 2, 3, 5, 8, 12])
        return (rng.choice([8, 16, 32, 40, 64]), experts, rng.randint(1, min(experts, 4)), rng.choice([0, 8, 24, 64]))

    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["gla", "attention", "parallel"])
        if kind == "gla":
            m = dict(heads=rng.choice([1, 2, 3, 5]), dim=rng.choice([4, 16, 24, 40, 64, 96, 144]),
                     vdim=rng.choice([8, 16, 24, 40, 64, 80, 130]), tau=rng.choice([1.0, 4.0, 16.0, 50.0]),
                     rank=rng.choice([1, 3, 8, 16, 40]))
        elif kind == "attention":
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 20, 32, 48, 64, 72])
            r = rot(dim)
            m = dict(heads=kv * rng.choice([1, 2, 3, 4]), kv_heads=kv, dim=dim,
                     scale=rng.choice([0.05, 0.125, 0.3, dim ** -0.5]), window=rng.choice([1, 2, 7, 16, 25, 40, 64, 300]),
                     rot_dims=r, base=rng.choice([100.0, 10000.0, 1000000.0]),
                     scaling=rng.choice([None, (rng.choice([2.0, 8.0]), 1.0, rng.choice([2.0, 4.0]), rng.choice([16, 64, 512]))]))
        else:
            kv = rng.choice([1, 2, 3])
            dim, mdim = rng.choice([8, 16, 20, 32, 48, 64]), rng.choice([4, 8, 16, 24, 32, 72])
            heads = rng.choice([1, 2, 3, 4])
            left = dict(heads=kv * rng.choice([1, 2, 4]), kv_heads=kv, dim=dim, vdim=rng.choice([8, 16, 24, 40, 64]),
                        scale=rng.choice([0.05, 0.125, 0.3]), chunk=rng.choice([1, 2, 7, 16, 25, 40, 64, 300]),
                        rot_dims=rot(dim), base=rng.choice([100.0, 10000.0]),
                        scaling=rng.choice([None, (rng.choice([2.0, 8.0]), rng.choice([16, 64, 2048]), 32.0, 1.0)]))
            right = dict(heads=heads, dim=mdim, vdim=rng.choice([8, 16, 24, 40, 64, 100]),
                         decay=[rng.choice([0.5, 0.9, 0.97, 0.999, 1.0]) for _ in range(heads)],
                         rot_dims=rot(mdim), base=rng.choice([100.0, 1000000.0]))
            m = dict(left=left, right=right, left_scale=rng.choice([0.5, 1.0, 1.2]),
                     right_scale=rng.choice([0.5, 1.0, 2.0]))
        layers.append((kind, m, mlp()))
    return make_config(vocab=rng.choice([17, 64, 100, 257, 512]), width=width, layers=layers,
                       eps=rng.choice([1e-6, 1e-5, 1e-3, 0.1]), max_positions=256)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(12))
def test_models_drawn_at_random(tmp_path, seed, dtype):
    """Whole, token by token, in portions and in a batch with pages and slots used again."""
    cfg = random_shape(seed)
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=seed, dtype=NAME[dtype])
    liven(folder)
    w = load_file(os.path.join(folder, "model.safetensors"))
    bs = [4, 8, 16, 24][seed % 4]
    seqs = prompts_for(cfg, [90, 41, 2, 64, 33], seed)
    runner = make_runner(folder, dtype, block_size=bs, num_blocks=-(-300 // bs), seqs=3)
    plan = ([[("r0", 0, 90)]] + [[("r1", i, i + 1)] for i in range(41)] + in_portions("r3", 64, (5, 2, 17, 3))
            + [[("r0", 0, 40), ("r2", 0, 1)], [("r2", 1, 2), ("r0", 40, 41), ("r4", 0, 20)],
               [("r0", 41, 90), ("r4", 20, 21), ("r1", 0, 30)], [("r4", 21, 33), ("r1", 30, 41)]])
    got = replay_all(runner, seqs, plan)
    for r, t in seqs.items():
        for k, logits in enumerate(got[r]):
            check(logits, cfg, w, t, dtype, f"seed {seed}, {r}, pass {k}: {cfg}")
    if runner.model.state_specs:
        assert runner.cache.slots.num_free == 3
    if runner.model.cache_groups:
        assert runner.cache.num_free_blocks == -(-300 // bs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name, dtype):
    """The framework's own entry point and scheduler: prompts admitted in portions under a small
    token budget, decode steps replayed from captured graphs (the memories advance on the
    device), three slots for five requests."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    engine = kvforge_amd.InferenceEngine.from_folder(
        folder, kvforge_amd.EngineConfig(
            cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=60), dtype=dtype,
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=24, max_model_len=256)))
    prompts = list(prompts_for(cfg, [30, 2, 11, 45, 1], 7).values())
    outs = engine.generate(prompts, kvforge_amd.SamplingParams(max_tokens=40, temperature=0.0, ignore_eos=True))
    margin = 1e-3 if dtype == torch.float32 else 0.25
    followed, missed = 0, []
    for p, o in zip(prompts, outs):
        assert len(o.output_token_ids) == 40
        logits = plain.forward(cfg, w, p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            if float(row.max() - row[tok]) > margin * float(row.std()):
                missed.append((len(p), i, tok))
        followed += o.output_token_ids != plain.greedy(cfg, w, p[-1:], 40)
    assert len(missed) <= (0 if dtype == torch.float32 else 6), missed
    assert followed >= 4          # what comes out depends on more than the last token
    assert engine.cache.slots.num_free == 3 and engine.cache.num_free_blocks == 60
    if engine.runner.use_graphs:
        assert engine.runner.num_graph_replays > 0


def test_a_request_that_loses_its_pages_and_slot_is_read_again_from_its_first_token(tmp_path_factory):
    """Shape b keeps every key of its widest window, so three requests outgrow the pool: the
    scheduler takes one's pages and state slot away and feeds it again later, prompt and
    generated tokens, into a slot and pages that others have used; its memories start from zeros
    again."""
    folder, cfg, w = model_folder(tmp_path_factory, "b", torch.float32)
    engine = kvforge_amd.InferenceEngine.from_folder(
        folder, kvforge_amd.EngineConfig(
            cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=20, watermark=0.0), dtype=torch.float32,
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=32, max_model_len=128)))
    prompts = list(prompts_for(cfg, [30, 26, 33], 10).values())
    outs = engine.generate(prompts, kvforge_amd.SamplingParams(max_tokens=40, temperature=0.0, ignore_eos=True))
    assert engine.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        assert len(o.output_token_ids) == 40
        logits = plain.forward(cfg, w, p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 1e-3 * float(row.std()), (i, tok)
    assert engine.cache.slots.num_free == 3 and engine.cache.num_free_blocks == 20


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_in_a_process_of_its_own(tmp_path_factory, tmp_path, dtype):
    """``bin/trace_run`` as a user runs it: whole, token by token, in portions and mixed, with
    a pool of exactly the peak of live tokens and four state slots."""
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    folder, cfg, w = model_folder(tmp_path_factory, "a", td)
    prompts = prompts_for(cfg, [37, 81, 100, 53], 8)
    tb = ru.TraceBuilder()
    for rid, toks in prompts.items():
        for mode, fn in (("w", ru.whole), ("d", ru.decode_tail), ("p", ru.portions)):
            fn(tb, f"{rid}#{mode}", toks)
    ru.mixed(tb, {f"{rid}#m": toks for rid, toks in prompts.items()}, 9)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out)
    want = {rid: plain_logits(cfg, w, toks, td) for rid, toks in prompts.items()}
    for sid, rows in enumerate(tb.expect):
        if not rows:
            continue
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{sid}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())
        truth = torch.stack([want[rid.split("#")[0]][0][pos] for rid, pos in rows])
        runs = [torch.stack([want[rid.split("#")[0]][1][k][pos] for rid, pos in rows])
                for k in range(len(next(iter(want.values()))[1]))]
        close_to_truth(got, truth, runs, td, f"step {sid}")
