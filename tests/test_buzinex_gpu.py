"""Buzinex on the GPU: each mechanism's kernels alone against the plain functions, then whole
models (other sizes in every test than anywhere else) through the engine's runner, cache and
state slots: whole prompts, the stream after every layer, token-by-token decoding, portions down
to two tokens, unequal requests in one batch, pages and slots that come back, marked keys on
either side of a window and far back, a memory that carries a token for hundreds of steps,
models drawn at random, and greedy generation through the engine and its scheduler."""

from __future__ import annotations

import math
import os
import random

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import kvforge_amd
from kvforge_amd.config.presets import buzinex as make_config
from kvforge_amd.engine.batch import StepEntry
from tests import replay_util as ru
from tests.plain import buzinex as plain
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
@pytest.mark.parametrize("h", [36, 100, 1024, 2500])
def test_a_sublayers_rows_are_normed_and_added_to_the_stream(h):
    x, y, w = rand(7, h, seed=h, scale=3.0), rand(7, h, seed=h + 1, scale=0.01), 1.0 + rand(h, seed=2, scale=0.3)
    y[3] = 0.0                                         # a row of zeros stays zeros (eps inside the root)
    dev = x.clone().to(DEV)
    ops().rms_add(dev, y.to(DEV), w.to(DEV), 1e-5)
    torch.testing.assert_close(dev.cpu(), x + plain.norm(y, w, 1e-5), atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [36, 100, 1024, 1030, 2500, 4096, 5000])
def test_the_sum_and_the_next_sublayers_norm_in_one_pass(dtype, h):
    x, y = rand(7, h, seed=h, scale=3.0), rand(7, h, seed=h + 1, scale=0.01)
    w, w2 = 1.0 + rand(h, seed=2, scale=0.3), 1.0 + rand(h, seed=3, scale=0.3)
    y[3] = 0.0
    x[5] = 0.0                                          # the stream is all the sublayer's here
    dev = x.clone().to(DEV)
    out = torch.zeros(7, h, dtype=dtype, device=DEV)
    ops().rms_add_norm(dev, y.to(DEV), w.to(DEV), 1e-5, w2.to(DEV), 1e-3, out)
    stream = x + plain.norm(y, w, 1e-5)
    torch.testing.assert_close(dev.cpu(), stream, atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(out.float().cpu(), plain.norm(stream, w2, 1e-3), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,dk,d,coef,every", [(4, 2, 16, 16, 0.5, 4), (3, 1, 24, 32, 0.25, 1), (8, 1, 64, 64, 2.0, 7),
                                                  (5, 5, 7, 16, 0.1, 1000), (2, 1, 256, 256, 1.0, 64)])
def test_head_norm_and_query_temperature_without_rotation(dtype, H, KV, dk, d, coef, every):
    """q and k heads divided by their root mean square and weighted, the queries then stretched
    by what their position asks; k and v go to scattered pages as they are."""
    n, bs, eps = 10, 8, 1e-4
    rows = rand(n, (H + 2 * KV) * d, seed=dk).view(n, H + 2 * KV, d).clone()
    rows[:, :H + KV, dk:] = 0.0
    rows = rows.view(n, -1).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 5, 6, 7, 13, 62, 63], dtype=torch.int32)
    qw, kw = 1.0 + rand(dk, seed=1, scale=0.2), 1.0 + rand(dk, seed=2, scale=0.2)
    table = i32([[7, 2, 5, 0, 3, 1, 6, 4]])
    kp = torch.full((8, KV, bs, d), 9.0, dtype=dtype, device=DEV)
    vp = torch.full((8, KV, d, bs), 9.0, dtype=dtype, device=DEV)
    dev = rows.clone().to(DEV)
    ops().qknorm_rope_kvwrite(dev, pos.to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV), None, None,
                              table, kp, vp, H, KV, d, qw.to(DEV), kw.to(DEV), dk, eps, q_temp=(coef, every))
    x = rows.float().view(n, H + 2 * KV, d)
    temp = plain.query_temperature(pos, coef, every)
    assert float(temp.max()) > 1.0 or every > 64
    q = plain.norm(x[:, :H, :dk], qw, eps) * temp[:, None, None]
    k = plain.norm(x[:, H:H + KV, :dk], kw, eps)
    got = dev.float().cpu().view(n, H + 2 * KV, d)
    torch.testing.assert_close(got[:, :H, :dk], q, **tol(dtype))
    for t, p in enumerate(pos.tolist()):
        page, off = int(table[0, p // bs]), p % bs
        torch.testing.assert_close(kp[page, :, off, :dk].float().cpu(), k[t], **tol(dtype))
        torch.testing.assert_close(vp[page, :, :, off].float().cpu(), x[t, H + KV:], **tol(dtype))


def capped_reference(paged, q, seq_lens, q_lens, scale, window, cap, sink, G):
    outs, off = [], 0
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        k = paged.keys[s].float().repeat_interleave(G, dim=1)
        v = paged.values[s].float().repeat_interleave(G, dim=1)
        outs.append(plain.attend(q[off:off + ql].float(), k, v, scale, plain.visible_keys(ql, n, window or None),
                                 cap, sink))
        off += ql
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (8, 1, 64, 16), (3, 1, 48, 8), (6, 2, 128, 16), (4, 4, 64, 16)])
@pytest.mark.parametrize("cap", [2.0, 50.0])
def test_attention_with_capped_scores(dtype, H, KV, d, bs, cap):
    """Query runs and single tokens (one cut and several).  Queries so long that many scores
    lie well beyond the small cap, where it flattens them, and within the large one."""
    scale = 1 / math.sqrt(d)
    for seq_lens, q_lens in (([90, 33, 70, 5], [40, 33, 2, 5]), ([7, 90, 1, 300], [1, 1, 1, 1])):
        paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + int(cap))
        n = sum(q_lens)
        buf = rand(n, H * d, seed=d + 1, scale=2.5).to(dtype)
        cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
        ctx = torch.tensor(seq_lens, dtype=torch.int32)
        want = capped_reference(paged, buf.view(n, H, d), seq_lens, q_lens, scale, 0, cap, None, H // KV).reshape(n, H * d)
        free = capped_reference(paged, buf.view(n, H, d), seq_lens, q_lens, scale, 0, None, None, H // KV).reshape(n, H * d)
        if cap < 10.0:
            assert float((want - free).abs().max()) > 0.05       # the cap matters here
        args = (buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV))
        if max(q_lens) > 1:
            out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
            ops().attn_prefill(*args, cu.to(DEV), ctx.to(DEV), prefill_work(q_lens, H // KV, dtype, d, bs).to(DEV),
                               out, H, KV, d, scale, 0, score_cap=cap)
            torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
            continue
        for splits in (1, 3):
            out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
            ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV))
            ops().attn_decode(*args, None, n, cu.to(DEV), ctx.to(DEV), out, H, KV, d, scale, 0, splits, ws,
                              score_cap=cap)
            torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dim,rot,rank,d", [(4, 16, 8, 24, 32), (3, 20, 12, 36, 48), (1, 64, 32, 96, 128),
                                              (5, 0, 16, 8, 32), (2, 24, 0, 40, 48), (8, 128, 64, 192, 256)])
def test_a_projected_row_becomes_one_key_and_per_head_queries(dtype, H, dim, rot, rank, d):
    n, eps = 6, 1e-3
    proj = rand(n, H * (dim + rot) + rank + rot + 3, seed=rank).to(dtype)     # something behind the row
    w = 1.0 + rand(rank, seed=1, scale=0.3)
    qkv = torch.full((n, (H + 2) * d), 7.0, dtype=dtype, device=DEV)
    ops().latent_split(proj.to(DEV), qkv, w.to(DEV), eps, H, dim, rot, rank, d)
    got = qkv.float().cpu().view(n, H + 2, d)
    x = proj.float()
    q = x[:, :H * (dim + rot)].view(n, H, dim + rot)
    down = x[:, H * (dim + rot):]
    c = plain.norm(down[:, :rank], w, eps)
    torch.testing.assert_close(got[:, :H, :rot], q[..., dim:], atol=0, rtol=0)
    if dim:
        assert float((got[:, :H, rot:rot + rank] - 7.0).abs().max()) == 0.0     # left for the queries' read-in
    else:
        assert float(got[:, :H, rot:].abs().max()) == 0.0
    assert float(got[:, :, rot + rank:].abs().max() if d > rot + rank else 0.0) == 0.0
    torch.testing.assert_close(got[:, H, :rot], down[:, rank:rank + rot], atol=0, rtol=0)
    torch.testing.assert_close(got[:, H, rot:rot + rank], c, **tol(dtype))
    torch.testing.assert_close(got[:, H + 1, rot:rot + rank], c, **tol(dtype))
    assert float(got[:, H + 1, :rot].abs().max() if rot else 0.0) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 33, 100, 200, 257, 330])
@pytest.mark.parametrize("lead", [2, 8])
@pytest.mark.parametrize("H,O,I,in_head,out_head", [(4, 24, 16, 24, 32), (3, 36, 20, 32, 48), (1, 100, 70, 70, 100),
                                                    (5, 8, 130, 130, 8), (2, 192, 128, 192, 256), (3, 72, 40, 48, 80),
                                                    (2, 130, 200, 200, 140), (2, 40, 256, 256, 40), (1, 24, 264, 264, 32)])
def test_a_matrix_per_head(dtype, n, lead, H, O, I, in_head, out_head):
    """Rows in which a head starts every ``in_head`` elements and uses ``I`` of them; outputs
    written into wider rows, the columns between them left alone.  Rows that start ``lead``
    elements into wider ones: with 8 (and sizes that are multiples of 8) bfloat16 heads start on
    16 bytes, which is what the matrix-core kernels take (one for few rows, one that keeps the rows
    in registers from 256 rows on); the others go through the plain one."""
    x = rand(n, H * in_head + 8, seed=O).to(dtype)
    w = rand(H, O, I, seed=I, scale=I ** -0.5).to(dtype)
    pad = 1 if lead == 2 else 4              # (with 4, output rows whose heads start on 8 bytes)
    out = torch.full((n, H * out_head + 2 * pad), 7.0, dtype=dtype, device=DEV)
    ops().head_product(x.to(DEV)[:, lead:], in_head, w.to(DEV), out[:, pad:], out_head)
    xs = torch.stack([x.float()[:, lead + h * in_head:lead + h * in_head + I] for h in range(H)], 1)
    want = torch.einsum("nhi,hoi->nho", xs, w.float())
    got = out.float().cpu()
    for h in range(H):
        torch.testing.assert_close(got[:, pad + h * out_head:pad + h * out_head + O], want[:, h], **tol(dtype))
    assert float(got[:, :pad].min()) == 7.0 and float(got[:, pad + (H - 1) * out_head + O:].min()) == 7.0
    if out_head > O:
        assert float((got[:, pad + O:pad + out_head] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [24, 72, 256, 1000])
def test_every_input_of_the_memory_mixes_a_token_with_the_one_before(dtype, width):
    """Three steps: runs and single tokens; a run's first token takes its predecessor from the
    slot, a sequence's first token from nowhere (whatever the slot holds), and a sequence without
    a slot from nowhere either."""
    M, S = 5, 10
    lens = {"a": 9, "b": 4, "c": 3}
    data = {r: rand(n, width, seed=i + width).to(dtype) for i, (r, n) in enumerate(lens.items())}
    mu = rand(M, width, seed=7, scale=0.5)
    state = torch.full((3, S + width), 3.0, device=DEV)
    slot = {"a": 2, "b": 0, "c": 2}                  # c comes when a has gone, into its slot
    got = {r: [] for r in lens}
    for step in ([("a", 0, 5), ("b", 0, 1)], [("b", 1, 2), ("a", 5, 6)], [("a", 6, 9), ("b", 2, 4)], [("c", 0, 1)],
                 [("c", 1, 3)]):
        h = torch.cat([data[r][a:b] for r, a, b in step] + [torch.ones(1, width, dtype=dtype)]).to(DEV)
        counts = [b - a for _, a, b in step] + [1]
        n = sum(counts)
        cu = i32([0] + list(np.cumsum(counts)))
        pos = torch.cat([torch.arange(a, b) for _, a, b in step] + [torch.full((1,), 4)]).int().to(DEV)
        seq_of = i32([s for s, c in enumerate(counts) for _ in range(c)])
        out = torch.zeros(M, n, width, dtype=dtype, device=DEV)
        ops().wkv_mix(h, mu.to(DEV), state, S, i32([slot[r] for r, _, _ in step] + [-1]), seq_of, cu, pos, out,
                      len(counts))
        off = 0
        for r, a, b in step:
            got[r].append(out[:, off:off + b - a].float().cpu())
            off += b - a
            torch.testing.assert_close(state[slot[r], S:].cpu(), data[r][b - 1].float(), atol=0, rtol=0)
        torch.testing.assert_close(out[:, off].float().cpu(), (1.0 - mu).to(dtype).float(), **tol(dtype))
        assert float((state[:, :S] - 3.0).abs().max()) == 0.0          # nothing in front of the kept row is touched
    for r in lens:
        x = data[r].float()
        want = x[None] + (plain.shifted(x) - x)[None] * mu[:, None, :]
        torch.testing.assert_close(torch.cat(got[r], 1), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk", [(2, 8), (6, 32), (1, 40), (3, 64), (2, 100), (2, 128), (1, 200), (1, 256)])
def test_the_memory_over_runs_and_steps(dtype, H, dk):
    """Four sequences in three steps: runs of many tokens (more than a stage), of two and of one;
    a sequence that starts in the slot another gave back (which still holds that one's memory);
    a sequence without a slot.  Decays from all but nothing to all but one."""
    HD = H * dk
    lens = {"a": 43, "b": 9, "c": 1, "d": 12}
    cols = 3 * HD + 5                                   # rows wider than r, k, v: something behind them
    data = {r: (rand(n, cols, seed=i + dk).to(dtype), rand(n, HD + 2, seed=i + 50, scale=2.0))
            for i, (r, n) in enumerate(lens.items())}
    w0, u = rand(HD, seed=9, scale=1.5) - 1.0, rand(HD, seed=10, scale=0.5)
    want = {}
    for r, (rows, z) in data.items():
        x = rows.float()
        decay = torch.exp(-torch.exp(z[:, :HD] + w0)).view(-1, H, dk)
        if r == "a":
            assert float(decay.min()) < 0.05 and float(decay.max()) > 0.95
        want[r] = plain.wkv_recurrence(x[:, 5:5 + HD].reshape(-1, H, dk), x[:, 5 + HD:5 + 2 * HD].reshape(-1, H, dk),
                                       x[:, 5 + 2 * HD:].reshape(-1, H, dk), decay, u.view(H, dk)).reshape(-1, HD)
    state = torch.full((3, ops().wkv_state_floats(H, dk, 24)), 3.0, device=DEV)   # junk
    slot = {"a": 2, "b": 0, "c": 1, "d": 1}
    got = {r: [] for r in lens}
    for step in ([("a", 0, 34), ("b", 0, 1), ("c", 0, 1)], [("b", 1, 3), ("d", 0, 11), ("a", 34, 35)],
                 [("a", 35, 43), ("d", 11, 12), ("b", 3, 9)]):
        rows = torch.cat([data[r][0][a:b] for r, a, b in step] + [data["a"][0][:2]]).to(DEV)
        z = torch.cat([data[r][1][a:b] for r, a, b in step] + [data["a"][1][:2]]).to(DEV)
        counts = [b - a for _, a, b in step] + [2]       # and a sequence without a slot
        cu = i32([0] + list(np.cumsum(counts)))
        pos = torch.cat([torch.arange(a, b) for _, a, b in step] + [torch.arange(2)]).int().to(DEV)
        out = torch.full((rows.shape[0], HD), 5.0, device=DEV)
        ops().wkv_scan(rows, 5, 5 + HD, 5 + 2 * HD, z, w0.to(DEV), u.to(DEV), cu, pos,
                       i32([slot[r] for r, _, _ in step] + [-1]), state, out, len(counts), H, dk)
        off = 0
        for (r, a, b) in step:
            got[r].append(out[off:off + b - a].cpu())
            off += b - a
        torch.testing.assert_close(out[off:].cpu(), want["a"][:2], atol=2e-4, rtol=2e-4)   # from zeros, nothing kept
        assert float((state[:, HD * dk:] - 3.0).abs().max()) == 0.0   # the kept row behind the memories is not the scan's
    for r in lens:      # sums of up to 256 products over up to 43 tokens, in another order than the plain one's
        torch.testing.assert_close(torch.cat(got[r]), want[r], atol=2e-5 * float(want[r].abs().max()), rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk", [(2, 8), (3, 64), (2, 100), (1, 132), (1, 256)])
def test_the_memory_over_long_runs_chunk_by_chunk(dtype, H, dk):
    """Runs of 64 tokens and more are cut into chunks that go side by side; in one step with
    them, short runs that go token by token.  A long run that goes on from what a short one left
    and the other way round, a last chunk of one token and a full one, a slot that still holds
    another's memory, a long run without a slot, and strong decays (whole chunks that forget
    all that was before them)."""
    HD = H * dk
    lens = {"a": 235, "b": 70, "c": 129, "d": 5}
    data = {r: (rand(n, 3 * HD, seed=i + dk).to(dtype), rand(n, HD, seed=i + 70, scale=2.0))
            for i, (r, n) in enumerate(lens.items())}
    data["c"][1][40:60] += 6.0                            # decays of exp(-exp(6 + ...)): nothing survives
    w0, u = rand(HD, seed=9, scale=1.5) - 1.0, rand(HD, seed=10, scale=0.5)
    want = {}
    for r, (rows, z) in data.items():
        x = rows.float()
        decay = torch.exp(-torch.exp(z + w0)).view(-1, H, dk)
        want[r] = plain.wkv_recurrence(x[:, :HD].reshape(-1, H, dk), x[:, HD:2 * HD].reshape(-1, H, dk),
                                       x[:, 2 * HD:].reshape(-1, H, dk), decay, u.view(H, dk)).reshape(-1, HD)
    state = torch.full((3, ops().wkv_state_floats(H, dk, 8)), 3.0, device=DEV)   # junk
    slot = {"a": 2, "b": 0, "c": 1, "d": 1}
    got = {r: [] for r in lens}
    steps = ([("a", 0, 150), ("d", 0, 3)], [("a", 150, 153), ("b", 0, 70), ("d", 3, 5)],
             [("c", 0, 64), ("a", 153, 170)], [("a", 170, 235), ("c", 64, 129)])
    for step in steps:
        rows = torch.cat([data[r][0][a:b] for r, a, b in step] + [data["b"][0][:65]]).to(DEV)
        z = torch.cat([data[r][1][a:b] for r, a, b in step] + [data["b"][1][:65]]).to(DEV)
        counts = [b - a for _, a, b in step] + [65]      # and a long run without a slot
        cu = i32([0] + list(np.cumsum(counts)))
        pos = torch.cat([torch.arange(a, b) for _, a, b in step] + [torch.arange(65)]).int().to(DEV)
        chunks, runs = ops().wkv_multi_plan(counts)
        assert len(runs) // 3 == sum(c >= 64 for c in counts) >= 2
        nc = len(chunks) // 4
        multi = {"chunks": i32(chunks).view(-1, 4), "runs": i32(runs).view(-1, 3),
                 "G": torch.full((nc, H, dk, dk), 7.0, device=DEV), "D": torch.full((nc, H, dk), 7.0, device=DEV)}
        out = torch.full((rows.shape[0], HD), 5.0, device=DEV)
        ops().wkv_scan(rows, 0, HD, 2 * HD, z, w0.to(DEV), u.to(DEV), cu, pos,
                       i32([slot[r] for r, _, _ in step] + [-1]), state, out, len(counts), H, dk, multi=multi,
                       short_runs=any(c < 64 for c in counts))
        off = 0
        for (r, a, b) in step:
            got[r].append(out[off:off + b - a].cpu())
            off += b - a
        torch.testing.assert_close(out[off:].cpu(), want["b"][:65], atol=2e-5 * float(want["b"].abs().max()), rtol=2e-4)
    for r in lens:
        torch.testing.assert_close(torch.cat(got[r]), want[r], atol=2e-5 * float(want[r].abs().max()), rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk", [(3, 16), (2, 40), (1, 256)])
def test_heads_normed_weighted_and_gated_and_the_decays_tanh(dtype, H, dk):
    n, eps = 5, 1e-3
    raw = rand(n, H * dk, seed=dk, scale=3.0)
    raw[2, :dk] = 0.0                                   # a head that gave nothing
    rows = rand(n, 2 * H * dk, seed=1).to(dtype)
    w = 1.0 + rand(H * dk, seed=2, scale=0.3)
    out = torch.zeros(n, H * dk, dtype=dtype, device=DEV)
    ops().wkv_out(raw.to(DEV), rows.to(DEV)[:, H * dk:], w.to(DEV), eps, out, H, dk)
    g = rows.float()[:, H * dk:]
    want = plain.rms(raw.view(n, H, dk), eps).reshape(n, H * dk) * w * g * torch.sigmoid(g)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
    x = rand(n, 48, seed=3, scale=2.0)
    t = torch.zeros(n, 48, dtype=dtype, device=DEV)
    ops().tanh_cast(x.to(DEV), t)
    torch.testing.assert_close(t.float().cpu(), torch.tanh(x).to(dtype).float(), atol=1e-6 if dtype == torch.float32 else 8e-3,
                               rtol=0)


# ============================================================================ whole models
def shape_a():
    """All three mixers, every size another than anywhere else in this file: groups of three
    query heads, value heads larger than key heads and neither a multiple of 16, a latent head
    whose parts are no multiples of 8, a window that ends inside a page, a memory in the middle
    and another at the end, layers with and without a feed-forward in every kind."""
    att = dict(heads=6, kv_heads=2, dim=24, vdim=40, scale=0.2, softcap=12.0, q_temp=(0.4, 5))
    lat = dict(heads=3, dim=20, rot_dim=12, vdim=28, kv_rank=36, scale=0.15, window=19, base=5000.0)
    rec = dict(heads=3, dim=16, decay_rank=6)
    return make_config(vocab=211, width=72, layers=[("attention", att, 88), ("latent_attention", lat, 40),
                                                    ("wkv", rec, None), ("latent_attention", lat, None),
                                                    ("attention", att, None), ("wkv", rec, 56)],
                       embedding_scale=6.5, logit_scale=0.3, logit_softcap=20.0, eps=1e-5, max_positions=2048)


def shape_b():
    """What a model may make equal or one: as many kv heads as heads, a query temperature that
    steps at every token and one that never steps, a cap far above every score, one head of
    latent attention, a window of one key in one layer and longer than any prompt in another,
    one memory head as wide as the stream, a decay of rank one, no cap on the logits, scales of
    one, a model that starts with a memory."""
    a1 = dict(heads=2, kv_heads=2, dim=32, vdim=32, scale=32 ** -0.5, softcap=1000.0, q_temp=(1.0, 1))
    a2 = dict(heads=4, kv_heads=4, dim=16, vdim=16, scale=0.25, softcap=5.0, q_temp=(0.5, 100000))
    l1 = dict(heads=1, dim=32, rot_dim=32, vdim=64, kv_rank=32, scale=0.125, window=1, base=10000.0)
    l2 = dict(heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=16, scale=0.18, window=4096, base=100.0)
    rec = dict(heads=1, dim=64, decay_rank=1)
    return make_config(vocab=97, width=64, layers=[("wkv", rec, 32), ("attention", a1, 32), ("latent_attention", l1, None),
                                                   ("latent_attention", l2, 48), ("attention", a2, None)],
                       embedding_scale=1.0, logit_scale=1.0, logit_softcap=None, eps=1e-6, max_positions=512)


def shape_c():
    """One kv head under eight, head size 64 (the matrix-core kernels' own) and a latent row of
    16 + 112 = 128 elements, a memory whose keys span two waves' rows, a window over several
    pages, nothing but memories behind the attention."""
    att = dict(heads=8, kv_heads=1, dim=64, vdim=48, scale=0.125, softcap=30.0, q_temp=(0.3, 16))
    lat = dict(heads=8, dim=48, rot_dim=16, vdim=32, kv_rank=112, scale=0.125, window=33, base=1000000.0)
    rec = dict(heads=2, dim=132, decay_rank=20)
    return make_config(vocab=300, width=128, layers=[("latent_attention", lat, 96), ("attention", att, 160),
                                                     ("wkv", rec, None), ("wkv", rec, 64)],
                       embedding_scale=11.3, logit_scale=0.09, logit_softcap=30.0, eps=1e-6, max_positions=512)


def shape_d():
    """Layers wide enough for the kernels that serving a real model takes: heads of 64 on the
    matrix cores, a latent row of 32 + 160 elements, `head_product` on the matrix cores, a
    feed-forward deep enough for a down projection cut in two halves of K, memory heads of one
    wave each, a vocabulary that ends inside a group of 16 columns."""
    att = dict(heads=6, kv_heads=2, dim=64, vdim=64, scale=0.125, softcap=25.0, q_temp=(0.35, 32))
    lat = dict(heads=6, dim=64, rot_dim=32, vdim=64, kv_rank=160, scale=0.1, window=50, base=100000.0)
    rec = dict(heads=6, dim=64, decay_rank=32)
    return make_config(vocab=1000, width=384, layers=[("latent_attention", lat, 4096), ("wkv", rec, None),
                                                      ("attention", att, 1024), ("latent_attention", lat, None)],
                       embedding_scale=19.6, logit_scale=0.05, logit_softcap=25.0, eps=1e-5, max_positions=2048)


SHAPE = {"a": shape_a, "b": shape_b, "c": shape_c, "d": shape_d}


def liven(folder: str) -> None:
    """Random weights of std 0.02 give flat attention and a memory that hardly turns.  Scaled so
    that attention is peaked (through the q/k norm weights in one kind, the projections in the
    other), sinks matter, decays swing with the tokens and gates open and close.  (A sublayer's
    size is lost in the norm behind it, so every layer moves the stream as it is.)"""
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        f = 1.0
        if k.endswith(("q.norm", "k.norm")):
            f = 2.5
        elif k.endswith((".mix.q", ".mix.dkv", ".mix.uk")):
            f = 5.0
        elif k.endswith((".mix.r", ".mix.k", ".mix.v", ".mix.g", ".mix.uv")):
            f = 6.0
        elif k.endswith((".mix.w1", ".mix.w2")):
            f = 12.0
        if f != 1.0:
            w[k] = (w[k].float() * f).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})


_MODELS: dict = {}


def model_folder(tmp_path_factory, name: str, dtype):
    key = (name, dtype)
    if key not in _MODELS:
        folder = str(tmp_path_factory.mktemp(f"buzinex_{name}_{NAME[dtype]}"))
        cfg = SHAPE[name]()
        kvforge_amd.write_random_model(folder, cfg, seed=len(name) + 41, dtype=NAME[dtype])
        liven(folder)
        _MODELS[key] = (folder, cfg, load_file(os.path.join(folder, "model.safetensors")))
    return _MODELS[key]


_WANT: dict = {}


def plain_logits(cfg, w, toks, dtype):
    """(the truth, plain runs with the roundings of ``dtype``): the plain model in 64-bit, and in
    32-bit (for a 32-bit engine) or in 32-bit with every trip through memory that a bfloat16
    engine may make rounded to bfloat16: as the weights are, and six times with them moved by
    half a bfloat16 step, which shows the rows where the design multiplies rounding (a memory
    head's first output is its value times the *sign* of ``sum_i r_i u_i k_i``, since the head
    is divided by its own size: where that sum of dozens of products is all but zero, rounding
    decides the sign, and about half of the moved runs show it)."""
    key = (id(w), tuple(toks), dtype)
    if key not in _WANT:
        truth = plain.forward(cfg, w, toks, dtype=torch.float64).float()
        if dtype == torch.bfloat16:
            runs = [plain.forward(cfg, w, toks, store=torch.bfloat16)]
            runs += [plain.forward(cfg, jittered(w, s), toks, store=torch.bfloat16) for s in range(1, 7)]
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
    """From the first token on, and from a prompt's end for 119 tokens, past every window."""
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
    # every key of the full-attention layers is kept: 83 + 50 + 9 + 16 tokens live at the most
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
@pytest.mark.parametrize("name", ["a", "d"])
def test_a_prompt_of_a_thousand_tokens(tmp_path_factory, name, dtype):
    """Dozens of chunks of the memory side by side, the window over many pages, the temperature
    over many steps: whole, in large and small portions, and its last tokens one by one."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    runner = make_runner(folder, dtype, block_size=16, num_blocks=80, tokens=1200)
    toks = prompts_for(cfg, [1100], 11)["r0"]
    for plan in ([[("r0", 0, 1100)]], in_portions("r0", 1100, (300, 64, 65, 7, 129, 2)),
                 [[("r0", 0, 1050)]] + [[("r0", i, i + 1)] for i in range(1050, 1100)]):
        got = replay(runner, {"r0": toks}, plan)["r0"]
        check(got, cfg, w, toks, dtype, f"{name}, {len(plan)} steps")


def marked_model(tmp_path, dtype, kind, window=None):
    """A one-layer model in which token 1 is marked: its embedding lies along one axis that no
    other token uses, the keys read that axis, every query has a constant that meets it, the
    values carry it on.  So the marked token's key scores far above all others for every query."""
    V, W = 50, 32
    if kind == "attention":
        mixer = dict(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, softcap=40.0, q_temp=(0.2, 16))
    else:
        mixer = dict(heads=2, dim=8, rot_dim=4, vdim=16, kv_rank=16, scale=1.0, window=window, base=10000.0)
    cfg = make_config(vocab=V, width=W, layers=[(kind, mixer, None)], embedding_scale=1.0, logit_scale=1.0,
                      logit_softcap=None, eps=1e-6, max_positions=1024)
    folder = str(tmp_path / f"m_{kind}")
    kvforge_amd.write_random_model(folder, cfg, seed=5, dtype=NAME[dtype])
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    e = rand(V, W, seed=1, scale=0.3)
    e[:, 0] = 0.0
    e[:, 1] = 1.0                       # a constant every token has: the queries' handle
    e[1] = 0.0
    e[1, 0] = 6.0
    new = {"embed": e, "l0.norm1": torch.ones(W), "l0.mix.o": rand(W, 32, seed=4, scale=0.5)}
    if kind == "attention":
        wq, wk = torch.zeros(32, W), torch.zeros(16, W)
        wq[15, 1] = wq[31, 1] = 1.0
        wk[15, 0] = 1.0
        wv = rand(16, W, seed=2, scale=0.05)
        wv[:, 0] = rand(16, seed=3, scale=2.0)
        new.update({"l0.mix.q": wq, "l0.mix.k": wk, "l0.mix.v": wv, "l0.mix.q.norm": torch.full((16,), 3.0),
                    "l0.mix.k.norm": torch.full((16,), 3.0)})
    else:
        # the latent's element 3 reads the marked axis; head h's key read-out puts it on the plain
        # element 7 of the head, which its query holds a constant in
        wq, dkv = torch.zeros(2 * 12, W), rand(16 + 4, W, seed=6, scale=0.02)
        wq[7, 1] = wq[12 + 7, 1] = 4.0
        dkv[3] = 0.0
        dkv[3, 0] = 1.0
        uk = torch.zeros(2 * 8, 16)
        uk[7, 3] = uk[8 + 7, 3] = 4.0
        uv = rand(2 * 16, 16, seed=2, scale=0.05)
        uv[:, 3] = rand(32, seed=3, scale=2.0)
        new.update({"l0.mix.q": wq, "l0.mix.dkv": dkv, "l0.mix.dkv.norm": torch.ones(16), "l0.mix.uk": uk,
                    "l0.mix.uv": uv, "l0.mix.sink": torch.tensor([0.5, -2.0])})
    for k, t in new.items():
        assert w[k].shape == t.shape, k
        w[k] = t.to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})
    return folder, cfg, load_file(path)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bs", [8, 16])
def test_one_key_among_hundreds_on_either_side_of_the_window(tmp_path, dtype, bs):
    """The logits follow whether the marked token is just inside the latent attention's window
    (itself and the ``size - 1`` before it) or just outside, at page borders and in the middle
    of pages, read whole, in portions and token by token."""
    window = 37
    folder, cfg, w = marked_model(tmp_path, dtype, "latent_attention", window)
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
def test_one_key_far_back_is_seen_by_every_later_query_of_full_attention(tmp_path, dtype):
    """No window in this kind: the marked token, hundreds of keys back, holds the logits at the
    prompt's end and through decoding, across the steps of the query temperature."""
    folder, cfg, w = marked_model(tmp_path, dtype, "attention")
    runner = make_runner(folder, dtype, block_size=16, num_blocks=40, tokens=512)
    g = torch.Generator().manual_seed(3)
    for at in (0, 15, 16, 200):
        toks = torch.randint(2, 50, (500,), generator=g).tolist()
        toks[at] = 1
        want = plain.forward(cfg, w, toks)
        blind = plain.forward(cfg, w, [t if i != at else 2 for i, t in enumerate(toks)])
        assert float((want[-1] - blind[-1]).abs().max()) > 0.3 * float(want.std())
        for plan in ([[("x", 0, 500)]], in_portions("x", 500, (64, 3, 2, 50)),
                     [[("x", 0, 430)]] + [[("x", i, i + 1)] for i in range(430, 500)]):
            got = replay(runner, {"x": toks}, plan)["x"]
            check(got, cfg, w, toks, dtype, f"marked at {at}")


def test_pages_behind_the_window_come_back_while_a_request_lives(tmp_path):
    lat = dict(heads=3, dim=20, rot_dim=12, vdim=28, kv_rank=36, scale=0.15, window=19, base=5000.0)
    cfg = make_config(vocab=120, width=48, layers=[("latent_attention", lat, 40), ("latent_attention", lat, None)],
                      embedding_scale=3.0, logit_softcap=None, eps=1e-5, max_positions=512)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=8, dtype="float32")
    liven(folder)
    w = load_file(os.path.join(folder, "model.safetensors"))
    runner = make_runner(folder, torch.float32, block_size=8, num_blocks=6)
    toks = prompts_for(cfg, [200], 6)["r0"]       # 25 pages if all were kept; a window of 19 needs 4 at most
    got = replay(runner, {"r0": toks}, in_portions("r0", 200, (24, 1, 9)))
    check(got["r0"], cfg, w, toks, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_memory_carries_a_token_from_the_far_past(tmp_path, dtype):
    """An all-memory model (no pages at all) whose decay is held near one: what token 0 was still
    shows in the logits hundreds of tokens later, through portions and single tokens and through
    a slot that others have used."""
    rec = dict(heads=2, dim=16, decay_rank=4)
    cfg = make_config(vocab=40, width=32, layers=[("wkv", rec, None), ("wkv", rec, 24)],
                      embedding_scale=4.0, logit_softcap=None, eps=1e-6, max_positions=512)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=6, dtype=NAME[dtype])
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        if k.endswith(".w0"):
            w[k] = torch.full_like(w[k], -8.0)         # decay exp(-exp(-8)): nothing fades
        elif k.endswith((".mix.r", ".mix.k", ".mix.v", ".mix.g")):
            w[k] = (w[k].float() * 8.0).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})
    w = load_file(path)
    runner = make_runner(folder, dtype, block_size=8, num_blocks=4, seqs=2, tokens=512)
    assert runner.model.cache_groups == [] and len(runner.model.state_specs) == 2
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
    width = rng.choice([24, 36, 50, 64, 88, 100, 128])
    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["attention", "latent_attention", "wkv"])
        if kind == "attention":
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 20, 32, 48, 64, 72])
            m = dict(heads=kv * rng.choice([1, 2, 3, 4]), kv_heads=kv, dim=dim,
                     vdim=rng.choice([8, 16, 24, 32, 40, 64, 80]), scale=rng.choice([0.05, 0.125, 0.3, dim ** -0.5]),
                     softcap=rng.choice([None, 3.0, 15.0, 50.0]),
                     q_temp=rng.choice([None, (rng.choice([0.1, 0.5, 1.5]), rng.choice([1, 3, 16, 64]))]))
        elif kind == "latent_attention":
            rot = rng.choice([2, 4, 8, 16, 20, 32])
            m = dict(heads=rng.choice([1, 2, 3, 5, 8]), dim=rng.choice([4, 8, 16, 24, 40, 64]), rot_dim=rot,
                     vdim=rng.choice([8, 16, 24, 40, 64]), kv_rank=rng.choice([8, 12, 32, 50, 96, 160]),
                     scale=rng.choice([0.05, 0.125, 0.3]), window=rng.choice([1, 2, 7, 16, 25, 40, 64, 300]),
                     base=rng.choice([100.0, 10000.0, 1000000.0]))
        else:
            m = dict(heads=rng.choice([1, 2, 3, 5]), dim=rng.choice([4, 16, 24, 40, 64, 96, 144]),
                     decay_rank=rng.choice([1, 3, 8, 16, 40]))
        layers.append((kind, m, rng.choice([None, 8, 24, 31, 64, 130])))
    return make_config(vocab=rng.choice([17, 64, 100, 257, 512]), width=width, layers=layers,
                       embedding_scale=rng.choice([1.0, 3.3, width ** 0.5]), logit_scale=rng.choice([1.0, 0.25, width ** -0.5]),
                       logit_softcap=rng.choice([None, 5.0, 30.0]), eps=rng.choice([1e-6, 1e-5, 1e-3, 0.1]),
                       max_positions=256)


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
    """Full attention keeps every key, so three requests outgrow the pool: the scheduler takes
    one's pages and state slot away and feeds it again later, prompt and generated tokens, into
    a slot and pages that others have used; its memory starts from zeros again."""
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


@pytest.mark.parametrize("kind", ["attention", "latent_attention", "wkv"])
def test_trace_replay_of_a_model_of_one_kind(tmp_path, kind):
    """A model with pages and no state slots, with windowed pages alone, and with state slots and
    no pages at all, through ``bin/trace_run`` in bfloat16."""
    mixer = {"attention": dict(heads=4, kv_heads=1, dim=32, vdim=16, scale=0.2, softcap=9.0, q_temp=(0.7, 24)),
             "latent_attention": dict(heads=2, dim=24, rot_dim=8, vdim=40, kv_rank=56, scale=0.2, window=70,
                                      base=30000.0),
             "wkv": dict(heads=4, dim=32, decay_rank=5)}[kind]
    cfg = make_config(vocab=150, width=80, layers=[(kind, mixer, 48), (kind, mixer, None)], embedding_scale=9.0,
                      logit_scale=0.4, logit_softcap=12.0, eps=1e-5, max_positions=1024)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=3, dtype="bfloat16")
    liven(folder)
    w = load_file(os.path.join(folder, "model.safetensors"))
    prompts = prompts_for(cfg, [90, 150, 33, 71], 12)
    tb = ru.TraceBuilder()
    for rid, toks in prompts.items():
        ru.decode_tail(tb, f"{rid}#d", toks)
        ru.portions(tb, f"{rid}#p", toks)
    ru.mixed(tb, {f"{rid}#m": toks for rid, toks in prompts.items()}, 4)
    out = str(tmp_path / "out")
    ru.run_trace(folder, "bfloat16", tb, out)
    want = {rid: plain_logits(cfg, w, toks, torch.bfloat16) for rid, toks in prompts.items()}
    for sid, rows in enumerate(tb.expect):
        if not rows:
            continue
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{sid}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())
        truth = torch.stack([want[rid.split("#")[0]][0][pos] for rid, pos in rows])
        runs = [torch.stack([want[rid.split("#")[0]][1][k][pos] for rid, pos in rows]) for k in range(7)]
        close_to_truth(got, truth, runs, torch.bfloat16, f"{kind}, step {sid}")

