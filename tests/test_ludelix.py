"""Ludelix without a GPU: configuration and its refusals, the builder's tensor names, cache
groups and state slots, and the plain model's mechanisms worked by hand."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from kvforge_amd import registry
from kvforge_amd.config import ConfigError, LudelixConfig
from kvforge_amd.config.presets import PRESETS, ludelix as make_config
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts import (LinearMemory, MixerPair, NamedRMSNorm, PagedAttention, PlainFeedForward,
                               PreNormBlock, RoutedExperts)
from kvforge_amd.weights.random_init import random_tensors
from tests.plain import ludelix as plain

GLA = dict(heads=3, dim=24, vdim=40, tau=6.0, rank=5)
ATT = dict(heads=6, kv_heads=2, dim=24, scale=0.3, window=21, rot_dims=10, base=5000.0, scaling=(3.0, 1.0, 3.0, 40))
PAR = dict(left=dict(heads=4, kv_heads=2, dim=20, vdim=28, scale=0.2, chunk=17, rot_dims=12, base=2000.0,
                     scaling=(5.0, 50, 8.0, 0.5)),
           right=dict(heads=3, dim=12, vdim=20, decay=[0.9, 0.97, 0.995], rot_dims=8, base=100.0),
           left_scale=0.8, right_scale=1.7)


def config(**kw):
    base = dict(vocab=211, width=72, layers=[("gla", GLA, 100), ("attention", ATT, (24, 5, 2, 56)),
                                             ("parallel", PAR, (40, 7, 3, 0)), ("attention", ATT, None)], eps=1e-5)
    base.update(kw)
    return make_config(**base)


def test_configuration_reads_every_key_and_writes_it_back():
    d = config()
    cfg = registry.config_from_dict(d)
    assert isinstance(cfg, LudelixConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps, cfg.num_hidden_layers, cfg.hidden_size) == (211, 72, 1e-5, 4, 72)
    g, a, p = cfg.layers[0].mixer, cfg.layers[1].mixer, cfg.layers[2].mixer
    assert (g.heads, g.dim, g.vdim, g.tau, g.rank) == (3, 24, 40, 6.0, 5)
    assert (a.heads, a.kv_heads, a.dim, a.scale, a.window) == (6, 2, 24, 0.3, 21)
    assert (a.rot.dims, a.rot.base, a.rot.pairs) == (10, 5000.0, "neighbours")
    assert (a.rot.scaling.factor, a.rot.scaling.low, a.rot.scaling.high, a.rot.scaling.original) == (3.0, 1.0, 3.0, 40)
    lt, rt = p.left, p.right
    assert (lt.heads, lt.kv_heads, lt.dim, lt.vdim, lt.scale, lt.chunk, lt.rot.pairs) == (4, 2, 20, 28, 0.2, 17, "halves")
    assert (lt.rot.scaling.factor, lt.rot.scaling.original, lt.rot.scaling.fast, lt.rot.scaling.slow) == (5.0, 50, 8.0, 0.5)
    assert (rt.heads, rt.dim, rt.vdim, rt.decay, rt.rot.dims, rt.rot.scaling) == (3, 12, 20, (0.9, 0.97, 0.995), 8, None)
    assert (p.left_scale, p.right_scale) == (0.8, 1.7)
    m0, m1, m2 = (cfg.layers[i].mlp for i in range(3))
    assert (m0.kind, m0.ff) == ("dense", 100)
    assert (m1.kind, m1.ff, m1.experts, m1.top, m1.shared_ff) == ("moe", 24, 5, 2, 56)
    assert m2.shared_ff == 0 and cfg.layers[3].mlp is None
    assert registry.config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    for name in ("ludelix-tiny", "ludelix-1b"):
        registry.build_spec(registry.config_from_dict(PRESETS[name]))


def test_what_a_file_may_leave_out():
    d = config()
    del d["layers"][0]["mixer"]["rank"]                  # the checkpoint's tensors decide
    for key in ("rot", "mask"):
        del d["layers"][1]["mixer"][key]
    del d["layers"][1]["mixer"]["kv_heads"]
    del d["layers"][2]["mixer"]["left"]["rot"]["scaling"]
    del d["layers"][2]["mixer"]["left"]["mask"]
    del d["layers"][2]["mixer"]["right"]["rot"]
    cfg = registry.config_from_dict(d)
    assert cfg.layers[0].mixer.rank is None
    a = cfg.layers[1].mixer
    assert (a.kv_heads, a.window, a.rot) == (6, None, None)
    assert cfg.layers[2].mixer.left.rot.scaling is None and cfg.layers[2].mixer.left.chunk is None
    assert cfg.layers[2].mixer.right.rot is None
    assert cfg.max_position_embeddings == 131072
    spec = registry.build_spec(cfg)
    assert spec.weight_specs()["l0.mix.a1"].shape == (None, 72)
    with pytest.raises(ValueError, match="only a checkpoint decides"):
        random_tensors(spec, 0)


@pytest.mark.parametrize("change,match", [
    (lambda d: d["layers"][0].update(type="mamba"), "not supported"),
    (lambda d: d["layers"][0]["mlp"].update(kind="glu"), "not supported"),
    (lambda d: d["layers"][1]["mixer"].update(vdim=32), "values are the keys"),
    (lambda d: d["layers"][1]["mixer"].update(kv_heads=4), "multiple of kv_heads"),
    (lambda d: d["layers"][1]["mixer"]["rot"].update(dims=26), "exceeds the head size"),
    (lambda d: d["layers"][1]["mixer"]["rot"].update(dims=7), "must be even"),
    (lambda d: d["layers"][1]["mixer"]["rot"]["scaling"].update(high=1.0), "must exceed"),
    (lambda d: d["layers"][1]["mlp"]["router"].update(top=6), "exceeds the 5 experts"),
    (lambda d: d["layers"][2]["mixer"]["right"].update(decay=[0.9, 0.9]), "one number per head"),
    (lambda d: d["layers"][2]["mixer"]["right"]["rot"].update(scaling={"factor": 2.0}), "takes no scaling"),
    (lambda d: d["layers"][2]["mixer"].pop("left_scale"), "left_scale"),
    (lambda d: d["layers"][0]["mixer"].update(tau=0.0), "positive"),
    (lambda d: d.update(layers=[]), "at least one layer"),
    (lambda d: d.pop("norm"), "norm"),
])
def test_refusals(change, match):
    d = copy.deepcopy(config())
    change(d)
    with pytest.raises((ConfigError, KeyError), match=match):
        registry.build_spec(registry.config_from_dict(d))


def test_parts_refuse_what_their_kernels_do_not_compute():
    with pytest.raises(ValueError, match="one of the two"):
        LinearMemory("m", 32, 2, 16, 16, 1e-5)
    with pytest.raises(ValueError, match="one number per head"):
        LinearMemory("m", 32, 2, 16, 16, 1e-5, head_decays=[0.9])
    with pytest.raises(ValueError, match="up to 256"):
        LinearMemory("m", 32, 2, 300, 16, 1e-5, gate_tau=2.0)
    with pytest.raises(ValueError, match="go with row_norm"):
        PagedAttention("a", 32, 2, 1, 16, None, values_are_keys=True)
    with pytest.raises(ValueError, match="place of a window"):
        PagedAttention("a", 32, 2, 1, 16, None, window=8, chunk=8)
    att = PagedAttention("a", 32, 2, 1, 16, None)
    with pytest.raises(ValueError, match="only one of them may keep pages"):
        MixerPair(att, PagedAttention("b", 32, 2, 1, 16, None))
    mem = LinearMemory("m", 32, 2, 16, 16, 1e-5, head_decays=[0.9, 0.8])
    with pytest.raises(ValueError, match="only one of them may keep a state"):
        MixerPair(mem, LinearMemory("n", 32, 2, 16, 16, 1e-5, head_decays=[0.9, 0.8]))
    with pytest.raises(ValueError, match="no identity outputs"):
        RoutedExperts("f", 32, 16, 4, 2, identity=1, table_vocab=10)


def test_tensor_names_and_parts_per_layer():
    spec = registry.build_spec(registry.config_from_dict(config()))
    names = spec.weight_specs()
    sh = lambda n: names[n].shape  # noqa: E731
    assert sh("embed") == (211, 72) and sh("final.norm") == (72,) and "head" not in names
    assert sh("l0.mix.q") == (72, 72) and sh("l0.mix.v") == (120, 72) and sh("l0.mix.g") == (120, 72)
    assert sh("l0.mix.o") == (72, 120) and sh("l0.mix.norm") == (40,)
    assert sh("l0.mix.a1") == (5, 72) and sh("l0.mix.a2") == (72, 5) and sh("l0.mix.a2.b") == (72,)
    assert sh("l0.mlp.up") == (100, 72) and sh("l0.mlp.down") == (72, 100)
    assert sh("l1.mix.q") == (144, 72) and sh("l1.mix.k") == (48, 72) and "l1.mix.v" not in names
    assert sh("l1.mix.q.b") == (144,) and sh("l1.mix.k.b") == (48,)
    assert sh("l1.mix.q.norm") == (144,) and sh("l1.mix.k.norm") == (48,) and sh("l1.mix.sink") == (6,)
    assert sh("l1.mix.o") == (72, 144)
    assert sh("l1.mlp.e4.gate") == (24, 72) and sh("l1.mlp.e4.down") == (72, 24) and "l1.mlp.e5.up" not in names
    assert sh("l1.mlp.table") == (211, 2) and names["l1.mlp.table"].integer and "l1.mlp.router" not in names
    assert sh("l1.mlp.shared.up") == (56, 72) and sh("l1.mlp.shared.sg") == (1, 72)
    assert sh("l2.mix.left.q") == (80, 72) and sh("l2.mix.left.k") == (40, 72) and sh("l2.mix.left.v") == (56, 72)
    assert sh("l2.mix.left.g") == (4, 72) and sh("l2.mix.left.o") == (72, 112)
    assert sh("l2.mix.right.q") == (36, 72) and sh("l2.mix.right.v") == (60, 72) and sh("l2.mix.right.g") == (60, 72)
    assert sh("l2.mix.right.o") == (72, 60) and "l2.mix.right.norm" not in names
    assert sh("l2.mlp.table") == (211, 3) and "l2.mlp.shared.gate" not in names
    assert "l3.norm2" not in names and "l3.norm1" in names
    b = spec.blocks
    assert all(isinstance(x, PreNormBlock) and isinstance(x.mixer_norm, NamedRMSNorm) for x in b)
    assert isinstance(b[0].mixer, LinearMemory) and isinstance(b[0].ffn, PlainFeedForward)
    assert isinstance(b[1].mixer, PagedAttention) and isinstance(b[1].ffn, RoutedExperts)
    assert isinstance(b[2].mixer, MixerPair) and isinstance(b[2].mixer.left, PagedAttention)
    assert isinstance(b[2].mixer.right, LinearMemory) and b[3].ffn is None
    assert b[1].mixer.rotary is b[3].mixer.rotary and len(spec.positions) == 3        # equal rotations share tables
    assert b[1].mixer.rotary.interleaved and not b[2].mixer.left.rotary.interleaved


def test_cache_groups_and_state_slots():
    cfg = registry.config_from_dict(config())
    model = Transformer(registry.build_spec(cfg), torch.float32, "cpu")
    # the two windowed layers share a group; the chunked one keeps other pages
    assert len(model.cache_groups) == 2
    windows = sorted(g.window for g in model.cache_groups)
    assert windows == [17, 21]
    # the first layer's memory and the retention beside the chunked attention
    assert sorted(model.state_specs) == [0, 2]
    assert model.state_specs[0].shape == (3 * 24 * 40,) and model.state_specs[2].shape == (3 * 12 * 20,)


def test_a_table_of_random_choices_holds_different_experts():
    spec = registry.build_spec(registry.config_from_dict(config()))
    t = random_tensors(spec, 3)["l2.mlp.table"]
    assert t.dtype == torch.int32 and t.shape == (211, 3) and int(t.min()) >= 0 and int(t.max()) < 7
    assert all(len(set(row)) == 3 for row in t.tolist())
    assert len({tuple(r) for r in t.tolist()}) > 20


# ---------------------------------------------------------------------------- mechanisms by hand
def test_frequencies_scaled_by_wavelength():
    f = plain.wavelength_frequencies(8, 10.0, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40})
    base = [10.0 ** (-2.0 * i / 8) for i in range(4)]
    # wavelengths 6.3, 11.2, 19.9, 35.3: below 10 kept; above 40 none; between blended by 40 / wavelength
    assert abs(float(f[0]) - base[0]) < 1e-12
    for i in (1, 2, 3):
        s = (40.0 / (2 * math.pi / base[i]) - 1.0) / 3.0
        assert abs(float(f[i]) - ((1 - s) * base[i] / 4.0 + s * base[i])) < 1e-12
    g = plain.wavelength_frequencies(8, 10000.0, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40})
    assert abs(float(g[3]) - 10000.0 ** -0.75 / 4.0) < 1e-15           # a wave of 6,283 positions is slowed
    from kvforge_amd.config.model import RopeScaling
    from kvforge_amd.parts.positions import scaled_inv_freq
    mine = scaled_inv_freq(8, 10.0, RopeScaling("llama3", 4.0, 1.0, 4.0, 40))
    torch.testing.assert_close(mine.double(), f, atol=1e-7, rtol=1e-6)


def test_yarn_frequencies_and_magnitude():
    f, mag = plain.yarn_frequencies(8, 100.0, {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 1.0})
    idx = lambda t: 8 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(100.0))  # noqa: E731
    lo, hi = max(math.floor(idx(4.0)), 0), min(math.ceil(idx(1.0)), 7)
    assert (lo, hi) == (0, 3)
    for i in range(4):
        ramp = min(max((i - lo) / (hi - lo), 0.0), 1.0)
        b = 100.0 ** (-2.0 * i / 8)
        assert abs(float(f[i]) - (b / 8.0 * ramp + b * (1 - ramp))) < 1e-12
    assert abs(mag - (0.1 * math.log(8.0) + 1.0)) < 1e-12


def test_the_two_ways_of_pairing():
    x = torch.arange(1.0, 9.0).view(1, 1, 8)
    f = torch.tensor([math.pi / 2, math.pi], dtype=torch.float64)             # at position 1: a quarter and a half turn
    pos = torch.tensor([1])
    n = plain.turn(x, pos, f, 1.0, True)[0, 0]
    torch.testing.assert_close(n, torch.tensor([-2.0, 1.0, -3.0, -4.0, 5.0, 6.0, 7.0, 8.0]), atol=1e-5, rtol=0)
    h = plain.turn(x, pos, f, 2.0, False)[0, 0]                               # (1, 3) and (2, 4), everything doubled
    torch.testing.assert_close(h, torch.tensor([-6.0, -4.0, 2.0, -8.0, 5.0, 6.0, 7.0, 8.0]), atol=1e-5, rtol=0)


def test_window_and_chunks():
    w = plain.window_mask(6, 3)
    assert w[5].tolist() == [False, False, False, True, True, True] and w[1].tolist() == [True, True] + [False] * 4
    c = plain.chunk_mask(7, 3)
    assert c[2].tolist() == [True, True, True, False, False, False, False]
    assert c[3].tolist() == [False, False, False, True, False, False, False]         # a chunk's first sees itself alone
    assert c[6].tolist() == [False] * 6 + [True]


def test_the_sink_counts_once_and_has_no_value():
    q, k, v = torch.ones(1, 1, 2), torch.ones(1, 1, 2), torch.tensor([[[3.0, 5.0]]])
    o = plain.softmax_attention(q, k, v, 0.5, torch.ones(1, 1, dtype=torch.bool), torch.tensor([1.0]))
    torch.testing.assert_close(o[0, 0], v[0, 0] * 0.5)           # exp(1) / (exp(1) + exp(1))
    o = plain.softmax_attention(q, k, v, 0.5, torch.ones(1, 1, dtype=torch.bool), None)
    torch.testing.assert_close(o[0, 0], v[0, 0])


def test_two_tokens_of_the_memory():
    q = torch.tensor([[[1.0, 2.0]], [[3.0, -1.0]]])
    k = torch.tensor([[[0.5, 1.0]], [[2.0, 0.0]]])
    v = torch.tensor([[[1.0, 10.0, 100.0]], [[2.0, 0.0, -1.0]]])
    a = torch.tensor([[[0.5, 0.25]], [[0.1, 0.5]]])
    o = plain.decay_scan(q, k, v, a)
    # S_0 = k_0 v_0^T (the first decay meets zeros); o_0 = (q_0 . k_0) v_0
    torch.testing.assert_close(o[0, 0], 2.5 * v[0, 0])
    # S_1 = diag(a_1) S_0 + k_1 v_1^T; o_1 = sum_i q_i (a_i k0_i v_0 + k1_i v_1)
    want = (3.0 * 0.1 * 0.5 - 1.0 * 0.5 * 1.0) * v[0, 0] + (3.0 * 2.0) * v[1, 0]
    torch.testing.assert_close(o[1, 0], want)
    const = plain.decay_scan(q, k, v, torch.tensor([[0.5]]))
    torch.testing.assert_close(const[1, 0], (3.0 * 0.5 * 0.5 - 1.0 * 0.5 * 1.0) * v[0, 0] + 6.0 * v[1, 0])


def test_gates_become_decays():
    w = {"m.a1": torch.tensor([[1.0, 0.0], [0.0, 2.0]]), "m.a2": torch.tensor([[1.0, 1.0], [0.0, -1.0]]),
         "m.a2.b": torch.tensor([0.5, 0.0])}
    a = plain.gla_decay(torch.tensor([[1.0, 1.0]]), w, "m.", 4.0)
    z = torch.tensor([1.0 + 2.0 + 0.5, -2.0])
    torch.testing.assert_close(a[0], torch.sigmoid(z) ** 0.25)


def test_a_table_names_the_experts_and_the_shared_one_is_gated():
    torch.manual_seed(0)
    h = torch.randn(3, 4)
    w = {f"f.e{e}.{n}": torch.randn(*s) for e in range(3) for n, s in (("gate", (5, 4)), ("up", (5, 4)), ("down", (4, 5)))}
    w.update({"f.shared.gate": torch.randn(6, 4), "f.shared.up": torch.randn(6, 4), "f.shared.down": torch.randn(4, 6),
              "f.shared.sg": torch.randn(1, 4), "f.table": torch.tensor([[0, 1], [2, 0], [1, 2], [2, 1]], dtype=torch.int32)})
    mlp = {"router": {"experts": 3, "top": 2}, "shared": {"ff": 6}}
    toks = torch.tensor([3, 0, 3])
    got = plain.table_ff(h, toks, w, "f.", mlp)
    for t, (e1, e2) in enumerate([(2, 1), (0, 1), (2, 1)]):
        want = 0.5 * (plain.expert(h[t:t + 1], w, f"f.e{e1}.") + plain.expert(h[t:t + 1], w, f"f.e{e2}."))[0]
        want = want + torch.sigmoid(h[t] @ w["f.shared.sg"][0]) * plain.expert(h[t:t + 1], w, "f.shared.")[0]
        torch.testing.assert_close(got[t], want, atol=1e-5, rtol=1e-5)


def test_the_plain_model_runs_and_its_layers_matter():
    d = PRESETS["ludelix-tiny"]
    spec = registry.build_spec(registry.config_from_dict(d))
    w = {k: v.float() * (3.0 if v.is_floating_point() and v.dim() == 2 and k != "embed" else 1.0)
         for k, v in random_tensors(spec, 1).items()}
    toks = [5, 9, 200, 31, 7, 7, 100, 2] * 6
    layers = []
    logits = plain.forward(d, w, toks, layers_out=layers)
    assert logits.shape == (48, 320) and len(layers) == 3 and bool(torch.isfinite(logits).all())
    other = plain.forward(d, w, [6] + toks[1:])
    assert float((logits[-1] - other[-1]).abs().max()) > 1e-6         # the memories carry the first token on
    assert len(plain.greedy(d, w, toks[:5], 3)) == 3
