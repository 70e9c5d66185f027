"""Buzinex without a GPU: configuration and its refusals, the builder's tensor names, cache
groups and state slots, and the plain model's mechanisms worked by hand."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from kvforge_amd import registry
from kvforge_amd.config import BuzinexConfig, ConfigError
from kvforge_amd.config.presets import PRESETS, buzinex as make_config
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts import (DecayMemory, GatedFeedForward, LatentAttention, NamedRMSNorm, PagedAttention,
                               SandwichBlock)
from tests.plain import buzinex as plain

ATT = dict(heads=6, kv_heads=2, dim=24, vdim=40, scale=0.2, softcap=12.0, q_temp=(0.4, 5))
LAT = dict(heads=3, dim=20, rot_dim=12, vdim=28, kv_rank=36, scale=0.15, window=19, base=5000.0)
REC = dict(heads=3, dim=16, decay_rank=6)


def config(**kw):
    base = dict(vocab=211, width=72, layers=[("attention", ATT, 88), ("latent_attention", LAT, 40), ("wkv", REC, None),
                                             ("latent_attention", LAT, None)],
                embedding_scale=6.5, logit_scale=0.3, logit_softcap=20.0, eps=1e-5)
    base.update(kw)
    return make_config(**base)


def random_weights(d, seed=0):
    spec = registry.build_spec(registry.config_from_dict(d))
    g = torch.Generator().manual_seed(seed)
    return {k: (torch.randn(s.shape, generator=g) * s.std + (1.0 if s.init == "norm" else 0.0)).bfloat16()
            for k, s in sorted(spec.weight_specs().items())}


def test_configuration_reads_every_key_and_writes_it_back():
    d = config()
    cfg = registry.config_from_dict(d)
    assert isinstance(cfg, BuzinexConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps, cfg.embedding_scale) == (211, 72, 1e-5, 6.5)
    assert (cfg.logit_scale, cfg.logit_softcap, cfg.num_hidden_layers, cfg.hidden_size) == (0.3, 20.0, 4, 72)
    a, l, r = cfg.layers[0].mixer, cfg.layers[1].mixer, cfg.layers[2].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.softcap, a.window) == (6, 2, 24, 40, 0.2, 12.0, None)
    assert (a.q_temp.coef, a.q_temp.every) == (0.4, 5)
    assert (l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank, l.scale, l.window) == (3, 20, 12, 28, 36, 0.15, 19)
    assert (l.rot.dims, l.rot.base) == (12, 5000.0)
    assert (r.heads, r.dim, r.decay_rank) == (3, 16, 6)
    assert cfg.layers[0].mlp.ff == 88 and cfg.layers[2].mlp is None and cfg.layers[3].mlp is None
    assert registry.config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    for name in ("buzinex-tiny", "buzinex-1b"):
        registry.build_spec(registry.config_from_dict(PRESETS[name]))


def test_what_a_file_may_leave_out():
    d = config()
    m = d["layers"][0]["mixer"]
    del m["kv_heads"], m["vdim"], m["q_temp"], m["softcap"]
    d["layers"][1]["mixer"]["mask"] = None
    del d["layers"][2]["mixer"]["decay_rank"]
    del d["embedding"], d["logit_softcap"], d["logit_scale"]
    cfg = registry.config_from_dict(d)
    a = cfg.layers[0].mixer
    assert (a.kv_heads, a.vdim, a.q_temp, a.softcap) == (6, 24, None, None)
    assert cfg.layers[1].mixer.window is None and cfg.layers[2].mixer.decay_rank is None
    assert (cfg.embedding_scale, cfg.logit_scale, cfg.logit_softcap) == (1.0, 1.0, None)
    # the rank of the decay's two matrices is then the checkpoint's to say
    spec = registry.build_spec(cfg)
    assert spec.weight_specs()["l2.mix.w1"].shape == (None, 72)


@pytest.mark.parametrize("change,complaint", [
    (lambda d: d["layers"][0].update(type="conv"), "mixer type"),
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=4), "multiple"),
    (lambda d: d["layers"][0]["mixer"]["q_temp"].update(every=0), "every"),
    (lambda d: d["layers"][1]["mixer"]["rot"].update(dims=14), "exceeds"),
    (lambda d: d["layers"][1]["mixer"].update(kv_rank=0), "kv_rank"),
    (lambda d: d["layers"][1]["mixer"].update(kv_rank=250), "256"),
    (lambda d: d["layers"][1]["mixer"]["mask"].update(size=0), "size"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda d: d["layers"][2]["mixer"].update(dim=300), "256"),
    (lambda d: d.pop("width"), "width"),
    (lambda d: d.update(layers=[]), "layer"),
])
def test_refusals(change, complaint):
    d = copy.deepcopy(config())
    change(d)
    with pytest.raises(ConfigError, match=complaint):
        registry.config_from_dict(d)


def test_builder_names_every_tensor_and_chooses_parts_per_layer():
    spec = registry.build_spec(registry.config_from_dict(config()))
    names = spec.weight_specs()
    assert {"embed", "final.norm", "l0.norm1", "l0.norm1b", "l0.norm2", "l0.norm2b", "l2.norm1b"} <= set(names)
    assert "head" not in names and "l2.norm2" not in names and "l3.mlp.up" not in names
    assert names["l0.mix.q"].shape == (6 * 24, 72) and names["l0.mix.k"].shape == (2 * 24, 72)
    assert names["l0.mix.v"].shape == (2 * 40, 72) and names["l0.mix.o"].shape == (72, 6 * 40)
    assert names["l0.mix.q.norm"].shape == (24,) and names["l0.mix.k.norm"].shape == (24,)
    assert "l0.mix.sink" not in names
    assert names["l1.mix.q"].shape == (3 * 32, 72) and names["l1.mix.dkv"].shape == (36 + 12, 72)
    assert names["l1.mix.dkv.norm"].shape == (36,) and names["l1.mix.sink"].shape == (3,)
    assert names["l1.mix.uk"].shape == (3 * 20, 36) and names["l1.mix.uv"].shape == (3 * 28, 36)
    assert names["l1.mix.o"].shape == (72, 3 * 28)
    for s in ("r", "k", "v", "g"):
        assert names[f"l2.mix.{s}"].shape == (48, 72) and names[f"l2.mix.mu.{s}"].shape == (72,)
    assert names["l2.mix.w1"].shape == (6, 72) and names["l2.mix.w2"].shape == (48, 6)
    assert names["l2.mix.w0"].shape == (48,) and names["l2.mix.u"].shape == (3, 16)
    assert names["l2.mix.norm"].shape == (48,) and names["l2.mix.o"].shape == (72, 48)
    assert names["l0.mlp.gate"].shape == (88, 72) and names["l1.mlp.down"].shape == (72, 40)
    kinds = [(type(b), type(b.mixer), type(b.ffn)) for b in spec.blocks]
    assert kinds == [(SandwichBlock, PagedAttention, GatedFeedForward), (SandwichBlock, LatentAttention, GatedFeedForward),
                     (SandwichBlock, DecayMemory, type(None)), (SandwichBlock, LatentAttention, type(None))]
    assert all(isinstance(p, NamedRMSNorm) for b in spec.blocks for p in (b.pre, b.post))
    assert spec.blocks[1].mixer.rotary is spec.blocks[3].mixer.rotary    # equal rotations share tables
    assert spec.blocks[0].mixer.rotary is None


def test_caches_hold_one_key_per_token_and_states_one_slot_per_request():
    spec = registry.build_spec(registry.config_from_dict(config()))
    model = Transformer(spec, torch.float32, "cpu")
    assert sorted(model.state_specs) == [2]
    assert model.state_specs[2].shape == (3 * 16 * 16 + 72,)               # every head's memory, the last input row
    full, latent = model.cache_groups
    assert full.layers == (0,) and full.window is None
    assert latent.layers == (1, 3) and latent.window == 19
    (k, v) = latent.pages                                                  # rot_dim + kv_rank, whatever the heads
    assert k.shape == (1, "block", 48) and v.shape == (1, 48, "block")


def test_query_temperature_by_hand():
    t = plain.query_temperature(torch.tensor([0, 3, 4, 8, 9, 14, 499]), 0.4, 5)
    want = [1.0, 1.0, 1 + 0.4 * math.log(2), 1 + 0.4 * math.log(2), 1 + 0.4 * math.log(3), 1 + 0.4 * math.log(4),
            1 + 0.4 * math.log(101)]
    torch.testing.assert_close(t, torch.tensor(want))
    assert float(plain.capped(torch.tensor(1e6), 15.0)) == pytest.approx(15.0)
    assert float(plain.capped(torch.tensor(0.3), 15.0)) == pytest.approx(15.0 * math.tanh(0.02))
    assert float(plain.capped(torch.tensor(7.0), None)) == 7.0


def test_rotation_turns_neighbouring_pairs_and_leaves_the_rest():
    x = torch.arange(1.0, 13.0).view(1, 2, 6).repeat(3, 1, 1)
    y = plain.rotate_pairs(x, torch.tensor([0, 1, 5]), 4, 10.0)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    a = 5 * 10.0 ** -0.5                                           # pair 1 at position 5
    assert float(y[2, 0, 2]) == pytest.approx(3 * math.cos(a) - 4 * math.sin(a), rel=1e-5)
    assert float(y[2, 0, 3]) == pytest.approx(4 * math.cos(a) + 3 * math.sin(a), rel=1e-5)
    assert float(y[1, 1, 0]) == pytest.approx(7 * math.cos(1.0) - 8 * math.sin(1.0), rel=1e-5)


def test_sink_takes_weight_and_gives_nothing_and_the_window_counts_the_query():
    q, k = torch.zeros(2, 1, 4), torch.zeros(2, 1, 4)
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]])
    o = plain.attend(q, k, v, 1.0, plain.visible_keys(2, 2), None, torch.tensor([0.0]))
    # scores 0 everywhere: position 0 shares with the sink, position 1 with one key more
    torch.testing.assert_close(o[:, 0], torch.tensor([[0.5, 0.0], [1 / 3, 1 / 3]]))
    o = plain.attend(q, k, v, 1.0, plain.visible_keys(2, 2), None, torch.tensor([-1e9]))
    torch.testing.assert_close(o[:, 0], torch.tensor([[1.0, 0.0], [0.5, 0.5]]))
    assert plain.visible_keys(5, 5, 2).int().tolist()[3] == [0, 0, 1, 1, 0]
    assert plain.visible_keys(2, 5, 3).int().tolist() == [[0, 1, 1, 1, 0], [0, 0, 1, 1, 1]]
    assert plain.visible_keys(1, 4, None).int().tolist() == [[1, 1, 1, 1]]


def test_latent_keys_are_read_out_per_head_and_the_rotated_part_is_shared():
    """One head pair whose read-outs differ: the same latent gives them different keys, while
    the rotated part scores alike for both."""
    m = {"heads": 2, "dim": 2, "rot_dim": 2, "vdim": 1, "kv_rank": 2, "scale": 1.0, "mask": None,
         "rot": {"dims": 2, "base": 10.0}}
    big = 1e4
    w = {"p.q": torch.tensor([[1.0, 0.0], [0.0, 0.0], [0.0, 0.0], [0.0, 0.0],      # head 0: plain (h0, 0), no rotated part
                              [1.0, 0.0], [0.0, 0.0], [0.0, 0.0], [0.0, 0.0]]),
         "p.dkv": torch.tensor([[1.0, 0.0], [0.0, 1.0], [0.0, 0.0], [0.0, 0.0]]),    # latent = h, no shared key part
         "p.dkv.norm": torch.ones(2),
         "p.uk": torch.tensor([[big, 0.0], [0.0, 0.0], [0.0, big], [0.0, 0.0]]),     # head 0 reads c0, head 1 reads c1
         "p.uv": torch.tensor([[1.0, 0.0], [1.0, 0.0]]),
         "p.sink": torch.tensor([-1e9, -1e9]), "p.o": torch.eye(2)}
    h = torch.tensor([[1.0, 0.1], [0.1, 1.0], [1.0, 1.0]])
    o = plain.latent_attention(h, w, "p.", m, 0.0)
    c = plain.rms(h, 0.0)
    # the last query: head 0 takes the token whose c0 is largest (token 0), head 1 token 1
    torch.testing.assert_close(o[2], torch.stack([c[0, 0], c[1, 0]]), atol=1e-5, rtol=1e-5)


def test_matrix_memory_first_steps_by_hand():
    r = torch.tensor([[[1.0, 2.0]], [[3.0, 1.0]], [[1.0, 1.0]]])
    k = torch.tensor([[[2.0, 1.0]], [[1.0, 1.0]], [[0.0, 2.0]]])
    v = torch.tensor([[[3.0, 1.0]], [[5.0, 2.0]], [[1.0, 1.0]]])
    w = torch.tensor([[[0.5, 0.25]], [[0.5, 1.0]], [[0.1, 0.1]]])
    u = torch.tensor([[2.0, 0.5]])
    o = plain.wkv_recurrence(r, k, v, w, u)
    # token 0: only the bonus, sum_i r_i u_i k_i = 1*2*2 + 2*0.5*1 = 5, times v
    torch.testing.assert_close(o[0, 0], torch.tensor([15.0, 5.0]))
    # token 1: S = k0 v0^T (token 0's decay never touches what token 0 wrote); r1 . S = (3*2 + 1*1) v0 = 7 v0
    # bonus 3*2*1 + 1*0.5*1 = 6.5, times v1
    torch.testing.assert_close(o[1, 0], torch.tensor([7 * 3.0 + 6.5 * 5.0, 7 * 1.0 + 6.5 * 2.0]))
    # token 2: S = diag(w1) k0 v0^T + k1 v1^T; r2 = (1, 1): (0.5*2 + 1*1) v0 + (1 + 1) v1; bonus 0 + 1*0.5*2 = 1
    torch.testing.assert_close(o[2, 0], torch.tensor([2 * 3.0 + 2 * 5.0 + 1.0, 2 * 1.0 + 2 * 2.0 + 1.0]))
    assert torch.equal(plain.shifted(torch.tensor([[1.0], [2.0], [3.0]])), torch.tensor([[0.0], [1.0], [2.0]]))


def test_a_layer_norms_what_a_sublayer_gives_before_it_joins_the_stream():
    d = config(layers=[("wkv", REC, 24)])
    w = random_weights(d, 3)
    toks = [5, 9, 200, 9]
    layers: list = []
    plain.forward(d, w, toks, layers_out=layers)
    wf = {k: v.float() for k, v in w.items()}
    x0 = wf["embed"][toks] * 6.5
    y = plain.wkv(plain.norm(x0, wf["l0.norm1"], 1e-5), wf, "l0.mix.", d["layers"][0]["mixer"], 1e-5)
    x1 = x0 + plain.norm(y, wf["l0.norm1b"], 1e-5)
    z = plain.dense_ff(plain.norm(x1, wf["l0.norm2"], 1e-5), wf, "l0.mlp.")
    torch.testing.assert_close(layers[0], x1 + plain.norm(z, wf["l0.norm2b"], 1e-5))


def test_bfloat16_roundings_of_the_plain_model_stay_small():
    d = config()
    w = random_weights(d)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, 211, (30,), generator=g).tolist()
    layers: list = []
    a = plain.forward(d, w, toks, layers_out=layers)
    b = plain.forward(d, w, toks, store=torch.bfloat16)
    assert len(layers) == 4 and a.shape == (30, 211)
    assert float((a - b).abs().max()) < 0.1 * float(a.std()) and not torch.equal(a, b)
    assert float(a.abs().max()) <= 20.0                              # capped
    # logits from the table itself, without the embedding's scale
    x = plain.norm(layers[-1], w["final.norm"].float(), 1e-5)
    torch.testing.assert_close(a, plain.capped(x @ w["embed"].float().T * 0.3, 20.0))
    two = plain.greedy(d, w, toks[:3], 2)
    assert two[0] == int(plain.forward(d, w, toks[:3])[-1].argmax())
    assert two[1] == int(plain.forward(d, w, toks[:3] + two[:1])[-1].argmax())
