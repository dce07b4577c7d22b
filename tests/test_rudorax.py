"""Rudorax without a GPU: configuration and its refusals, the builder's tensor names, cache
groups and state slots of looped layers, and the plain model's mechanisms worked by hand."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from kvforge_amd import registry
from kvforge_amd.config import ConfigError, RudoraxConfig
from kvforge_amd.config.presets import PRESETS, rudorax as make_config
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts import MatrixLSTM, PagedAttention, RoutedExperts
from kvforge_amd.parts.positions import RotaryPositions, YarnStretch
from tests.plain import rudorax as plain

ATT = dict(heads=6, kv_heads=2, dim=24, vdim=40, window=19, rot_dims=12, scale=0.2,
           scaling={"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0})
REC = dict(heads=3, dim=16, vdim=24, gate_cap=8.0)
MOE = dict(ff=24, experts=5, top=2, identity=2, shared_ff=40)


def config(**kw):
    base = dict(vocab=211, width=72, layers=[("attention", ATT, MOE), ("mlstm", REC, MOE), ("attention", ATT, None)],
                loop=(1, 3, 2), embedding_scale=6.5, logit_softcap=20.0, eps=1e-5)
    base.update(kw)
    return make_config(**base)


def test_configuration_reads_every_key_and_writes_it_back():
    d = config()
    cfg = registry.config_from_dict(d)
    assert isinstance(cfg, RudoraxConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps, cfg.embedding_scale, cfg.logit_softcap) == (211, 72, 1e-5, 6.5, 20.0)
    a, r = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.scale) == (6, 2, 24, 40, 19, 0.2)
    assert (a.rot.dims, a.rot.base, a.rot.scaling.factor, a.rot.scaling.original) == (12, 10000.0, 4.0, 16)
    assert (r.heads, r.dim, r.vdim, r.gate_cap) == (3, 16, 24, 8.0)
    m = cfg.layers[0].mlp
    assert (m.ff, m.experts, m.top, m.identity, m.shared_ff) == (24, 5, 2, 2, 40)
    assert cfg.layers[2].mlp is None
    assert cfg.run_order() == [0, 1, 2, 1, 2] == plain.run_order(d)
    assert registry.config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    for name in ("rudorax-tiny", "rudorax-1b"):
        registry.build_spec(registry.config_from_dict(PRESETS[name]))


def test_what_a_file_may_leave_out():
    d = config(loop=None, logit_softcap=None)
    m = d["layers"][0]["mixer"]
    del m["kv_heads"], m["vdim"]
    m["rot"]["scaling"] = None
    d["layers"][1]["mlp"]["shared"] = None
    d["layers"][1]["mlp"]["router"].pop("identity")
    del d["embedding"], d["loop"], d["logit_softcap"]
    cfg = registry.config_from_dict(d)
    a = cfg.layers[0].mixer
    assert (a.kv_heads, a.vdim, a.rot.scaling) == (6, 24, None)
    assert (cfg.layers[1].mlp.shared_ff, cfg.layers[1].mlp.identity) == (0, 0)
    assert cfg.embedding_scale == 1.0 and cfg.loop is None and cfg.logit_softcap is None
    assert cfg.run_order() == [0, 1, 2]


@pytest.mark.parametrize("change,complaint", [
    (lambda d: d["layers"][0].update(type="conv"), "mixer type"),
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=4), "multiple"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=26), "exceeds"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=11), "even"),
    (lambda d: d["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda d: d["layers"][0]["mlp"]["router"].update(top=8), "exceeds"),
    (lambda d: d["layers"][1]["mixer"].update(gate_cap=0.0), "gate_cap"),
    (lambda d: d["loop"].update(stop=4), "loop"),
    (lambda d: d["loop"].update(times=0), "loop"),
    (lambda d: d.pop("width"), "width"),
])
def test_refusals(change, complaint):
    d = copy.deepcopy(config())
    change(d)
    with pytest.raises(ConfigError, match=complaint):
        registry.config_from_dict(d)


def test_builder_names_every_tensor_and_chooses_parts_per_layer():
    spec = registry.build_spec(registry.config_from_dict(config()))
    names = spec.weight_specs()
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l2.norm1"} <= set(names)
    assert "l2.norm2" not in names                                     # no feed-forward there
    assert names["l0.mix.q"].shape == (6 * 24, 72) and names["l0.mix.k"].shape == (2 * 24, 72)
    assert names["l0.mix.v"].shape == (2 * 40, 72) and names["l0.mix.o"].shape == (72, 6 * 40)
    assert names["l0.mix.q.norm"].shape == (24,) and names["l0.mix.sink"].shape == (6,)
    assert names["l1.mix.q"].shape == (3 * 16, 72) and names["l1.mix.v"].shape == (3 * 24, 72)
    assert names["l1.mix.i"].shape == (3, 72) and names["l1.mix.f.b"].shape == (3,)
    assert names["l1.mix.norm"].shape == (3 * 24,)
    assert names["l0.mlp.router"].shape == (7, 72) and names["l0.mlp.correction"].shape == (7,)
    assert names["l0.mlp.e4.down"].shape == (72, 24) and "l0.mlp.e5.gate" not in names
    assert names["l0.mlp.shared.gate"].shape == (40, 72)
    kinds = [(type(b.mixer), type(b.ffn)) for b in spec.blocks]
    assert kinds == [(PagedAttention, RoutedExperts), (MatrixLSTM, RoutedExperts), (PagedAttention, type(None))]
    assert spec.blocks[0].mixer.rotary is spec.blocks[2].mixer.rotary    # equal rotations share tables
    assert spec.blocks[0].mixer.pair_permutation().tolist() == list(range(24))   # pairs are neighbours already
    assert spec.embedding.pick_table() is None                           # a scaled table is no pick table


def test_every_pass_of_a_looped_layer_has_cache_and_state_of_its_own():
    spec = registry.build_spec(registry.config_from_dict(config()))
    model = Transformer(spec, torch.float32, "cpu")
    assert [c.layer for c in model.order] == [0, 1, 2, 1, 2]
    assert sorted(model.state_specs) == [1, 3]                            # the recurrent layer, once per pass
    assert model.state_specs[1].shape == (3 * (16 * 24 + 16 + 1),)
    (group,) = model.cache_groups                                         # equal attention layers, one group
    assert group.layers == (0, 2, 4) and group.window == 19


def test_yarn_frequencies_by_hand():
    f, mag = plain.yarn_frequencies(8, 100.0, {"factor": 4.0, "original": 16, "fast": 2.0, "slow": 0.25})
    base = [100.0 ** (-2 * i / 8) for i in range(4)]
    turn = lambda t: 8 * math.log(16 / (2 * math.pi * t)) / (2 * math.log(100.0))   # noqa: E731
    lo, hi = max(math.floor(turn(2.0)), 0), min(math.ceil(turn(0.25)), 7)
    assert (lo, hi) == (0, 3)
    for i in range(4):
        ramp = min(max((i - lo) / (hi - lo), 0.0), 1.0)
        assert float(f[i]) == pytest.approx(base[i] / 4.0 * ramp + base[i] * (1 - ramp), rel=1e-12)
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    # the engine's tables hold the same numbers
    rp = RotaryPositions(8, 100.0, YarnStretch(4.0, 16, 2.0, 0.25), interleaved=True)
    torch.testing.assert_close(rp.inv_freq, f.float())
    rp.prepare(50, "cpu")
    ang = torch.arange(50).float()[:, None] * f.float()
    torch.testing.assert_close(rp.cos, ang.cos() * mag)
    torch.testing.assert_close(rp.sin, ang.sin() * mag)
    plain_f, one = plain.yarn_frequencies(8, 100.0, None)
    assert one == 1.0 and float(plain_f[1]) == pytest.approx(100.0 ** -0.25)


def test_rotation_turns_neighbouring_pairs_and_leaves_the_rest():
    x = torch.arange(1.0, 13.0).view(1, 2, 6).repeat(3, 1, 1)
    y = plain.rotate(x, torch.tensor([0, 1, 5]), {"dims": 4, "base": 10.0, "scaling": None})
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    a = 5 * 10.0 ** -0.5                                           # pair 1 at position 5
    assert float(y[2, 0, 2]) == pytest.approx(3 * math.cos(a) - 4 * math.sin(a), rel=1e-5)
    assert float(y[2, 0, 3]) == pytest.approx(4 * math.cos(a) + 3 * math.sin(a), rel=1e-5)


def test_sink_takes_weight_and_gives_nothing():
    q, k = torch.zeros(2, 1, 4), torch.zeros(2, 1, 4)
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]])
    mask = plain.window_mask(2, 2)
    o = plain.sink_attention(q, k, v, 1.0, mask, torch.tensor([0.0]))
    # scores 0 everywhere: position 0 shares with the sink, position 1 with one key more
    torch.testing.assert_close(o[:, 0], torch.tensor([[0.5, 0.0], [1 / 3, 1 / 3]]))
    o = plain.sink_attention(q, k, v, 1.0, mask, torch.tensor([-1e9]))
    torch.testing.assert_close(o[:, 0], torch.tensor([[1.0, 0.0], [0.5, 0.5]]))
    assert plain.window_mask(5, 2).int().tolist()[3] == [0, 0, 1, 1, 0]


def test_matrix_memory_first_steps_by_hand():
    q = torch.tensor([[1.0, 0.0], [0.0, 2.0]])
    k = torch.tensor([[2.0, 0.0], [1.0, 1.0]])
    v = torch.tensor([[3.0], [5.0]])
    li, lf = torch.tensor([-1.0, 0.5]), torch.tensor([-0.2, -0.3])
    o = plain.mlstm_scan(q, k, v, li, lf)
    # token 0: m = max(-0.2 + 0, -1) = -0.2; S = e^(-0.8) k v^T; n = e^(-0.8) k
    g0 = math.exp(-0.8)
    assert float(o[0, 0]) == pytest.approx(g0 * 6.0 / (max(g0 * 2.0, math.exp(0.2)) + 1e-6), rel=1e-5)
    # token 1: a = -0.5, m = 0.5: S = e^(-1) S0 + k1 v1^T, n likewise; q picks the second row
    s_row1, n_row1 = 5.0, 1.0
    assert float(o[1, 0]) == pytest.approx(2 * s_row1 / (max(2 * n_row1, math.exp(-0.5)) + 1e-6), rel=1e-5)
    assert float(plain.capped(torch.tensor(1e6), 15.0)) == pytest.approx(15.0)


def test_router_chooses_with_the_correction_and_weighs_without():
    h = torch.eye(3)
    router = torch.tensor([[2.0, 0.0, 0.0], [1.0, 0.0, 0.0], [0.0, 0.0, 0.0], [-1.0, 0.0, 0.0]])
    corr = torch.tensor([0.0, 0.0, 0.0, 10.0])
    chosen, weight = plain.route(h[:1], router, corr, 2)
    s = torch.softmax(torch.tensor([2.0, 1.0, 0.0, -1.0]), 0)
    assert chosen.tolist() == [[3, 0]]                              # the corrected output first
    torch.testing.assert_close(weight[0], torch.stack([s[3], s[0]]) / (s[3] + s[0]))
    # an identity output passes the input on, times its weight
    w = {"p.router": router, "p.correction": corr, "p.e0.gate": torch.zeros(2, 3), "p.e0.up": torch.zeros(2, 3),
         "p.e0.down": torch.zeros(3, 2)}
    out = plain.routed_ff(h[:1], w, "p", {"router": {"experts": 1, "top": 1}, "shared": None})
    torch.testing.assert_close(out, h[:1])                          # output 3 >= 1 expert: identity, weight 1


def test_bfloat16_roundings_of_the_plain_model_stay_small():
    d = config()
    spec = registry.build_spec(registry.config_from_dict(d))
    g = torch.Generator().manual_seed(0)
    w = {k: (torch.randn(s.shape, generator=g) * s.std + (1.0 if s.init == "norm" else 0.0)).bfloat16()
         for k, s in sorted(spec.weight_specs().items())}
    toks = torch.randint(0, 211, (30,), generator=g).tolist()
    layers: list = []
    a = plain.forward(d, w, toks, layers_out=layers)
    b = plain.forward(d, w, toks, store=torch.bfloat16)
    assert len(layers) == 5 and a.shape == (30, 211)
    assert float((a - b).abs().max()) < 0.1 * float(a.std()) and not torch.equal(a, b)
    assert float(a.abs().max()) <= 20.0                              # capped
    assert plain.greedy(d, w, toks[:3], 2) == [int(plain.forward(d, w, toks[:3])[-1].argmax()),
                                               plain.greedy(d, w, toks[:3], 2)[1]]
