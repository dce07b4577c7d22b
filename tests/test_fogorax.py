"""Fogorax without a GPU: its configuration, what the builder asks of the checkpoint, how its
cache groups and state come out, the cache manager's upkeep of kept first pages, and the plain
model's own mechanisms against cases worked out by hand."""

from __future__ import annotations

import copy
import json

import pytest
import torch

import kvforge_amd
from kvforge_amd import registry
from kvforge_amd.cache.manager import CacheGroup, CacheManager
from kvforge_amd.config.fogorax import FogoraxConfig
from kvforge_amd.config.presets import fogorax as make_config
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts.base import CacheSpec, attention_pages
from tests.plain import fogorax as plain


def two_masks() -> dict:
    """Four layers; layer 2 reads layer 0's keys through a wider window, layer 3 layer 1's."""
    cfg = make_config(vocab=50, width=24, layers=4, heads=4, kv_heads=2, dim=16, ff=40, window=6,
                      keep_first=1, side_dim=3, max_positions=64, share_every=1)
    cfg["layers"][1]["mixer"]["mask"] = {"keep_first": 0, "size": 9}
    cfg["layers"][2]["mixer"].update(kv_from=0, mask={"keep_first": 5, "size": 11})
    cfg["layers"][3]["mixer"].update(kv_from=1, mask={"keep_first": 0, "size": 4})
    cfg["layers"][3]["mlp"] = None
    return cfg


def test_config_round_trip_and_registry_key():
    d = two_masks()
    cfg = registry.config_from_dict(d)
    assert isinstance(cfg, FogoraxConfig) and cfg.architecture == "Fogorax"
    assert json.dumps(cfg.to_dict(), sort_keys=True) == json.dumps(d, sort_keys=True)
    assert cfg.layers[2].mixer.kv_from == 0 and cfg.layers[3].mlp is None
    assert cfg.vocab_size == 50 and cfg.max_position_embeddings == 64 and cfg.side_dim == 3
    # a list of names, as other files write it, names the same model
    alt = dict(d, architectures=["Fogorax"])
    del alt["architecture"]
    assert isinstance(registry.config_from_dict(alt), FogoraxConfig)
    with pytest.raises(kvforge_amd.ConfigError):
        registry.config_from_dict({"vocab": 5})
    # kv_heads and vdim may be left out
    short = copy.deepcopy(d)
    for i in (1, 3):                  # layer 3 reads layer 1's keys: the two agree again
        del short["layers"][i]["mixer"]["kv_heads"], short["layers"][i]["mixer"]["vdim"]
    m = registry.config_from_dict(short).layers[1].mixer
    assert (m.kv_heads, m.vdim) == (m.heads, m.dim)


@pytest.mark.parametrize("change,needle", [
    (lambda d: d["layers"][2]["mixer"].update(kv_from=3), "later layer"),
    (lambda d: d["layers"][2]["mixer"].update(kv_from=2), "not another layer"),
    (lambda d: d["layers"][3]["mixer"].update(kv_from=2), "no keys of its own"),
    (lambda d: d["layers"][2]["mixer"].update(dim=32), "differ"),
    (lambda d: d["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda d: d["layers"][0].update(type="recurrent"), "not supported"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "not supported"),
    (lambda d: d["layers"][0]["mixer"]["mask"].update(size=0), "positive"),
    (lambda d: d["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda d: d.pop("norm"), "norm"),
])
def test_config_refuses_what_the_model_cannot_be(change, needle):
    d = copy.deepcopy(two_masks())
    change(d)
    with pytest.raises(kvforge_amd.ConfigError, match=needle):
        registry.config_from_dict(d)


def test_builder_names_the_checkpoints_tensors():
    d = two_masks()
    spec = registry.build_spec(registry.config_from_dict(d))
    ws = {k: tuple(v.shape) for k, v in spec.weight_specs().items()}
    assert ws["embed"] == (50, 24) and ws["pos"] == (64, 24) and ws["head"] == (50, 24)
    assert ws["side.embed"] == (50, 12) and ws["final.norm"] == () and ws["l0.norm1"] == ()
    assert ws["l0.mix.q"] == (64, 24) and ws["l0.mix.k"] == (32, 24) and ws["l0.mix.g"] == (64, 24)
    assert ws["l0.mix.o"] == (24, 64) and ws["l1.shift"] == (24,)
    assert ws["l0.mlp.gate"] == (40, 24) and ws["l0.mlp.down.b"] == (24,) and ws["l0.mlp.up.b"] == (40,)
    assert ws["l3.side.gate"] == (3, 24) and ws["l3.side.proj"] == (24, 3) and ws["l3.side.norm"] == (24,)
    # a layer that reads another's cache projects no keys and values; one without mlp has none
    assert "l2.mix.k" not in ws and "l2.mix.v" not in ws and "l3.mlp.gate" not in ws
    assert [c.cache_of for c in spec.run_order()] == [None, None, 0, 1]


def test_cache_groups_keep_what_every_reader_needs_and_every_call_has_state():
    spec = registry.build_spec(registry.config_from_dict(two_masks()))
    model = Transformer(spec, torch.float32, "cpu")
    got = sorted((g.layers, g.window, g.keep_first) for g in model.cache_groups)
    # call 0 is read through windows of 6 (keeping 1) and 11 (keeping 5); call 1 through 9 and 4
    assert got == [((0,), 11, 5), ((1,), 9, 0)]
    assert sorted(model.state_specs) == [0, 1, 2, 3]
    assert all(s.shape == (24,) and s.dtype == torch.float32 for s in model.state_specs.values())


def test_covering_spec():
    pages = attention_pages(2, 16)
    a, b = CacheSpec(pages, 8, 2), CacheSpec(pages, 5, 3)
    assert a.covering(b) == CacheSpec(pages, 8, 3)
    assert a.covering(CacheSpec(pages, None)) == CacheSpec(pages, None, 0)
    with pytest.raises(ValueError):
        a.covering(CacheSpec(attention_pages(2, 32), 8, 2))


@pytest.mark.parametrize("keep,kept_pages", [(0, 0), (1, 1), (4, 1), (5, 2), (8, 2), (9, 3)])
def test_pages_of_kept_first_positions_are_never_given_back(keep, kept_pages):
    cm = CacheManager(4, [CacheGroup((0,), (), window=6, keep_first=keep)], 32)
    cm.allocate("a", 0)
    cm.append_slots("a", 50, 0)
    before = cm.num_free_blocks
    cm.release_behind("a", 50)        # the next query, at 50, sees keys from 45 on: pages 11 and up
    table = cm.block_table("a")
    assert [i for i, p in enumerate(table) if p >= 0] == list(range(kept_pages)) + [11, 12]
    assert cm.num_free_blocks == before + 11 - kept_pages
    cm.free("a")
    assert cm.num_free_blocks == 32


# ------------------------------------------------------------------ the plain model's mechanisms
def test_window_mask_by_hand():
    m = plain.window_mask(7, 3, 2)
    assert m[0].tolist() == [True] + [False] * 6
    assert m[4].tolist() == [True, True, True, True, True, False, False]     # 0, 1 kept; 2, 3, 4 in the window
    assert m[6].tolist() == [True, True, False, False, True, True, True]
    assert torch.equal(plain.window_mask(5, 99, 0), torch.ones(5, 5).tril().bool())
    assert torch.equal(plain.window_mask(5, 1, 0), torch.eye(5).bool())


def test_token_shift_by_hand():
    h = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 8.0]])
    mu = torch.tensor([0.0, 0.5])
    assert plain.token_shift(h, mu).tolist() == [[1.0, 1.0], [3.0, 3.0], [5.0, 6.0]]
    assert torch.equal(plain.token_shift(h, torch.ones(2))[1:], h[:-1])


def test_scalar_norm_and_gelu_by_hand():
    x = torch.tensor([[3.0, 4.0]])
    y = plain.scalar_norm(x, torch.tensor(2.0), 0.0)
    torch.testing.assert_close(y, torch.tensor([[6.0, 8.0]]) / (12.5 ** 0.5))
    z = torch.linspace(-4, 4, 33)
    torch.testing.assert_close(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))


def test_attention_heads_share_keys_in_groups_and_see_through_the_mask():
    g = torch.Generator().manual_seed(0)
    T, H, KV, d, dv = 6, 4, 2, 3, 5
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, KV, d, generator=g), torch.randn(T, KV, dv, generator=g)
    mask = plain.window_mask(T, 2, 1)
    out = plain.masked_attention(q, k, v, 0.7, mask)
    assert out.shape == (T, H, dv)
    i, h = 5, 3                       # sees keys 0 (kept), 4, 5; head 3 reads kv head 1
    s = torch.stack([q[i, h] @ k[j, 1] for j in (0, 4, 5)]) * 0.7
    torch.testing.assert_close(out[i, h], torch.softmax(s, 0) @ v[[0, 4, 5], 1])


def test_a_far_window_is_plain_causal_attention_and_kv_sharing_changes_the_output():
    cfg = two_masks()
    spec = registry.build_spec(registry.config_from_dict(cfg))
    from kvforge_amd.weights.random_init import random_tensors
    w = random_tensors(spec, 3, "float32")
    toks = list(range(20, 45))
    base = plain.forward(cfg, w, toks)
    far = copy.deepcopy(cfg)
    for layer in far["layers"]:
        layer["mixer"]["mask"] = {"keep_first": 0, "size": 1000}
    kept = copy.deepcopy(far)
    for layer in kept["layers"]:
        layer["mixer"]["mask"]["keep_first"] = 7           # nothing to keep that is not seen anyway
    torch.testing.assert_close(plain.forward(far, w, toks), plain.forward(kept, w, toks))
    assert not torch.allclose(plain.forward(far, w, toks)[12:], base[12:], atol=1e-4)
    assert torch.allclose(plain.forward(far, w, toks)[:4], base[:4], atol=1e-5)   # inside every window
