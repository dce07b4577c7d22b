"""Rudorax on the GPU against the plain model of ``tests/plain/rudorax.py``: every new kernel
alone, then whole models of several shapes through the engine's own step function, cache and
state manager, scheduler and entry points, cut in every way a server cuts its work."""

from __future__ import annotations

import math
import os
import random

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import kvforge_amd
from kvforge_amd.config.presets import rudorax as make_config
from kvforge_amd.engine.batch import StepEntry
from tests import replay_util as ru
from tests.plain import rudorax as plain
from tests.test_fogorax_gpu import in_portions, make_runner, prompts_for, replay, replay_all, row_error
from tests.test_kernels_gpu import Paged, prefill_work

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


# ============================================================================ kernels alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_with_a_scale_and_capped_logits(dtype):
    table = rand(37, 48, seed=1).to(dtype)
    ids = torch.tensor([0, 36, 5, 99, -1], dtype=torch.int32)
    out = torch.full((5, 48), 7.0, device=DEV)
    ops().embed(ids.to(DEV), table.to(DEV), out, 13.75)
    want = torch.zeros(5, 48)
    want[:3] = table.float()[ids[:3].long()] * 13.75
    assert torch.equal(out.cpu(), want)
    z = rand(3, 1001, seed=2, scale=40.0)
    got = z.clone().to(DEV)
    ops().softcap(got, 30.0)
    torch.testing.assert_close(got.cpu(), 30.0 * torch.tanh(z / 30.0), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_with_a_weight_stored_around_zero(dtype):
    from kvforge_amd.parts import OnePlusRMSNorm
    h = 100
    norm = OnePlusRMSNorm("l0.norm1", h, 1e-3)
    w = rand(h, seed=3, scale=0.3).to(dtype)
    norm.load({"l0.norm1": w.to(DEV)})
    x = rand(6, h, seed=4, scale=3.0)
    out = torch.empty(6, h, dtype=dtype, device=DEV)
    norm.forward(x.to(DEV), out)
    torch.testing.assert_close(out.float().cpu(), plain.one_plus_norm(x, w.float(), 1e-3), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [36, 100, 1024, 2500])
@pytest.mark.parametrize("owed", [None, "same", "float32"])
def test_two_norms_of_one_stream_in_one_pass(dtype, h, owed):
    x, w1, w2 = rand(5, h, seed=h, scale=3.0), rand(h, seed=1, scale=0.3), rand(h, seed=2, scale=0.3)
    add = None if owed is None else rand(5, h, seed=3).to(dtype if owed == "same" else torch.float32)
    dev = x.clone().to(DEV)
    o1, o2 = torch.empty(5, h, dtype=dtype, device=DEV), torch.empty(5, h, dtype=dtype, device=DEV)
    ops().rmsnorm_pair(dev, (1.0 + w1).to(DEV), (1.0 + w2).to(DEV), 1e-5, o1, o2, add=None if add is None else add.to(DEV))
    total = x + (add.float() if add is not None else 0.0)
    torch.testing.assert_close(dev.cpu(), total, atol=1e-6, rtol=1e-6)          # what was owed is in the stream now
    torch.testing.assert_close(o1.float().cpu(), plain.one_plus_norm(total, w1, 1e-5), **tol(dtype))
    torch.testing.assert_close(o2.float().cpu(), plain.one_plus_norm(total, w2, 1e-5), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,dk,d,rot", [(4, 2, 16, 16, 16), (3, 1, 24, 32, 10), (8, 1, 64, 64, 64),
                                           (2, 2, 100, 112, 64), (5, 5, 7, 16, 6), (2, 1, 256, 256, 128)])
def test_head_norm_rotation_and_cache_write_in_one_kernel(dtype, H, KV, dk, d, rot):
    """q and k heads normalised over their first dk elements, rotated in neighbouring pairs over
    the first rot, k and v written to scattered pages; padding elements stay zero."""
    from kvforge_amd.parts.positions import RotaryPositions, YarnStretch
    n, bs, eps = 9, 8, 1e-4
    rp = RotaryPositions(rot, 5000.0, YarnStretch(4.0, 32, 8.0, 1.0), interleaved=True)
    rp.prepare(64, DEV)
    rot_cfg = {"dims": rot, "base": 5000.0, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    rows = rand(n, (H + 2 * KV) * d, seed=dk).view(n, H + 2 * KV, d).clone()
    rows[:, :H + KV, dk:] = 0.0            # zero rows of the projections give zeros here
    rows = rows.view(n, -1).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 17, 18, 40, 41, 63], dtype=torch.int32)
    qw, kw = 1.0 + rand(dk, seed=1, scale=0.2), 1.0 + rand(dk, seed=2, scale=0.2)
    table = i32([[7, 2, 5, 0, 3, 1, 6, 4]])
    kp = torch.full((8, KV, bs, d), 9.0, dtype=dtype, device=DEV)
    vp = torch.full((8, KV, d, bs), 9.0, dtype=dtype, device=DEV)
    dev = rows.clone().to(DEV)
    ops().qknorm_rope_kvwrite(dev, pos.to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV), rp.cos, rp.sin,
                              table, kp, vp, H, KV, d, qw.to(DEV), kw.to(DEV), dk, eps)
    x = rows.float().view(n, H + 2 * KV, d)
    q = plain.rotate(plain.rms(x[:, :H, :dk], eps) * qw, pos, rot_cfg)
    k = plain.rotate(plain.rms(x[:, H:H + KV, :dk], eps) * kw, pos, rot_cfg)
    got = dev.float().cpu().view(n, H + 2 * KV, d)
    torch.testing.assert_close(got[:, :H, :dk], q, **tol(dtype))
    assert float(got[:, :H, dk:].abs().max() if d > dk else 0.0) == 0.0
    for t, p in enumerate(pos.tolist()):
        page, off = int(table[0, p // bs]), p % bs
        torch.testing.assert_close(kp[page, :, off, :dk].float().cpu(), k[t], **tol(dtype))
        assert float(kp[page, :, off, dk:].abs().max() if d > dk else 0.0) == 0.0
        torch.testing.assert_close(vp[page, :, :, off].float().cpu(), x[t, H + KV:], **tol(dtype))


def sink_reference(paged, q, seq_lens, q_lens, scale, window, sink):
    outs, off = [], 0
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        mask = plain.window_mask(n, window if window else n)[n - ql:]
        outs.append(plain.sink_attention(q[off:off + ql].float(), paged.keys[s].float(),
                                         paged.values[s].float(), scale, mask, sink))
        off += ql
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 4), (8, 1, 64, 16), (3, 1, 48, 8), (6, 2, 128, 16)])
@pytest.mark.parametrize("window", [0, 1, 21, 40])
def test_attention_with_a_sink_in_the_softmax(dtype, H, KV, d, bs, window):
    """Query runs and single tokens (one cut and several): the sink takes weight from the keys.
    Sinks from far below every score to far above."""
    scale = 1 / math.sqrt(d)
    sink = torch.tensor([(-30.0, -1.0, 0.5, 3.0, 8.0, 0.0, 2.0, 40.0)[h % 8] for h in range(H)])
    for seq_lens, q_lens in (([90, 33, 70, 5], [40, 33, 2, 5]), ([7, 90, 1, 300], [1, 1, 1, 1])):
        paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + window)
        n = sum(q_lens)
        buf = rand(n, H * d, seed=d + 1, scale=2.0).to(dtype)
        cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
        ctx = torch.tensor(seq_lens, dtype=torch.int32)
        want = sink_reference(paged, buf.view(n, H, d), seq_lens, q_lens, scale, window, sink).reshape(n, H * d)
        without = sink_reference(paged, buf.view(n, H, d), seq_lens, q_lens, scale, window,
                                 torch.full((H,), -1e9)).reshape(n, H * d)
        assert float((want - without).abs().max()) > 0.05        # the sink matters here
        args = (buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV))
        if max(q_lens) > 1:
            out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
            ops().attn_prefill(*args, cu.to(DEV), ctx.to(DEV), prefill_work(q_lens, H // KV, dtype, d, bs).to(DEV),
                               out, H, KV, d, scale, window, sinks=sink.to(DEV))
            torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))
            continue
        for splits in (1, 3):
            out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
            ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV))
            ops().attn_decode(*args, None, n, cu.to(DEV), ctx.to(DEV), out, H, KV, d, scale, window, splits, ws,
                              sinks=sink.to(DEV))
            torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


def scan_reference(q, k, v, zi, zf, bias, cap, H, dk, dv):
    """``q k [T, H dk]``, ``v [T, H dv]``, gate pre-activations ``[T, H]``: the heads' raw outputs."""
    T = q.shape[0]
    li = plain.capped(zi + bias[:H], cap)
    lf = torch.nn.functional.logsigmoid(plain.capped(zf + bias[H:], cap))
    qs = q.view(T, H, dk) * dk ** -0.5
    return torch.stack([plain.mlstm_scan(qs[:, j], k.view(T, H, dk)[:, j], v.view(T, H, dv)[:, j], li[:, j], lf[:, j])
                        for j in range(H)], dim=1).reshape(T, H * dv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(2, 8, 16), (6, 32, 64), (1, 40, 100), (3, 64, 24), (2, 100, 130),
                                     (2, 128, 64), (1, 200, 70), (1, 256, 8)])
@pytest.mark.parametrize("chunk_from", [1, 8, 1000])
def test_matrix_memory_over_runs_and_steps(dtype, H, dk, dv, chunk_from):
    """Four sequences in three steps: runs of many tokens, of two and of one; a sequence that
    starts in the slot another gave back (which still holds that one's state); a sequence
    without a slot.  Gates reach both ends of their cap.  ``chunk_from``: every run chunk by
    chunk on the matrix cores, every run token by token, and the two kernels side by side in
    one step, each carrying on from the state the other left."""
    cap = 6.0
    lens = {"a": 23, "b": 9, "c": 1, "d": 12}
    cols = 2 * H * dk + H * dv + 5                      # rows wider than q, k, v: something behind them
    data = {r: (rand(n, cols, seed=i + dk).to(dtype), rand(n, 2 * H, seed=i + 50, scale=5.0))
            for i, (r, n) in enumerate(lens.items())}
    bias = rand(2 * H, seed=9, scale=2.0)
    want = {}
    for r, (rows, z) in data.items():
        x = rows.float()
        want[r] = scan_reference(x[:, :H * dk], x[:, H * dk:2 * H * dk], x[:, 2 * H * dk:2 * H * dk + H * dv],
                                 z[:, :H], z[:, H:], bias, cap, H, dk, dv)
    state = torch.full((3, ops().mlstm_state_floats(H, dk, dv)), 3.0, device=DEV)   # junk
    slot = {"a": 2, "b": 0, "c": 1, "d": 1}
    got = {r: [] for r in lens}
    for step in ([("a", 0, 14), ("b", 0, 1), ("c", 0, 1)], [("b", 1, 3), ("d", 0, 11), ("a", 14, 15)],
                 [("a", 15, 23), ("d", 11, 12), ("b", 3, 9)]):
        rows = torch.cat([data[r][0][a:b] for r, a, b in step]).to(DEV)
        z = torch.cat([data[r][1][a:b] for r, a, b in step]).to(DEV)
        counts = [b - a for _, a, b in step] + [1]       # and a padding sequence without a slot
        rows = torch.cat([rows, torch.full((1, cols), float("nan"), dtype=dtype, device=DEV)])
        z = torch.cat([z, torch.zeros(1, 2 * H, device=DEV)])
        cu = i32([0] + list(np.cumsum(counts)))
        pos = torch.cat([torch.arange(a, b) for _, a, b in step] + [torch.zeros(1, dtype=torch.long)]).int().to(DEV)
        out = torch.full((rows.shape[0], H * dv), 5.0, device=DEV)
        ops().mlstm_scan(rows, z, bias.to(DEV), cu, pos, i32([slot[r] for r, _, _ in step] + [-1]), state, out,
                         len(counts), H, dk, dv, 0, H * dk, 2 * H * dk, cap, dk ** -0.5, chunk_from=chunk_from)
        off = 0
        for (r, a, b) in step:
            got[r].append(out[off:off + b - a].cpu())
            off += b - a
        assert float(out[off:].abs().max()) == 0.0       # the sequence without a slot
    for r in lens:
        torch.testing.assert_close(torch.cat(got[r]), want[r], atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(2, 40, 72), (1, 136, 64), (1, 256, 40), (3, 16, 130)])
def test_matrix_memory_over_many_chunks(dtype, H, dk, dv):
    """A run of 203 tokens in portions that end inside chunks, the state handed from chunk to
    chunk and from step to step; forget gates that stay open, so that the first tokens still
    weigh at the end."""
    cap, T = 15.0, 203
    cols = 2 * H * dk + H * dv
    rows, z = rand(T, cols, seed=dk).to(dtype), rand(T, 2 * H, seed=dv, scale=3.0)
    bias = torch.cat([torch.full((H,), -1.0), torch.full((H,), 6.0)])
    x = rows.float()
    want = scan_reference(x[:, :H * dk], x[:, H * dk:2 * H * dk], x[:, 2 * H * dk:], z[:, :H], z[:, H:], bias, cap, H, dk, dv)
    state = torch.full((2, ops().mlstm_state_floats(H, dk, dv)), 3.0, device=DEV)
    got = []
    for a, b in ((0, 130), (130, 131), (131, 203)):
        out = torch.empty(b - a, H * dv, device=DEV)
        ops().mlstm_scan(rows[a:b].to(DEV), z[a:b].to(DEV), bias.to(DEV), i32([0, b - a]),
                         torch.arange(a, b, dtype=torch.int32, device=DEV), i32([1]), state, out, 1, H, dk, dv,
                         0, H * dk, 2 * H * dk, cap, dk ** -0.5)
        got.append(out.cpu())
    torch.testing.assert_close(torch.cat(got), want, atol=3e-4, rtol=3e-4)
    assert float(state[0].min()) == 3.0                       # the other slot is nobody's business


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(2, 40, 72), (1, 136, 64), (1, 256, 40), (3, 16, 130)])
def test_matrix_memory_with_all_chunks_at_once(dtype, H, dk, dv):
    """Three sequences in two steps: the longest runs go through the passes that take all
    chunks at once, beside a run for the one-kernel chunks and single tokens; every run carries
    on from the state that another kernel left in its slot."""
    cap = 15.0
    lens = {"a": 300, "b": 210, "c": 150}
    cols = 2 * H * dk + H * dv
    data = {r: (rand(n, cols, seed=i + dk).to(dtype), rand(n, 2 * H, seed=i + 9, scale=3.0)) for i, (r, n) in enumerate(lens.items())}
    bias = torch.cat([torch.full((H,), -1.0), torch.full((H,), 5.0)])
    want = {}
    for r, (rows, z) in data.items():
        x = rows.float()
        want[r] = scan_reference(x[:, :H * dk], x[:, H * dk:2 * H * dk], x[:, 2 * H * dk:], z[:, :H], z[:, H:], bias, cap, H, dk, dv)
    state = torch.full((3, ops().mlstm_state_floats(H, dk, dv)), 3.0, device=DEV)
    slot = {"a": 1, "b": 2, "c": 0}
    got = {r: [] for r in lens}
    multi_from = 100
    for step in ([("a", 0, 131), ("b", 0, 1), ("c", 0, 40)], [("b", 1, 210), ("c", 40, 150), ("a", 131, 132)],
                 [("a", 132, 300)]):
        rows = torch.cat([data[r][0][a:b] for r, a, b in step]).to(DEV)
        z = torch.cat([data[r][1][a:b] for r, a, b in step]).to(DEV)
        q_lens = [b - a for _, a, b in step]
        chunks, runs = ops().mlstm_multi_plan(q_lens, dk, multi_from)
        multi = {"chunks": i32(chunks).view(-1, 4), "runs": i32(runs).view(-1, 3)}
        for name, (shape, dt) in ops().mlstm_multi_scratch(rows.shape[0], len(chunks) // 4, H, dk, dv).items():
            multi[name] = torch.full(shape, float("nan"), dtype=dt, device=DEV)
        out = torch.full((rows.shape[0], H * dv), 5.0, device=DEV)
        ops().mlstm_scan(rows, z, bias.to(DEV), i32([0] + list(np.cumsum(q_lens))),
                         torch.cat([torch.arange(a, b) for _, a, b in step]).int().to(DEV),
                         i32([slot[r] for r, _, _ in step]), state, out, len(step), H, dk, dv, 0, H * dk, 2 * H * dk,
                         cap, dk ** -0.5, multi_from=multi_from, multi=multi)
        off = 0
        for (r, a, b) in step:
            got[r].append(out[off:off + b - a].cpu())
            off += b - a
    for r in lens:
        torch.testing.assert_close(torch.cat(got[r]), want[r], atol=3e-4, rtol=3e-4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_normed_weighted_and_gated(dtype):
    H, dv, n, eps = 3, 40, 5, 1e-3
    raw, w = rand(n, H * dv, seed=1, scale=4.0), 1.0 + rand(H * dv, seed=2, scale=0.2)
    wide = rand(n, 3 * H * dv, seed=3, scale=2.0).to(dtype)
    out = torch.empty(n, H * dv, dtype=dtype, device=DEV)
    ops().mlstm_out(raw.to(DEV), wide.to(DEV)[:, H * dv:2 * H * dv], w.to(DEV), eps, out, H, dv)
    want = plain.rms(raw.view(n, H, dv), eps).reshape(n, H * dv) * w * torch.sigmoid(wide[:, H * dv:2 * H * dv].float())
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("R,top", [(5, 1), (20, 3), (64, 8), (130, 4), (512, 16), (3, 3)])
def test_router_chooses_by_corrected_probability_and_weighs_by_probability(R, top):
    n = 50
    z, corr = rand(n, R, seed=R, scale=3.0), rand(R, seed=1, scale=0.3)
    chosen = torch.empty(n, top, dtype=torch.int32, device=DEV)
    weights = torch.empty(n, top, device=DEV)
    ops().moe_topk(z.to(DEV), corr.to(DEV), chosen, weights)
    s = torch.softmax(z, dim=-1)
    want = torch.topk(s + corr, top, dim=-1).indices
    assert torch.equal(chosen.cpu().long(), want)                # in order of the corrected score
    g = s.gather(-1, want)
    torch.testing.assert_close(weights.cpu(), g / g.sum(-1, keepdim=True), atol=1e-6, rtol=1e-5)
    # the correction changes the choice somewhere and the weights nowhere
    assert not torch.equal(want.sort(-1).values, torch.topk(s, top, dim=-1).indices.sort(-1).values) or R == top


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 5, 70, 300])
@pytest.mark.parametrize("E,I,top,ff,shared", [(4, 0, 1, 16, 0), (16, 4, 3, 24, 40), (5, 2, 7, 8, 16), (8, 1, 2, 72, 0),
                                               (6, 2, 3, 32, 16), (33, 0, 4, 64, 0), (3, 1, 2, 96, 8)])
def test_routed_feed_forward_alone(dtype, n, E, I, top, ff, shared):
    """The part by itself on a step of ``n`` rows: few rows and many take other products; expert
    widths that are a multiple of 32 take the grouped kernels in bfloat16, the others (and
    32-bit) the product over all experts."""
    from kvforge_amd.engine.batch import Step, Workspace
    from kvforge_amd.parts import RoutedExperts
    h = 48
    part = RoutedExperts("l0.mlp", h, ff, E, top, I, shared)
    names = {k: rand(*v.shape, seed=i, scale=(1.0 if k.endswith("router") else 0.15))
             for i, (k, v) in enumerate(sorted(part.weight_specs().items()))}
    part.load({k: t.to(dtype).to(DEV) for k, t in names.items()})
    part.seal()
    w = {k: t.to(dtype).float() for k, t in names.items()}
    x = rand(n, h, seed=77).to(dtype)
    res0 = rand(n, h, seed=78)
    step = Step()
    step.ws, step.act_dtype, step.device = Workspace(DEV), dtype, DEV
    res = res0.clone().to(DEV)
    part.forward(x.to(DEV), step, res)
    step.settle()
    mlp = {"router": {"experts": E, "top": top}, "shared": {"ff": shared} if shared else None}
    want = res0 + plain.routed_ff(x.float(), w, "l0.mlp", mlp)
    torch.testing.assert_close(res.cpu(), want, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32
                                                   else dict(atol=5e-2, rtol=5e-2)))


# ============================================================================ whole models
def shape_a():
    """Attention and recurrence mixed, a stretch gone through three times, every size another
    than anywhere else in this file: groups of three heads, value heads larger than key heads
    and neither a multiple of 16, half of a head rotated, an odd number of experts."""
    att = dict(heads=6, kv_heads=2, dim=24, vdim=40, window=19, rot_dims=12, scale=0.2,
               scaling={"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0})
    rec = dict(heads=3, dim=16, vdim=24, gate_cap=8.0)
    moe = dict(ff=24, experts=5, top=2, identity=2, shared_ff=40)
    return make_config(vocab=211, width=72, layers=[("attention", att, moe), ("mlstm", rec, moe),
                                                    ("attention", att, moe), ("mlstm", rec, None)],
                       loop=(1, 3, 3), embedding_scale=6.5, logit_softcap=20.0, eps=1e-5, max_positions=512)


def shape_b():
    """What a model may make equal or one: as many kv heads as heads, the whole head rotated
    without stretched frequencies, one expert per token and no identity outputs, no shared
    expert, one recurrent head, a window of one key in one layer and longer than any prompt in
    another, no loop, no cap on the logits, an embedding scale of one."""
    a1 = dict(heads=2, kv_heads=2, dim=32, vdim=32, window=1, rot_dims=32, scale=32 ** -0.5, scaling=None)
    a2 = dict(heads=4, kv_heads=4, dim=16, vdim=16, window=4096, rot_dims=16, scale=0.25, scaling=None)
    rec = dict(heads=1, dim=72, vdim=64, gate_cap=30.0)
    moe = dict(ff=32, experts=4, top=1, identity=0, shared_ff=0)
    return make_config(vocab=97, width=64, layers=[("mlstm", rec, moe), ("attention", a1, moe),
                                                   ("attention", a2, None), ("mlstm", rec, moe)],
                       loop=None, embedding_scale=1.0, logit_softcap=None, eps=1e-6, max_positions=512)


def shape_c():
    """One kv head under eight, head size 64 (the matrix-core kernels' own), a recurrence whose
    keys span two waves' rows, the loop from the first layer on, nothing but recurrence after it."""
    att = dict(heads=8, kv_heads=1, dim=64, vdim=48, window=33, rot_dims=64, scale=0.125,
               scaling={"factor": 8.0, "original": 64, "fast": 32.0, "slow": 1.0})
    rec = dict(heads=2, dim=136, vdim=72, gate_cap=15.0)
    moe = dict(ff=64, experts=9, top=3, identity=3, shared_ff=96)
    return make_config(vocab=300, width=128, layers=[("attention", att, moe), ("mlstm", rec, moe),
                                                     ("mlstm", rec, moe)],
                       loop=(0, 2, 2), embedding_scale=11.3, logit_softcap=30.0, eps=1e-6, max_positions=512)


SHAPE = {"a": shape_a, "b": shape_b, "c": shape_c}


def liven(folder: str) -> None:
    """Random weights of std 0.02 give a model whose layers hardly move the stream and whose
    attention and routing are flat.  Scaled so that attention is peaked (through the q/k norm
    weights, which set the scores' size), the gates of the recurrence swing with the tokens, the
    router prefers some experts clearly and every layer outweighs the embedding."""
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        f = 1.0
        if k.endswith(("q.norm", "k.norm")):
            f = 2.5
        elif k.endswith((".mix.v", ".mix.o", ".mix.g", ".down")):
            f = 6.0
        elif ".mix." in k and k.endswith((".q", ".k")):
            f = 6.0
        elif k.endswith((".mix.i", ".mix.f")):
            f = 25.0
        elif k.endswith(".router"):
            f = 40.0
        if f != 1.0:
            w[k] = (w[k].float() * f).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})


_MODELS: dict = {}


def model_folder(tmp_path_factory, name: str, dtype):
    key = (name, dtype)
    if key not in _MODELS:
        folder = str(tmp_path_factory.mktemp(f"rudorax_{name}_{NAME[dtype]}"))
        cfg = SHAPE[name]()
        kvforge_amd.write_random_model(folder, cfg, seed=len(name) + 23, dtype=NAME[dtype])
        liven(folder)
        _MODELS[key] = (folder, cfg, load_file(os.path.join(folder, "model.safetensors")))
    return _MODELS[key]


_WANT: dict = {}


def jittered(w: dict, seed: int) -> dict:
    """The weights with every matrix moved by about half a bfloat16 step (relative 2^-9, random
    sign per element): what rounding could have made of them."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for k, v in w.items():
        if v.is_floating_point() and v.dim() == 2:
            sign = torch.randint(0, 2, v.shape, generator=g).float() * 2.0 - 1.0
            out[k] = v.float() * (1.0 + sign * 2.0 ** -9)
        else:
            out[k] = v
    return out


def plain_logits(cfg, w, toks, dtype):
    """(the truth, plain runs with the roundings of ``dtype``): the plain model in 64-bit, and in
    32-bit (for a 32-bit engine) or in 32-bit with every trip through memory that a bfloat16
    engine may make rounded to bfloat16.  The design has places where rounding is multiplied
    many times (a recurrent head whose query is all but orthogonal to its memory is then divided
    by its own small size; a first token's head is its value times the *sign* of q . k), so the
    bfloat16 runs are three: as the weights are, and twice with them moved by half a bfloat16
    step, which shows the rows where such a place is near."""
    key = (id(w), tuple(toks), dtype)
    if key not in _WANT:
        truth = plain.forward(cfg, w, toks, dtype=torch.float64).float()
        if dtype == torch.bfloat16:
            runs = [plain.forward(cfg, w, toks, store=torch.bfloat16)]
            runs += [plain.forward(cfg, jittered(w, s), toks, store=torch.bfloat16) for s in (1, 2)]
        else:
            runs = [plain.forward(cfg, w, toks)]
        _WANT[key] = (truth, runs)
    return _WANT[key]


def close_to_truth(got, truth, plain_runs, dtype, what="") -> None:
    """Lively weights, loops and a recurrence multiply rounding, so the bound is measured, not
    widened: a row of the engine may be off the 64-bit truth by three times what the plain runs
    with the same kind of roundings are off in that row (the worst of them), or a multiple of
    their worst row (one and a half times in bfloat16; five times in 32-bit, where the worst of
    a few hundred rows is a wide-tailed thing and two correct orders of summation differ by as
    much), or a fixed small share of the logits' spread, whichever is most.  A lost key, state,
    page or expert moves a row by about the whole spread."""
    err = row_error(got, truth)
    off = torch.stack([row_error(r, truth) for r in plain_runs]).max(0).values
    floor = torch.full_like(err, 2e-4 if dtype == torch.float32 else 3e-2)
    limit = torch.maximum(floor, torch.maximum(3.0 * off, (5.0 if dtype == torch.float32 else 1.5) * off.max()))
    worst = int((err / limit).argmax())
    assert float(err[worst]) <= float(limit[worst]), (
        f"{what}: position {worst} is off by {float(err[worst]):.3e} of the logits' spread "
        f"(allowed {float(limit[worst]):.3e})")


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
def test_the_stream_after_every_layer_run(tmp_path_factory, name):
    """In 32-bit, after every run of a layer (a looped layer every time), so that a fault names
    its layer and pass."""
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
    assert len(model.order) == len(want) == len(plain.run_order(cfg))
    with torch.inference_mode():
        residual = model.embed(step)
        for i, (call, ls) in enumerate(zip(model.order, model.layer_states)):
            model.spec.blocks[call.layer].forward(residual, step, ls)
            step.settle()
            # against the 64-bit stream, within eight times what the plain 32-bit run is off it
            # there (lively weights and loops multiply rounding), or a small fixed margin
            own = float((want[i].double() - truth[i]).abs().max())
            torch.testing.assert_close(residual.cpu().double(), truth[i], atol=max(3e-4, 8.0 * own), rtol=3e-4,
                                       msg=lambda m: f"run {i}: {m}")


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
    runner = make_runner(folder, dtype, block_size=8, num_blocks=34, seqs=4)
    together = replay(runner, seqs, plan)
    assert runner.cache.num_free_blocks == 34 and runner.cache.slots.num_free == 4
    for r, t in seqs.items():
        check(together[r], cfg, w, t, dtype, f"{name} {r} in the batch")
        alone = replay(runner, {r: t}, [[(r, 0, len(t))]])[r]
        check(alone, cfg, w, t, dtype, f"{name} {r} alone")
        # beyond rounding, a request's logits do not depend on its company or on how it was cut:
        # the two runs are no further apart than each may be from the truth
        truth, plain_runs = plain_logits(cfg, w, t, dtype)
        close_to_truth(together[r], alone, [p + (alone - truth) for p in plain_runs], dtype,
                       f"{name} {r} against itself alone")


def test_pages_behind_the_window_come_back_while_a_request_lives(tmp_path_factory):
    folder, cfg, w = model_folder(tmp_path_factory, "a", torch.float32)
    runner = make_runner(folder, torch.float32, block_size=8, num_blocks=6)
    toks = prompts_for(cfg, [200], 6)["r0"]       # 25 pages if all were kept; a window of 19 needs 4 at most
    got = replay(runner, {"r0": toks}, in_portions("r0", 200, (24, 1, 9)))
    check(got["r0"], cfg, w, toks, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bs", [8, 16])
def test_one_key_among_hundreds_on_either_side_of_the_window(tmp_path, dtype, bs):
    """The marked token's key scores far above all others for every query; the logits follow
    whether it is just inside the window (visible) or just outside (gone), at page borders and
    in the middle of pages, read whole, in portions and token by token."""
    window = 37
    att = dict(heads=2, kv_heads=1, dim=16, vdim=16, window=window, rot_dims=4, scale=1.0, scaling=None)
    cfg = make_config(vocab=50, width=32, layers=[("attention", att, None)], loop=None,
                      embedding_scale=1.0, logit_softcap=None, eps=1e-6, max_positions=1024)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=5, dtype=NAME[dtype])
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    # token 1 is the marked one: its embedding lies along one axis that no other token uses; k
    # reads that axis into an unrotated element, every query has a constant there, v carries it on
    e = rand(50, 32, seed=1, scale=0.3)
    e[:, 0] = 0.0
    e[:, 1] = 1.0                       # a constant every token has: the queries' handle
    e[1] = 0.0
    e[1, 0] = 6.0
    wq, wk = torch.zeros(32, 32), torch.zeros(16, 32)
    wq[15, 1] = wq[31, 1] = 1.0         # element 15 of both heads: beyond the rotated four
    wk[15, 0] = 1.0
    wv = rand(16, 32, seed=2, scale=0.05)
    wv[:, 0] = rand(16, seed=3, scale=2.0)
    for k, t in (("embed", e), ("l0.mix.q", wq), ("l0.mix.k", wk), ("l0.mix.v", wv),
                 ("l0.mix.q.norm", torch.full((16,), 3.0)), ("l0.mix.k.norm", torch.full((16,), 3.0)),
                 ("l0.mix.o", rand(32, 32, seed=4, scale=0.5)), ("l0.mix.sink", torch.tensor([0.5, -2.0])),
                 ("head", rand(50, 32, seed=6, scale=0.5))):
        w[k] = t.to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})
    w = load_file(path)
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
def test_recurrence_carries_a_token_from_the_far_past(tmp_path, dtype):
    """An all-recurrent model (no pages at all) whose forget gate is held open: what token 0 was
    still shows in the logits hundreds of tokens later, through portions and single tokens and
    through a slot that others have used."""
    rec = dict(heads=2, dim=16, vdim=16, gate_cap=12.0)
    cfg = make_config(vocab=40, width=32, layers=[("mlstm", rec, None), ("mlstm", rec, None)], loop=(0, 2, 2),
                      embedding_scale=4.0, logit_softcap=None, eps=1e-6, max_positions=512)
    folder = str(tmp_path / "m")
    kvforge_amd.write_random_model(folder, cfg, seed=6, dtype=NAME[dtype])
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        if k.endswith(".f.b"):
            w[k] = torch.full_like(w[k], 9.0)         # log forget gate about -1e-4: nothing fades
        elif k.endswith(".i.b"):
            w[k] = torch.full_like(w[k], -1.0)
        elif k.endswith((".mix.v", ".mix.o", ".mix.q", ".mix.k", ".mix.g")):
            w[k] = (w[k].float() * 8.0).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})
    w = load_file(path)
    runner = make_runner(folder, dtype, block_size=8, num_blocks=4, seqs=2, tokens=512)
    assert runner.model.cache_groups == [] and len(runner.model.state_specs) == 4
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
    n = rng.randint(1, 5)
    layers = []
    for _ in range(n):
        if rng.random() < 0.55:
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 20, 32, 48, 64, 72])
            rot = rng.choice([r for r in (2, 4, 8, 16, 20, 32, 64) if r <= dim])
            scaling = rng.choice([None, {"factor": rng.choice([2.0, 8.0, 40.0]), "original": rng.choice([8, 64, 2048]),
                                         "fast": rng.choice([4.0, 32.0]), "slow": rng.choice([0.5, 1.0, 2.0])}])
            mixer = ("attention", dict(heads=kv * rng.choice([1, 2, 3, 4]), kv_heads=kv, dim=dim,
                                       vdim=rng.choice([8, 16, 24, 32, 40, 64, 80]),
                                       window=rng.choice([1, 2, 7, 16, 25, 40, 64, 300]), rot_dims=rot,
                                       scale=rng.choice([0.05, 0.125, 0.3, dim ** -0.5]), scaling=scaling,
                                       base=rng.choice([100.0, 10000.0, 500000.0])))
        else:
            mixer = ("mlstm", dict(heads=rng.choice([1, 2, 3, 5]), dim=rng.choice([4, 16, 24, 40, 64, 96, 144]),
                                   vdim=rng.choice([12, 16, 40, 64, 72, 130]), gate_cap=rng.choice([2.0, 15.0, 50.0])))
        moe = None
        if rng.random() > 0.2:
            E, I = rng.choice([1, 2, 5, 8, 16, 33]), rng.choice([0, 0, 1, 4])
            moe = dict(ff=rng.choice([8, 24, 31, 64]), experts=E, top=rng.randint(1, min(E + I, 6)), identity=I,
                       shared_ff=rng.choice([0, 16, 40]))
        layers.append((*mixer, moe))
    loop = None
    if rng.random() < 0.6:
        a = rng.randint(0, n - 1)
        loop = (a, rng.randint(a, n), rng.randint(1, 3))
    return make_config(vocab=rng.choice([17, 64, 100, 257, 512]), width=width, layers=layers, loop=loop,
                       embedding_scale=rng.choice([1.0, 3.3, width ** 0.5]),
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
    runner = make_runner(folder, dtype, block_size=bs, num_blocks=-(-260 // bs), seqs=3)
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
        assert runner.cache.num_free_blocks == -(-260 // bs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name, dtype):
    """The framework's own entry point and scheduler: prompts admitted in portions under a small
    token budget, decode steps replayed from captured graphs (the recurrent state advances on
    the device), three slots for five requests."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    engine = kvforge_amd.InferenceEngine.from_folder(
        folder, kvforge_amd.EngineConfig(
            cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=48), dtype=dtype,
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
    # in bfloat16 a few of the 200 rows may sit where the design multiplies rounding (see
    # ``plain_logits``); a lost state or key would miss nearly all of them
    assert len(missed) <= (0 if dtype == torch.float32 else 6), missed
    assert followed >= 4          # what comes out depends on more than the last token
    assert engine.cache.slots.num_free == 3 and engine.cache.num_free_blocks == 48
    if engine.runner.use_graphs:
        assert engine.runner.num_graph_replays > 0


def test_a_request_that_loses_its_pages_and_slot_is_read_again_from_its_first_token(tmp_path_factory):
    """Shape b keeps every key of one layer, so three requests outgrow the pool: the scheduler
    takes one's pages and state slot away and feeds it again later, prompt and generated tokens,
    into a slot and pages that others have used; its recurrence starts from zeros again."""
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
