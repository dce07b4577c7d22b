"""Fogorax on the GPU against the plain model of ``tests/plain/fogorax.py``: every new kernel
alone, then whole models of several shapes through the engine's own step function, cache
manager, scheduler and entry points, cut in every way a server cuts its work."""

from __future__ import annotations

import copy
import math
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import kvforge_amd
from kvforge_amd.config.presets import fogorax as make_config
from kvforge_amd.engine.batch import StepEntry
from kvforge_amd.engine.runner import ModelRunner
from kvforge_amd.models.transformer import Transformer
from tests import replay_util as ru
from tests.plain import fogorax as plain
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


# ============================================================================ kernels alone
def test_add_positions():
    x, table = rand(5, 24, seed=1), rand(9, 24, seed=2).bfloat16()
    pos = torch.tensor([3, 0, 8, 9, -1], dtype=torch.int32)        # the last two lie outside the table
    got = x.clone().to(DEV)
    ops().add_positions(got, table.to(DEV), pos.to(DEV))
    want = x.clone()
    want[:3] += table.float()[pos[:3].long()]
    torch.testing.assert_close(got.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [24, 200, 1031, 4100, 9001])
def test_norm_shift_over_runs_and_steps(dtype, h):
    """Three sequences in two steps; the second step continues two of them from their state
    slots and starts a new one in the slot the third gave back, which still holds its state."""
    eps, g = 1e-5, 1.3
    mu, w = rand(h, seed=3, scale=0.5), torch.full((h,), g)
    seqs = {"a": rand(9, h, seed=4), "b": rand(5, h, seed=5), "c": rand(1, h, seed=6), "d": rand(4, h, seed=7)}
    want = {r: (plain.scalar_norm(x, torch.tensor(g), eps),
                plain.token_shift(plain.scalar_norm(x, torch.tensor(g), eps), mu)) for r, x in seqs.items()}
    state = torch.full((4, h), 7.0, device=DEV)                     # junk: a slot's first user must not read it
    slot = {"a": 2, "b": 0, "c": 3, "d": 3}
    got = {r: ([], []) for r in seqs}
    for step in ([("a", 0, 6), ("b", 0, 1), ("c", 0, 1)], [("b", 1, 5), ("d", 0, 4), ("a", 6, 9)],):
        x = torch.cat([seqs[r][a:b] for r, a, b in step]).to(DEV)
        lens = [b - a for _, a, b in step]
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
        seq_of = torch.repeat_interleave(torch.arange(len(step)), torch.tensor(lens)).int().to(DEV)
        pos = torch.cat([torch.arange(a, b) for _, a, b in step]).int().to(DEV)
        slots = torch.tensor([slot[r] for r, _, _ in step], dtype=torch.int32, device=DEV)
        p, s = torch.empty(x.shape, dtype=dtype, device=DEV), torch.empty(x.shape, dtype=dtype, device=DEV)
        ops().norm_shift(x, w.to(DEV), mu.to(DEV), state, slots, seq_of, cu, pos, eps, p, s)
        off = 0
        for (r, a, b), n in zip(step, lens):
            got[r][0].append(p[off:off + n].float().cpu())
            got[r][1].append(s[off:off + n].float().cpu())
            off += n
    for r in seqs:
        torch.testing.assert_close(torch.cat(got[r][0]), want[r][0], **tol(dtype))
        torch.testing.assert_close(torch.cat(got[r][1]), want[r][1], **tol(dtype))
    # the slots hold the last normalised row of their last users, in 32-bit
    for r in ("a", "b", "d"):
        torch.testing.assert_close(state[slot[r]].cpu(), want[r][0][-1], atol=3e-5, rtol=3e-5)
    assert (state[1] == 7.0).all()


def test_norm_shift_leaves_sequences_without_a_slot_alone():
    h = 40
    x = rand(3, h, seed=8).to(DEV)
    state = torch.full((2, h), 5.0, device=DEV)
    p, s = torch.empty_like(x), torch.empty_like(x)
    i32 = dict(dtype=torch.int32, device=DEV)
    ops().norm_shift(x, torch.ones(h, device=DEV), torch.full((h,), 0.25, device=DEV), state,
                     torch.tensor([-1, 1, -1], **i32), torch.tensor([0, 1, 2], **i32),
                     torch.tensor([0, 1, 2, 3], **i32), torch.tensor([0, 4, 4], **i32), 1e-5, p, s)
    y = plain.rms(x.cpu(), 1e-5)
    torch.testing.assert_close(s[0].cpu(), 0.75 * y[0])                  # position 0: no predecessor
    torch.testing.assert_close(s[1].cpu(), 0.75 * y[1] + 0.25 * 5.0)     # from its slot
    torch.testing.assert_close(s[2].cpu(), 0.75 * y[2])                  # no slot: nothing to read
    assert (state[0] == 5.0).all()
    torch.testing.assert_close(state[1].cpu(), y[1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["gelu_tanh", "silu"])
@pytest.mark.parametrize("paired,bias", [(True, True), (False, True), (True, False)])
@pytest.mark.parametrize("inter", [37, 72])        # 72: four pairs per thread in bfloat16
def test_gated_act(dtype, activation, paired, bias, inter):
    m = 7
    gate, up = rand(m, inter, seed=1, scale=4.0).to(dtype), rand(m, inter, seed=2).to(dtype)
    bg, bu = (rand(inter, seed=3), rand(inter, seed=4)) if bias else (None, None)
    gu = torch.stack([gate, up], dim=2).reshape(m, 2 * inter) if paired else torch.cat([gate, up], dim=1)
    out = torch.empty(m, inter, dtype=dtype, device=DEV)
    ops().gated_act(gu.contiguous().to(DEV), out, activation, paired,
                    bg.to(DEV) if bias else None, bu.to(DEV) if bias else None)
    a = gate.float() + (bg if bias else 0.0)
    b = up.float() + (bu if bias else 0.0)
    act = plain.gelu_tanh(a) if activation == "gelu_tanh" else a * torch.sigmoid(a)
    torch.testing.assert_close(out.float().cpu(), act * b, **tol(dtype))
    with pytest.raises(ops().KernelError):
        ops().gated_act(gu.contiguous().to(DEV), out, "relu", paired)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sigmoid_gate_reads_a_block_of_columns(dtype):
    m, c = 5, 48
    y, wide = rand(m, c, seed=1).to(dtype), rand(m, 3 * c, seed=2, scale=3.0).to(dtype)
    got, dev = y.clone().to(DEV), wide.to(DEV)
    ops().sigmoid_gate(got, dev[:, c:2 * c])
    torch.testing.assert_close(got.float().cpu(), y.float() * torch.sigmoid(wide[:, c:2 * c].float()), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h,dim,extras", [(24, 3, "both"), (96, 8, "none"), (2500, 17, "bias"), (256, 64, "owed"),
                                          (2048, 64, "both"), (4096, 128, "bias"), (8200, 8, "none"), (40, 1024, "owed")])
@pytest.mark.parametrize("transposed", [False, True])
def test_token_side(dtype, h, dim, extras, transposed):
    """``transposed``: the projection is also given transposed, which lets rows of a multiple of
    eight elements take the kernel of 1,024 threads."""
    n, vocab, layers, layer = 6, 11, 3, 1
    x = rand(n, h, seed=1)
    side, gate, proj = (rand(vocab, layers * dim, seed=2).to(dtype), rand(dim, h, seed=3, scale=h ** -0.5).to(dtype),
                        rand(h, dim, seed=4).to(dtype))
    w = 1.0 + rand(h, seed=5, scale=0.1)
    bias = rand(h, seed=6) if extras in ("both", "bias") else None
    owed = rand(n, h, seed=7).to(dtype) if extras in ("both", "owed") else None
    tokens = torch.tensor([3, 0, 10, 11, -2, 7], dtype=torch.int32)       # two lie outside the table
    got = x.clone().to(DEV)
    ops().token_side(got, tokens.to(DEV), side.to(DEV), layer * dim, gate.to(DEV), proj.to(DEV), w.to(DEV),
                     1e-5, bias=None if bias is None else bias.to(DEV), owed=None if owed is None else owed.to(DEV),
                     proj_t=proj.t().contiguous().to(DEV) if transposed else None)
    base = x + (bias if bias is not None else 0.0) + (owed.float() if owed is not None else 0.0)
    known = (tokens >= 0) & (tokens < vocab)
    rows = side.float()[tokens.clamp(0, vocab - 1).long()][:, layer * dim:(layer + 1) * dim]
    want = base + plain.token_side(base, rows, gate.float(), proj.float(), w, 1e-5) * known[:, None]
    torch.testing.assert_close(got.cpu(), want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("extras", ["both", "none", "bias", "owed"])
def test_token_side_in_pieces_for_many_rows(dtype, extras):
    """The part's two routes give the same stream: one kernel for few rows, the matrix kernels
    with three row-wise kernels around them for many."""
    from kvforge_amd.engine.batch import Step, Workspace
    from kvforge_amd.parts import TokenSideInput

    n, h, dim, vocab = 70, 96, 24, 50
    part = TokenSideInput("l1.side", h, dim, vocab, "side.embed", 3 * dim, dim, 1e-5)
    part.load({"side.embed": rand(vocab, 3 * dim, seed=2).to(dtype).to(DEV),
               "l1.side.gate": rand(dim, h, seed=3, scale=h ** -0.5).to(dtype).to(DEV),
               "l1.side.proj": rand(h, dim, seed=4).to(dtype).to(DEV),
               "l1.side.norm": (1.0 + rand(h, seed=5, scale=0.1)).to(dtype).to(DEV)})
    x = rand(n, h, seed=1)
    bias = rand(h, seed=6).to(DEV) if extras in ("both", "bias") else None
    owed = rand(n, h, seed=7).to(dtype).to(DEV) if extras in ("both", "owed") else None
    tokens = torch.randint(-1, vocab + 1, (n,), generator=torch.Generator().manual_seed(8)).int()
    got = []
    for limit in (1 << 30, 0):
        part.FUSED_MAX_ROWS = limit
        step = Step()
        step.ws, step.act_dtype, step.device, step.token_ids = Workspace(DEV), dtype, DEV, tokens.to(DEV)
        res = x.clone().to(DEV)
        if owed is not None:
            step.owe(res, owed)
        part.forward(res, step, bias=bias)
        assert step.owed is None
        got.append(res.cpu())
    base = x + (bias.cpu() if bias is not None else 0.0) + (owed.float().cpu() if owed is not None else 0.0)
    known = (tokens >= 0) & (tokens < vocab)
    rows = part.table.float().cpu()[tokens.clamp(0, vocab - 1).long()][:, dim:2 * dim]
    want = base + plain.token_side(base, rows, part.gate.float().cpu(), part.proj.float().cpu(),
                                   part.weight.cpu(), 1e-5) * known[:, None]
    torch.testing.assert_close(got[0], want, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(got[1], want, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32
                                                 else dict(atol=4e-2, rtol=4e-2)))


@pytest.mark.parametrize("m", [1, 8, 33])
@pytest.mark.parametrize("activation,bias", [("gelu_tanh", True), ("silu", True), ("gelu_tanh", False)])
def test_gate_folded_into_the_projection(m, activation, bias):
    """The weight-streaming product with biases, activation and gate in its store against the
    product followed by the activation kernel."""
    k, inter = 96, 70
    a = rand(m, k, seed=1).bfloat16().to(DEV)
    w = ops().streamed(rand(2 * inter, k, seed=2, scale=k ** -0.5).bfloat16().to(DEV))
    bg, bu = (rand(inter, seed=3).to(DEV), rand(inter, seed=4).to(DEV)) if bias else (None, None)
    got = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    ops().gemm_gated(a, w, got, activation, bg, bu)
    c = a.float().cpu() @ w.plain.float().cpu().T
    g, u = c[:, 0::2] + (bg.cpu() if bias else 0.0), c[:, 1::2] + (bu.cpu() if bias else 0.0)
    want = (plain.gelu_tanh(g) if activation == "gelu_tanh" else g * torch.sigmoid(g)) * u
    torch.testing.assert_close(got.float().cpu(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("m", [1, 5, 40])
@pytest.mark.parametrize("own_kv", [True, False])
def test_projection_with_cache_write_carries_a_gates_columns(m, own_kv):
    """Rows of W behind q, k and v come out behind q; without k and v rows nothing is written."""
    H, KV, d, k, bs = 3, 1, 32, 64, 8
    kv = KV if own_kv else 0
    n = (H + 2 * kv) * d + H * d
    a = rand(m, k, seed=1).bfloat16().to(DEV)
    w = rand(n, k, seed=2, scale=k ** -0.5).bfloat16().to(DEV)
    pos = torch.arange(3, 3 + m, dtype=torch.int32, device=DEV)
    seq_of = torch.zeros(m, dtype=torch.int32, device=DEV)
    table = torch.arange(8, dtype=torch.int32, device=DEV).flip(0).reshape(1, 8).contiguous()
    kp = torch.zeros(8, KV, bs, d, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(8, KV, d, bs, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(m, 2 * H * d, dtype=torch.bfloat16, device=DEV)
    ops().gemm_qkv_rope(a, ops().streamed(w), out, pos, seq_of, None, None, table, kp, vp, H, kv, d,
                        write_kv=own_kv, extra_cols=H * d)
    c = (a.float() @ w.float().T).cpu()
    torch.testing.assert_close(out[:, :H * d].float().cpu(), c[:, :H * d], atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(out[:, H * d:].float().cpu(), c[:, n - H * d:], atol=2e-2, rtol=2e-2)
    if not own_kv:
        assert float(kp.abs().max()) == 0.0 and float(vp.abs().max()) == 0.0
        return
    for t in range(m):
        p = 3 + t
        page, off = 7 - p // bs, p % bs
        torch.testing.assert_close(kp[page, 0, off].float().cpu(), c[t, H * d:(H + 1) * d], atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(vp[page, 0, :, off].float().cpu(), c[t, (H + 1) * d:(H + 2) * d], atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("H,KV,d,bs", [(4, 2, 16, 8), (6, 2, 64, 16), (5, 1, 128, 16)])
@pytest.mark.parametrize("splits", [1, 3])
def test_attention_gates_its_output_as_it_stores_it(H, KV, d, bs, splits):
    """Query runs and single tokens on the matrix cores, the gate read from columns of the
    buffer that holds q."""
    dtype, window, keep = torch.bfloat16, 21, 2
    scale = 1 / math.sqrt(d)
    for seq_lens, q_lens in (([90, 33, 70], [40, 33, 2]), ([7, 90, 1, 300], [1, 1, 1, 1])):
        paged = Paged(seq_lens, KV, d, bs, dtype, seed=d)
        n = sum(q_lens)
        buf = rand(n, 2 * H * d, seed=d + 1).to(dtype)
        q = buf[:, :H * d].reshape(n, H, d)
        cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
        ctx = torch.tensor(seq_lens, dtype=torch.int32)
        want = masked_reference(paged, q, seq_lens, q_lens, scale, window, keep).reshape(n, H * d)
        want = want * torch.sigmoid(buf[:, H * d:].float())
        dev = buf.to(DEV)
        out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
        if max(q_lens) > 1:
            ops().attn_prefill(dev, paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), cu.to(DEV), ctx.to(DEV),
                               prefill_work(q_lens, H // KV, dtype, d, bs).to(DEV), out, H, KV, d, scale, window,
                               keep_first=keep, gate=dev[:, H * d:])
        else:
            ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV))
            ops().attn_decode(dev, paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, n, cu.to(DEV),
                              ctx.to(DEV), out, H, KV, d, scale, window, splits, ws, keep_first=keep,
                              gate=dev[:, H * d:])
        torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


def masked_reference(paged, q, seq_lens, q_lens, scale, window, keep):
    outs, off = [], 0
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        mask = plain.window_mask(n, window, keep)[n - ql:]
        outs.append(plain.masked_attention(q[off:off + ql].float(), paged.keys[s].float(),
                                           paged.values[s].float(), scale, mask))
        off += ql
    return torch.cat(outs)


def give_back_hidden_pages(paged, seq_lens, q_lens, bs, window, keep):
    """What the cache manager does while a request lives: pages that neither the window of the
    step's first query nor the kept first keys reach are no longer the sequence's, and whoever
    owns them now has written to them."""
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        first_live = max(0, n - ql - window + 1) // bs
        for b in range(-(-keep // bs), first_live):
            page = int(paged.table[s, b])
            paged.k[page] = float("nan")
            paged.v[page] = float("nan")
            paged.table[s, b] = -1


MASKS = [(11, 3), (40, 4), (64, 33), (5, 0), (7, 70), (33, 1), (1, 2), (2048, 4)]
SHAPES = [(4, 2, 16, 4), (6, 2, 32, 8), (3, 1, 48, 16), (8, 2, 64, 16), (32, 8, 64, 16), (4, 1, 128, 32), (5, 5, 80, 24)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", SHAPES)
@pytest.mark.parametrize("window,keep", MASKS)
def test_attention_of_query_runs_keeps_the_first_keys(dtype, H, KV, d, bs, window, keep):
    seq_lens, q_lens = [200, 131, 77, 9], [67, 131, 2, 9]
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + window)
    give_back_hidden_pages(paged, seq_lens, q_lens, bs, window, keep)
    n = sum(q_lens)
    buf = rand(n, (H + 2 * KV) * d, seed=d).to(dtype)
    q = buf[:, :H * d].reshape(n, H, d)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor(seq_lens, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    want = masked_reference(paged, q, seq_lens, q_lens, scale, window, keep).reshape(n, H * d)
    for tiles in (1, 2):
        per_item = ops().prefill_rows_per_item(dtype, d, bs, tiles)
        out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
        ops().attn_prefill(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), cu.to(DEV),
                           ctx.to(DEV), prefill_work(q_lens, H // KV, dtype, d, bs, tiles).to(DEV), out,
                           H, KV, d, scale, window, rows_per_item=per_item, keep_first=keep)
        torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,d,bs", SHAPES)
@pytest.mark.parametrize("window,keep", MASKS)
@pytest.mark.parametrize("splits", [1, 3])
def test_attention_of_single_tokens_keeps_the_first_keys(dtype, H, KV, d, bs, window, keep, splits):
    seq_lens = [7, 13, 1, 41, 300, 64, 65, 130]
    q_lens = [1] * len(seq_lens)
    paged = Paged(seq_lens, KV, d, bs, dtype, seed=d + H + keep)
    give_back_hidden_pages(paged, seq_lens, q_lens, bs, window, keep)
    n = len(seq_lens)
    buf = rand(n, (H + 2 * KV) * d, seed=d).to(dtype)
    q = buf[:, :H * d].reshape(n, H, d)
    cu, ctx = torch.arange(n + 1, dtype=torch.int32), torch.tensor(seq_lens, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    want = masked_reference(paged, q, seq_lens, q_lens, scale, window, keep).reshape(n, H * d)
    ws = (torch.empty(n * H * splits * d, device=DEV), torch.empty(n * H * splits * 2, device=DEV))
    out = torch.zeros(n, H * d, dtype=dtype, device=DEV)
    ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, n, cu.to(DEV),
                      ctx.to(DEV), out, H, KV, d, scale, window, splits, ws, keep_first=keep)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("single", [False, True])
def test_one_key_that_stands_out_is_seen_exactly_where_the_mask_says(dtype, single):
    """Among 500 keys one has a score far above the rest.  Placed just inside the window, or
    among the kept first keys, it is all the query sees; placed just outside either, the output
    must not know of it.  Checked at page borders too (pages of 16, window of 48, 5 kept)."""
    H, KV, d, bs, window, keep, n = 2, 1, 32, 16, 48, 5, 500
    scale = 1 / math.sqrt(d)
    qv = torch.zeros(d)
    qv[0] = 8.0
    for place in (n - 1, n - window, n - window - 1, keep - 1, keep, 0, 15, 16, n - window + 3, 447, 448):
        def stand_out(kk, place=place):
            kk = kk * 0.1
            kk[place, :, 0] = 30.0
            return kk
        paged = Paged([n], KV, d, bs, dtype, seed=place, shape_keys=stand_out)
        ql = 1 if single else 3
        give_back_hidden_pages(paged, [n], [ql], bs, window, keep)
        buf = torch.zeros(ql, (H + 2 * KV) * d)
        buf[:, :H * d] = qv.repeat(H)
        buf = buf.to(dtype)
        cu, ctx = torch.tensor([0, ql], dtype=torch.int32), torch.tensor([n], dtype=torch.int32)
        out = torch.zeros(ql, H * d, dtype=dtype, device=DEV)
        if single:
            ops().attn_decode(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), None, 1,
                              cu.to(DEV), ctx.to(DEV), out, H, KV, d, scale, window, 1, None, keep_first=keep)
        else:
            ops().attn_prefill(buf.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), cu.to(DEV),
                               ctx.to(DEV), prefill_work([ql], H // KV, dtype, d, bs).to(DEV), out, H, KV, d,
                               scale, window, keep_first=keep)
        got = out.float().cpu()[-1, :d]
        visible = place < keep or (n - 1) - place < window
        value = paged.values[0][place, 0].float()
        if visible:
            torch.testing.assert_close(got, value, **tol(dtype))
        else:
            assert (got - value).abs().max() > 0.5, place
        q = buf[:, :H * d].reshape(ql, H, d)
        want = masked_reference(paged, q, [n], [ql], scale, window, keep).reshape(ql, H * d)
        torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


# ============================================================================ whole models
def shape_a() -> dict:
    """Groups of three query heads, value heads larger than key heads, neither a size the
    kernels take as it is; every other layer reads the cache of the one before."""
    return make_config(vocab=211, width=72, layers=4, heads=6, kv_heads=2, dim=24, vdim=40, ff=100,
                       window=13, keep_first=3, side_dim=5, max_positions=400, share_every=2)


def shape_b() -> dict:
    """Every layer another mask; layers 2 and 3 read layers 0 and 1 through other windows than
    theirs; one layer without a feed-forward; no per-layer token input; an odd width."""
    cfg = make_config(vocab=97, width=44, layers=4, heads=4, kv_heads=4, dim=16, vdim=16, ff=52,
                      window=9, keep_first=0, side_dim=0, max_positions=400, share_every=1, eps=1e-3)
    cfg["layers"][1]["mixer"]["mask"] = {"keep_first": 6, "size": 17}
    cfg["layers"][2]["mixer"].update(kv_from=0, mask={"keep_first": 2, "size": 30}, scale=0.4)
    cfg["layers"][3]["mixer"].update(kv_from=1, mask={"keep_first": 1, "size": 5})
    cfg["layers"][1]["mlp"] = None
    cfg["layers"][2]["mlp"]["ff"] = 31
    return cfg


def shape_c() -> dict:
    """One kv head under eight query heads at head size 64, a window longer than any request
    here, a per-layer input as wide as a head."""
    return make_config(vocab=300, width=128, layers=2, heads=8, kv_heads=1, dim=64, ff=256,
                       window=1000, keep_first=4, side_dim=64, max_positions=400, share_every=1)


def shape_d() -> dict:
    """Layers wide enough for what serving a real model takes: tiled weights, a down projection
    deep and narrow enough to be cut in two halves of K (one half stays owed to the stream until
    the per-layer input takes it), gate/up wide enough for two groups of columns a wave, the
    kernel of 1,024 threads for the per-layer input."""
    return make_config(vocab=1000, width=256, layers=2, heads=4, kv_heads=2, dim=64, ff=4096,
                       window=50, keep_first=3, side_dim=24, max_positions=400, share_every=2)


SHAPE = {"a": shape_a, "b": shape_b, "c": shape_c, "d": shape_d}


def liven(folder: str) -> None:
    """Random weights as drawn give nearly flat attention, and layers that add little to the
    embedding: a lost key or state would hide.  Queries and keys are scaled up so that attention
    is peaked, values and outputs so that the layers outweigh the embedding, the shift vector so
    that a good part of every token comes from the one before."""
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        leaf = k.rsplit(".", 1)[-1]
        if ".mix." in k and leaf in ("q", "k"):
            w[k] = (w[k].float() * 12.0).to(w[k].dtype)
        elif (".mix." in k and leaf in ("v", "o", "g")) or k.endswith(".mlp.down"):
            w[k] = (w[k].float() * 6.0).to(w[k].dtype)
        elif k.endswith(".b"):
            w[k] = (w[k].float() * 10.0).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})


_MODELS: dict = {}


def model_folder(tmp_path_factory, name: str, dtype) -> tuple[str, dict, dict]:
    key = (name, dtype)
    if key not in _MODELS:
        folder = str(tmp_path_factory.mktemp(f"fogorax_{name}_{NAME[dtype]}"))
        cfg = SHAPE[name]()
        kvforge_amd.write_random_model(folder, cfg, seed=len(name) + 11, dtype=NAME[dtype])
        liven(folder)
        _MODELS[key] = (folder, cfg, load_file(os.path.join(folder, "model.safetensors")))
    return _MODELS[key]


def make_runner(folder, dtype, block_size=8, num_blocks=64, seqs=4, tokens=256, use_graphs=True):
    model = Transformer.from_folder(folder, dtype, DEV)
    return ModelRunner(model, block_size, num_blocks, max_num_seqs=seqs, max_num_batched_tokens=tokens,
                       max_model_len=model.config.max_position_embeddings, use_graphs=use_graphs)


def replay(runner, seqs: dict, plan) -> dict:
    """``plan``: steps of (request, from, to); all logits are asked for.  Pages behind the
    windows are given back after every step and a request's pages and slot when it ends."""
    got = {r: [] for r in seqs}
    cache = runner.cache
    for step in plan:
        entries = []
        for rid, a, b in step:
            if not cache.has_request(rid):
                cache.allocate(rid, 0)
            cache.append_slots(rid, b, a)
            entries.append(StepEntry(rid, seqs[rid][a:b], a, "all"))
        logits = runner.step(entries).cpu()
        off = 0
        for rid, a, b in step:
            got[rid].append(logits[off:off + b - a].clone())
            off += b - a
            cache.release_behind(rid, b)
            if b == len(seqs[rid]):
                cache.free(rid)
    return {r: torch.cat(v) for r, v in got.items() if v}


def row_error(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: the root mean square of the difference (its mean taken off) over the mean spread
    of the wanted logits."""
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().mean()


def close_to_plain(got: torch.Tensor, want: torch.Tensor, dtype, what="", rounded: torch.Tensor | None = None) -> None:
    """32-bit: a fixed small share of the logits' spread.  bfloat16: peaked attention multiplies
    what rounding queries and keys to eight bits does, so the bound is measured, not widened:
    ``rounded`` is the plain model run with the roundings a bfloat16 engine may make
    (``plain.forward(store=bfloat16)``), and a row may be off by three times what that run is
    off in the same row (or the fixed share, if that is more).  A lost key, state or page moves a row
    by about the whole spread, twenty times any of these."""
    err = row_error(got, want)
    limit = torch.full_like(err, 2e-4 if dtype == torch.float32 else 3e-2)
    if rounded is not None and dtype != torch.float32:
        off = row_error(rounded, want)
        # (the largest of hundreds of rows is a wide-tailed thing: a row is also allowed one and
        # a half times what the worst row of the rounded run is off)
        limit = torch.maximum(limit, torch.maximum(3.0 * off, 1.5 * off.max()))
    worst = int((err / limit).argmax())
    assert float(err[worst]) <= float(limit[worst]), (
        f"{what}: position {worst} is off by {float(err[worst]):.3e} of the logits' spread "
        f"(allowed {float(limit[worst]):.3e})")


_WANT: dict = {}


def plain_logits(cfg, w, toks, dtype):
    """(32-bit logits, logits with bfloat16 roundings or None) of the plain model."""
    key = (id(w), tuple(toks), dtype)
    if key not in _WANT:
        _WANT[key] = (plain.forward(cfg, w, toks),
                      plain.forward(cfg, w, toks, store=torch.bfloat16) if dtype == torch.bfloat16 else None)
    return _WANT[key]


def check(got, cfg, w, toks, dtype, what=""):
    want, rounded = plain_logits(cfg, w, toks, dtype)
    close_to_plain(got, want, dtype, what, rounded)


def prompts_for(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def in_portions(rid, n, sizes):
    out, p, k = [], 0, 0
    while p < n:
        m = min(sizes[k % len(sizes)], n - p)
        out.append([(rid, p, p + m)])
        p, k = p + m, k + 1
    return out


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


def test_the_stream_after_every_layer(tmp_path_factory):
    """Layer by layer in 32-bit: the engine's residual stream after each block against the plain
    model's, so that a fault names its layer."""
    folder, cfg, w = model_folder(tmp_path_factory, "a", torch.float32)
    runner = make_runner(folder, torch.float32)
    toks = prompts_for(cfg, [60], 2)["r0"]
    want: list = []
    plain.forward(cfg, w, toks, layers_out=want)
    runner.cache.allocate("x", 0)
    runner.cache.append_slots("x", len(toks), 0)
    step, _ = runner.build_step([StepEntry("x", toks, 0, "all")])
    model = runner.model
    with torch.inference_mode():
        residual = model.embed(step)
        for p in model.spec.positions:
            p.on_embedding(residual, step)
        for i, (call, ls) in enumerate(zip(model.order, model.layer_states)):
            model.spec.blocks[call.layer].forward(residual, step, ls)
            step.settle()
            torch.testing.assert_close(residual.cpu(), want[i], atol=2e-4, rtol=2e-4, msg=lambda m: f"layer {i}: {m}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(SHAPE))
def test_decoding_token_by_token_equals_the_prompt_read_at_once(tmp_path_factory, name, dtype):
    """From the first token on, and from a prompt's end, far past every window and kept key."""
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
    # keys and values of every position for the layers without a window to speak of, of the
    # window's reach for the others: r3 alone needs 15 pages of 8 where nothing is given back
    runner = make_runner(folder, dtype, block_size=8, num_blocks=34, seqs=4)
    together = replay(runner, seqs, plan)
    assert runner.cache.num_free_blocks == 34 and runner.cache.slots.num_free == 4
    for r, t in seqs.items():
        check(together[r], cfg, w, t, dtype, f"{name} {r} in the batch")
        alone = replay(runner, {r: t}, [[(r, 0, len(t))]])[r]
        check(alone, cfg, w, t, dtype, f"{name} {r} alone")
        if dtype == torch.float32:
            # beyond rounding, a request's logits do not depend on its company or on how it was cut
            close_to_plain(together[r], alone, dtype, f"{name} {r} against itself alone")


def test_pages_behind_the_window_come_back_while_a_request_lives(tmp_path_factory):
    folder, cfg, w = model_folder(tmp_path_factory, "a", torch.float32)
    runner = make_runner(folder, torch.float32, block_size=8, num_blocks=10)
    toks = prompts_for(cfg, [200], 6)["r0"]       # 25 pages if all were kept; the window needs 3 and the kept keys 1
    got = replay(runner, {"r0": toks}, in_portions("r0", 200, (24, 1, 9)))
    check(got["r0"], cfg, w, toks, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation_through_the_engine(tmp_path_factory, name, dtype):
    """The framework's own entry point and scheduler: prompts admitted in portions under a small
    token budget, decode steps replayed from captured graphs (the state advances on the
    device), three slots for five requests."""
    folder, cfg, w = model_folder(tmp_path_factory, name, dtype)
    engine = kvforge_amd.InferenceEngine.from_folder(
        folder, kvforge_amd.EngineConfig(
            cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=48), dtype=dtype,
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=24, max_model_len=256)))
    prompts = list(prompts_for(cfg, [30, 2, 11, 45, 1], 7).values())
    outs = engine.generate(prompts, kvforge_amd.SamplingParams(max_tokens=40, temperature=0.0, ignore_eos=True))
    margin = 1e-3 if dtype == torch.float32 else 0.25
    followed = 0
    for p, o in zip(prompts, outs):
        assert len(o.output_token_ids) == 40
        logits = plain.forward(cfg, w, p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= margin * float(row.std()), (i, tok)
        followed += o.output_token_ids != plain.greedy(cfg, w, p[-1:], 40)
    assert followed >= 4          # what comes out depends on more than the last token
    assert engine.cache.slots.num_free == 3 and engine.cache.num_free_blocks == 48
    if engine.runner.use_graphs:
        assert engine.runner.num_graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_parallel_block_without_shift_or_anything_behind_it(dtype):
    """The block as another design would use it: a norm with a weight vector, plain attention
    (no gate, no window) and a silu feed-forward without biases side by side."""
    from kvforge_amd.engine.batch import MetaBuffers, Step, Workspace, fill_step
    from kvforge_amd.cache.manager import CacheGroup, CacheManager
    from kvforge_amd.parts import GatedFeedForward, LayerState, PagedAttention, ParallelBlock, RMSNorm

    h, H, KV, d, ff, n, bs = 48, 4, 2, 16, 40, 21, 8
    block = ParallelBlock(RMSNorm("n", h, 1e-5), PagedAttention("a", h, H, KV, d, None, scale=0.2),
                          GatedFeedForward("f", h, ff), h)
    assert block.state_spec is None
    names = {k: rand(*v.shape, seed=i, scale=0.3) + (1.0 if v.init == "norm" else 0.0)
             for i, (k, v) in enumerate(sorted(block.weight_specs().items()))}
    block.load({k: t.to(dtype).to(DEV) for k, t in names.items()})
    block.seal()
    w = {k: t.to(dtype).float() for k, t in names.items()}
    x = rand(n, h, seed=50)
    cache = CacheManager(bs, [CacheGroup((0,), block.mixer.cache_spec.pages)], 8)
    cache.allocate("s", 0)
    layer = LayerState(group=0, pages={"k": torch.zeros(8, KV, bs, d, dtype=dtype, device=DEV),
                                       "v": torch.zeros(8, KV, d, bs, dtype=dtype, device=DEV)})
    meta, ws, got = MetaBuffers(64, 4, [8], DEV), Workspace(DEV), []
    for a, b in ((0, 13), (13, 14), (14, 21)):
        cache.append_slots("s", b, a)
        step = Step()
        step.ws, step.act_dtype, step.device = ws, dtype, DEV
        fill_step(step, meta, [StepEntry("s", list(range(a, b)), a, "all")], cache.block_table, lambda r: -1, bs)
        res = x[a:b].clone().to(DEV)
        block.forward(res, step, layer)
        step.settle()
        got.append(res.cpu())
    hn = plain.rms(x, 1e-5) * w["n.weight"]
    q, k, v = (hn @ w[f"a.{m}_proj.weight"].T for m in "qkv")
    o = plain.masked_attention(q.view(n, H, d), k.view(n, KV, d), v.view(n, KV, d), 0.2,
                               plain.window_mask(n, n, 0)).reshape(n, H * d)
    g = hn @ w["f.gate_proj.weight"].T
    want = x + o @ w["a.o_proj.weight"].T + (g * torch.sigmoid(g) * (hn @ w["f.up_proj.weight"].T)) @ w["f.down_proj.weight"].T
    torch.testing.assert_close(torch.cat(got), want, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32
                                                         else dict(atol=6e-2, rtol=6e-2)))


def random_shape(seed: int) -> dict:
    """A model whose every size, count, constant and layer order is drawn: widths that are no
    multiple of 8, head sizes that are no multiple of 16, query/key and value sizes apart, any
    group size, windows from one key up, kept keys from none up, layers that read any earlier
    layer with keys of its own (each reader with a mask of its own), layers without a
    feed-forward, with and without the per-layer input."""
    import random
    rng = random.Random(seed)
    kv_heads = rng.choice([1, 2, 3])
    heads = kv_heads * rng.choice([1, 2, 3, 4])
    dim, vdim = rng.choice([8, 16, 20, 32, 48, 64, 72]), rng.choice([8, 16, 24, 32, 40, 64, 80])
    width = rng.choice([24, 36, 50, 64, 88, 100, 128, 200])
    n = rng.randint(1, 6)
    layers, owners = [], []
    for i in range(n):
        mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim,
                 "mask": {"keep_first": rng.choice([0, 0, 1, 2, 5, 9, 17]), "size": rng.choice([1, 2, 7, 16, 25, 40, 64, 300])},
                 "scale": rng.choice([0.05, 0.125, 0.3, dim ** -0.5])}
        if owners and rng.random() < 0.5:
            mixer["kv_from"] = rng.choice(owners)
        else:
            owners.append(i)
        mlp = None if rng.random() < 0.2 else {"ff": rng.choice([8, 31, 64, 130, 256]), "kind": "dense"}
        layers.append({"mixer": mixer, "mlp": mlp, "type": "attention"})
    side = rng.choice([0, 1, 6, 8, 16, 40])
    return {"architecture": "Fogorax", "layers": layers, "max_positions": 256,
            "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3, 0.1])},
            "token_side": {"dim": side} if side else None,
            "vocab": rng.choice([17, 64, 100, 257, 512]), "width": width}


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
    got: dict = {}
    for r, v in replay_all(runner, seqs, plan).items():
        got[r] = v
    for r, t in seqs.items():
        for k, logits in enumerate(got[r]):
            check(logits, cfg, w, t, dtype, f"seed {seed}, {r}, pass {k}: {cfg}")
    assert runner.cache.slots.num_free == 3 and runner.cache.num_free_blocks == -(-260 // bs)


def replay_all(runner, seqs, plan) -> dict:
    """Like ``replay`` for a plan that reads requests more than once: a list of whole-sequence
    logits per request, one per time it was read to its end."""
    out = {r: [] for r in seqs}
    part = {r: [] for r in seqs}
    cache = runner.cache
    for step in plan:
        entries = []
        for rid, a, b in step:
            if not cache.has_request(rid):
                cache.allocate(rid, 0)
            cache.append_slots(rid, b, a)
            entries.append(StepEntry(rid, seqs[rid][a:b], a, "all"))
        logits = runner.step(entries).cpu()
        off = 0
        for rid, a, b in step:
            part[rid].append(logits[off:off + b - a].clone())
            off += b - a
            cache.release_behind(rid, b)
            if b == len(seqs[rid]):
                cache.free(rid)
                out[rid].append(torch.cat(part[rid]))
                part[rid] = []
    return out


def test_a_request_that_loses_its_pages_and_slot_is_read_again_from_its_first_token(tmp_path_factory):
    """Nothing is given back behind this shape's window, so three requests outgrow the pool:
    the scheduler takes one's pages and state slot away and feeds it again later, prompt and
    generated tokens, into a slot and pages that others have used."""
    folder, cfg, w = model_folder(tmp_path_factory, "c", torch.float32)
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
    a pool of exactly the peak of live tokens."""
    folder, cfg, w = model_folder(tmp_path_factory, "a", {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    prompts = prompts_for(cfg, [37, 81, 100, 53], 8)
    tb = ru.TraceBuilder()
    names = {}
    for rid, toks in prompts.items():
        for mode, fn in (("w", ru.whole), ("d", ru.decode_tail), ("p", ru.portions)):
            names[f"{rid}#{mode}"] = toks
            fn(tb, f"{rid}#{mode}", toks)
    mixed = {f"{rid}#m": toks for rid, toks in prompts.items()}
    names.update(mixed)
    ru.mixed(tb, mixed, 9)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out, user_args=["--max-live", "4"])
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    want = {rid: plain_logits(cfg, w, toks, td) for rid, toks in prompts.items()}
    import numpy as np
    for sid, rows in enumerate(tb.expect):
        if not rows:
            continue
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{sid}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())
        ref = torch.stack([want[rid.split("#")[0]][0][pos] for rid, pos in rows])
        rounded = None if td == torch.float32 else torch.stack([want[rid.split("#")[0]][1][pos] for rid, pos in rows])
        close_to_plain(got, ref, td, f"step {sid}", rounded)
