"""Lagedra on the GPU: each new kernel alone against the plain stand-ins, the engine against the plain
implementation under every way of cutting requests into steps, keys just inside and outside the
windows that decide the result, long decoding through the captured step, and the programs."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_lagedra as pl
import plain_ops
from lagedra_tiny import LG, LG_A, LG_C, attention, dense, random_config, write_lagedra
from replays import batch_steps, chunk_steps, requests_for, run_steps, tail_steps, whole_steps
from paged_cases import (DEV, attention_case as _attention_case, pages as _pages, rnd, run_logged,
                         step_context as _step_context)
from tiny import random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# bfloat16 logits against the 64-bit plain implementation, as fractions of the logits' standard
# deviation (measured 0.5 to 1.5 % rms at three and four layers); 32-bit in absolute terms
BF16_RMS, BF16_MAX, F32_ABS = 0.04, 0.2, 2e-4
SHARP = 3.0        # where the queries are scaled up so that single keys decide, the scores' roundings grow with them
# A router decides a token between two experts (or groups) whose logits differ by less than this differently
# in bfloat16 than in 64 bits now and then (seen at margins of 0.001 to 0.003); the token's row then differs
# by a whole expert and the layers behind carry the difference on.  So a bfloat16 run is compared with the
# plain implementation taking the run's own choices (`routes=`), and the choices themselves must be the
# plain router's wherever its margin is at least this.  The 32-bit comparison forces nothing.
CLOSE_CALL = 0.02


def check(engine, steps, plain, reqs, dtype, what, loosen=1.0, f32_abs=F32_ABS):
    """Runs the steps and compares every row with the plain implementation.  32-bit: as it decides itself.
    bfloat16: taking the run's choices of experts, which must be the plain router's own except at close calls."""
    layers = plain.routed_layers()
    rows, routes = run_logged(engine, steps, layers)
    assert rows, "nothing was produced"
    for rid, toks in reqs.items():
        if not any(k[0] == rid for k in rows):
            continue
        forced = None
        if dtype != "float32" and layers:
            forced = {l: np.stack([routes[rid][l][p] for p in range(len(toks))]) for l in layers}
        margins, choices = [], []
        want_all = plain.forward(toks, routes=forced, margins=margins, choices=choices)
        for l, m, c in zip(layers, margins, choices):      # the run's choices are the plain router's, close calls aside
            for p in range(len(toks)):
                if (rid, p) in rows and (dtype == "float32" or m[p] >= CLOSE_CALL):
                    assert sorted(routes[rid][l][p].tolist()) == sorted(c[p].tolist()), \
                        f"{what} [{dtype}]: request {rid} position {p} layer {l}: experts {routes[rid][l][p]} for {c[p]}"
        for p in range(len(toks)):
            if (rid, p) not in rows:
                continue
            got, want = rows[(rid, p)], want_all[p]
            assert np.isfinite(got).all(), f"{what}: non-finite logits at request {rid} position {p}"
            diff = got.astype(np.float64) - want
            if dtype == "float32":
                assert np.abs(diff).max() <= f32_abs * max(1.0, want.std()), \
                    f"{what} [float32]: request {rid} position {p} of {len(toks)}: {np.abs(diff).max():.3e}"
            else:
                rms, std = float(np.sqrt(np.mean(diff * diff))), float(want.std())
                assert rms <= loosen * BF16_RMS * std and np.abs(diff).max() <= loosen * BF16_MAX * std, \
                    f"{what} [bfloat16]: request {rid} position {p} of {len(toks)}: rms {rms / std:.3f}, max {np.abs(diff).max() / std:.3f}"


# ------------------------------------------------------------------ kernels alone
def test_position_rows_gelu_and_weighted_sums():
    from minfer_amd.kernels import ops
    table, pos_table = rnd(50, 72, seed=1).bfloat16(), rnd(30, 72, seed=2).bfloat16()
    ids = torch.tensor([3, 49, 0, 7], dtype=torch.int32)
    pos = torch.tensor([0, 29, 5, 5], dtype=torch.int32)
    want, got = torch.empty(4, 72), torch.empty(4, 72, device=DEV)
    plain_ops.embed_pos(table, pos_table, ids, pos, want)
    ops.embed_pos(table.to(DEV), pos_table.to(DEV), ids.to(DEV), pos.to(DEV), got)
    assert torch.equal(got.cpu(), want)
    x = rnd(9, 130, seed=3, scale=3.0)
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 2e-2)):
        want, got = torch.empty(9, 130, dtype=dtype), torch.empty(9, 130, dtype=dtype, device=DEV)
        plain_ops.gelu_tanh(x, want)
        ops.gelu_tanh(x.to(DEV), got)
        assert (got.cpu().float() - want.float()).abs().max() < tol
    for n in (2, 5, 40):                        # 40: more buffers than a launch takes
        bufs = [rnd(11, 70, seed=10 + j) for j in range(n - 1)] + [rnd(4, 70, seed=99)]
        w, idx = rnd(n, seed=5), torch.tensor([10, 0, 3, 3], dtype=torch.int32)
        want, got = torch.empty(4, 70), torch.empty(4, 70, device=DEV)
        plain_ops.weighted_sum(bufs, w, want, idx, n - 1)
        ops.weighted_sum([b.to(DEV) for b in bufs], w.to(DEV), got, idx.to(DEV), n - 1)
        assert (got.cpu() - want).abs().max() < 1e-5
        want, got = torch.empty(11, 70), torch.empty(11, 70, device=DEV)
        plain_ops.weighted_sum(bufs[:-1], w[:-1].contiguous(), want)
        ops.weighted_sum([b.to(DEV) for b in bufs[:-1]], w[:-1].contiguous().to(DEV), got)
        assert (got.cpu() - want).abs().max() < 1e-5


@pytest.mark.parametrize("heads, dim, vdim, lens", [(3, 20, 12, (1, 5, 200, 64, 129)), (1, 40, 72, (700,)),
                                                    (2, 136, 16, (3, 128, 65)), (3, 5, 7, (1, 1, 1)), (2, 128, 130, (300, 2))])
def test_lightning_scan_kernels(heads, dim, vdim, lens):
    """Ragged sequences, carried state, shuffled slots; the sequential and the chunked form."""
    from minfer_amd.kernels import ops
    n = sum(lens)
    proj = rnd(n, 2 * heads * (dim + vdim), seed=1)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    slots = torch.tensor(np.random.default_rng(0).permutation(len(lens) + 2)[:len(lens)], dtype=torch.int32)
    decays = torch.tensor(np.random.default_rng(1).uniform(0.3, 1.0, heads), dtype=torch.float32)
    state0 = rnd(len(lens) + 2, heads, dim, vdim, seed=2, scale=0.5)
    want, st_want = torch.empty(n, heads * vdim), state0.clone()
    plain_ops.lightning_scan(proj, cu, slots, decays, st_want, want, heads, dim, vdim)
    table, count = ops.la_chunks(list(lens))
    for chunks in (None, (table.to(DEV), count)):
        got, st = torch.empty(n, heads * vdim, device=DEV), state0.clone().to(DEV)
        ops.lightning_scan(proj.to(DEV), cu.to(DEV), slots.to(DEV), decays.to(DEV), st, got, heads, dim, vdim, chunks)
        scale = float(want.abs().max())
        assert (got.cpu() - want).abs().max() < 2e-5 * scale, "outputs" + (" (chunked)" if chunks else "")
        assert (st.cpu() - st_want).abs().max() < 2e-5 * float(st_want.abs().max()), "state"
    o, w = rnd(n, heads * vdim, seed=3, scale=4.0), rnd(heads * vdim, seed=4) + 1
    off = 2 * heads * dim + heads * vdim
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        y_want, y = torch.empty(n, heads * vdim, dtype=dtype), torch.empty(n, heads * vdim, dtype=dtype, device=DEV)
        plain_ops.gated_rmsnorm(o, proj, off, w, 1e-5, y_want)
        ops.gated_rmsnorm(o.to(DEV), proj.to(DEV), off, w.to(DEV), 1e-5, y)
        assert (y.cpu().float() - y_want.float()).abs().max() < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, taps, rot", [(6, 3, 24, 40, 4, 16), (9, 1, 8, 24, 1, 4), (2, 1, 12, 5, 3, 2),
                                                   (4, 4, 16, 16, None, 0), (2, 2, 64, 32, 6, 64)])
def test_convolution_rotation_blend_and_cache_write(dtype, H, G, D, V, taps, rot):
    """Sequences that bring 1, 2, 70 and 5 tokens onto 0, 3, 60 and 127 held ones: the rows before a
    portion come from the carried state, which is moved on."""
    from minfer_amd.kernels import ops
    held, new = (0, 3, 60, 127), (1, 2, 70, 5)
    C = H * D + G * (D + V)
    n = sum(new)
    qkv = rnd(n, C, seed=1)
    conv = None if taps is None else rnd(C, taps, seed=2)
    K = 0 if taps is None else taps - 1
    state0 = rnd(6, max(K, 1), C, seed=3)[:, :K].contiguous()
    cu = torch.tensor(np.concatenate([[0], np.cumsum(new)]), dtype=torch.int32)
    seq = torch.repeat_interleave(torch.arange(4, dtype=torch.int32), torch.tensor(new)).to(torch.int32)
    slots = torch.tensor([4, 0, 5, 2], dtype=torch.int32)
    pos = torch.cat([torch.arange(h, h + m) for h, m in zip(held, new)]).to(torch.int32)
    table = _pages([h + m for h, m in zip(held, new)], 7)
    cos = sin = None
    if rot:
        cos, sin = rnd(256, rot // 2, seed=4), rnd(256, rot // 2, seed=5)
    v_first = rnd(n, G * V, seed=6)
    outs = []
    for side in ("plain", "gpu"):
        dev = "cpu" if side == "plain" else DEV
        mv = lambda t: None if t is None else t.to(dev)
        kc = torch.zeros(40, G, 64, D, dtype=dtype, device=dev)
        from minfer_amd.cache.paged import v_page_shape
        vc = torch.zeros((40,) + v_page_shape(G, V, dtype), dtype=dtype, device=dev)
        q = torch.empty(n, H * D, dtype=dtype, device=dev)
        own = torch.empty(n, G * V, device=dev)
        st = state0.clone().to(dev)
        fn = plain_ops.qkv_conv_prep if side == "plain" else ops.qkv_conv_prep
        fn(mv(qkv), mv(conv), st if K else None, mv(cu), mv(seq), mv(slots), mv(pos), mv(cos), mv(sin), 0.3, mv(v_first), own,
           mv(table), q, kc, vc, H, G, D, V, True)
        outs.append([t.cpu().float() for t in (q, kc, vc, own, st)])
    tol = 2e-5 if dtype == torch.float32 else 5e-2
    for name, a, b in zip(("q", "k pages", "v pages", "own values", "state"), *outs):
        if a.numel() == 0:
            continue
        assert (a - b).abs().max() < (2e-5 if name in ("own values", "state") else tol), name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, window, cap", [(6, 3, 24, 40, 17, 8.0), (9, 1, 8, 24, 5, 0.0), (2, 1, 12, 5, 1, 30.0),
                                                     (4, 4, 16, 16, 0, 0.0), (16, 2, 128, 64, 70, 50.0)])
def test_capped_attention_kernel_against_plain(dtype, H, G, D, V, window, cap):
    """Prompts, portions on held tokens and single tokens in one launch, over shuffled pages."""
    from minfer_amd.kernels import ops
    lens, new = (1, 130, 64, 300, 65), (1, 130, 3, 1, 40)
    q, kc, vc, table, pos, seq, temp = _attention_case(dtype, H, G, D, V, lens, new, window, cap, 3)
    want = torch.empty(sum(new), H * V, dtype=dtype)
    plain_ops.capped_attn(q, kc, vc, table, pos, seq, temp, want, H, G, D, V, 0.2, cap, window, max(lens))
    got = torch.empty(sum(new), H * V, dtype=dtype, device=DEV)
    ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), temp.to(DEV), got, H, G, D, V,
                    0.2, cap, window, max(lens))
    err = (got.cpu().float() - want.float()).abs().max()
    assert torch.isfinite(got).all() and err < (2e-5 if dtype == torch.float32 else 4e-2), float(err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window, back, inside", [(17, 16, True), (17, 17, False), (70, 69, True), (70, 70, False),
                                                  (0, 299, True), (65, 64, True), (64, 64, False), (1, 0, True), (1, 1, False)])
def test_a_key_at_the_window_edge_decides_or_is_not_seen(dtype, window, back, inside):
    """A key `back` positions behind the last query, made to win the softmax with a value row of 50s: it
    decides the result where the window holds it (also 299 positions back without a window, and across
    page edges), and leaves no trace one position further; in a prompt and for a single token."""
    from minfer_amd.kernels import ops
    H, G, D, V = 4, 2, 16, 8
    for lens, new in (((300, 90), (300, 1)), ((300, 90), (1, 1))):
        q, kc, vc, table, pos, seq, temp = _attention_case(dtype, H, G, D, V, lens, new, window, 0.0, 5,
                                                           needle=(0, 299 - back, 1))
        got = torch.empty(sum(new), H * V, dtype=dtype, device=DEV)
        ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), temp.to(DEV), got, H, G,
                        D, V, 1.0, 0.0, window, 300)
        row = got[new[0] - 1].float().cpu().view(H, V)
        if inside:
            assert (row[2:] - 50.0).abs().max() < 0.5, (lens, new)
        else:
            assert row[2:].abs().max() < 10.0, (lens, new)


@pytest.mark.parametrize("H, G, D, V, window, cap", [(6, 3, 32, 48, 17, 8.0), (8, 2, 96, 48, 40, 30.0), (4, 4, 16, 16, 0, 0.0),
                                                     (16, 2, 128, 64, 70, 50.0), (7, 7, 48, 16, 1, 0.0), (2, 1, 64, 128, 33, 2.0)])
@pytest.mark.parametrize("new", [(1, 130, 3, 1, 40), (1, 64, 64, 300, 65), (1, 1, 1, 2, 17), (1, 1, 1, 1, 1)])
def test_capped_attention_matrix_core_kernel(H, G, D, V, window, cap, new):
    """The matrix-core form against the plain one: whole prompts, portions on held tokens and single tokens in
    one launch, blocks of 16 tokens that end inside a sequence, and a decode step (one token a sequence: the
    keys split over several waves and merged), over shuffled pages of a poisoned pool."""
    from minfer_amd.kernels import ops
    lens = (1, 130, 64, 300, 65)
    q, kc, vc, table, pos, seq, temp = _attention_case(torch.bfloat16, H, G, D, V, lens, new, window, cap, 4)
    want = torch.empty(sum(new), H * V, dtype=torch.bfloat16)
    plain_ops.capped_attn(q, kc, vc, table, pos, seq, temp, want, H, G, D, V, 0.2, cap, window, max(lens))
    got = torch.empty(sum(new), H * V, dtype=torch.bfloat16, device=DEV)
    ctx = _step_context(lens, new, table, pos, seq)
    ops.capped_attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx, temp.to(DEV), got, H, G, D, V, 0.2, cap,
                            window)
    err = (got.cpu().float() - want.float()).abs().max()
    assert torch.isfinite(got).all() and err < 4e-2, float(err)


@pytest.mark.parametrize("window, back, inside", [(17, 16, True), (17, 17, False), (70, 69, True), (70, 70, False),
                                                  (0, 299, True), (65, 64, True), (64, 64, False), (33, 32, True), (32, 32, False)])
def test_matrix_core_form_a_key_at_the_window_edge(window, back, inside):
    from minfer_amd.kernels import ops
    H, G, D, V = 4, 2, 16, 16
    for lens, new in (((300, 90), (300, 20)), ((300, 90), (1, 1))):          # a prompt; a decode step with key splits
        q, kc, vc, table, pos, seq, temp = _attention_case(torch.bfloat16, H, G, D, V, lens, new, window, 0.0, 5,
                                                           needle=(0, 299 - back, 1))
        got = torch.empty(sum(new), H * V, dtype=torch.bfloat16, device=DEV)
        ops.capped_attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), _step_context(lens, new, table, pos, seq),
                                temp.to(DEV), got, H, G, D, V, 1.0, 0.0, window)
        row = got[new[0] - 1].float().cpu().view(H, V)
        assert ((row[2:] - 50.0).abs().max() < 0.5) if inside else (row[2:].abs().max() < 10.0), (lens, new)


def test_router_and_experts_kernels():
    from minfer_amd.kernels import ops
    for E, groups, keep, top, n in ((6, 3, 2, 3, 40), (8, 4, 4, 8, 5), (4, 1, 1, 1, 3), (64, 8, 3, 6, 33), (5, 5, 2, 2, 1)):
        want = [torch.empty(n, E), torch.empty(n, top, dtype=torch.int32), torch.empty(n, top)]
        got = [t.clone().to(DEV) for t in want]
        for xt in (torch.float32, torch.bfloat16):
            xr, wr = rnd(n, 70, seed=E).to(xt), rnd(E, 70, seed=E + 1, scale=0.3)
            plain_ops.moe_route(xr, wr, want[0], want[1], want[2], groups, keep)
            ops.moe_route(xr.to(DEV), wr.to(DEV), got[0], got[1], got[2], groups, keep)
            assert torch.equal(got[1].cpu(), want[1]) and (got[0].cpu() - want[0]).abs().max() < 1e-5
            assert (got[2].cpu() - want[2]).abs().max() < 1e-5
        F, K, N = 24, 72, 40
        gu = rnd(n, E * 2 * F, seed=2, scale=2.0)
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
            y_want, y = torch.empty(n, E * F, dtype=dtype), torch.empty(n, E * F, dtype=dtype, device=DEV)
            plain_ops.moe_act(gu, want[0], y_want, 1.5)
            ops.moe_act(gu.to(DEV), got[0], y, 1.5)
            assert (y.cpu().float() - y_want.float()).abs().max() < tol
            x, w1, w2 = rnd(n, K, seed=3).to(dtype), (rnd(E, 2 * F, K, seed=4) / 8).to(dtype), (rnd(E, N, F, seed=5) / 5).to(dtype)
            o_want, o = rnd(n, N, seed=6), rnd(n, N, seed=6).to(DEV)
            few = min(n, 16)             # the step sizes the sparse form takes
            plain_ops.moe_sparse(x[:few], w1, w2, want[1][:few], want[2][:few], o_want[:few], E, 1.5)
            ops.moe_sparse(x[:few].contiguous().to(DEV), w1.to(DEV), w2.to(DEV), got[1][:few].contiguous(),
                           got[2][:few].contiguous(), o[:few], E, 1.5)
            assert (o.cpu()[:few] - o_want[:few]).abs().max() < (1e-4 if dtype == torch.float32 else 5e-2)
        # the grouping of the pairs by expert, the rows side by side and the weighted sums back
        rank_want, counts_want = torch.empty(n, top, dtype=torch.int32), torch.empty(E, dtype=torch.int32)
        rank, counts = rank_want.clone().to(DEV), counts_want.clone().to(DEV)
        plain_ops.moe_group(want[1], E, rank_want, counts_want)
        ops.moe_group(got[1], E, rank, counts)
        assert torch.equal(rank.cpu(), rank_want) and torch.equal(counts.cpu(), counts_want) and int(counts_want.sum()) == n * top
        offsets = torch.cat([torch.zeros(1, dtype=torch.int32), counts_want.cumsum(0)[:-1].to(torch.int32)])
        xr = rnd(n, 70, seed=8).bfloat16()
        xs_want, xs = torch.zeros(n * top, 70, dtype=torch.bfloat16), torch.zeros(n * top, 70, dtype=torch.bfloat16, device=DEV)
        plain_ops.moe_gather(xr, want[1], rank_want, offsets, xs_want)
        ops.moe_gather(xr.to(DEV), got[1], rank, offsets.to(DEV), xs)
        assert torch.equal(xs.cpu(), xs_want)
        rows = rnd(n * top, 50, seed=9)
        o_want, o = rnd(n, 50, seed=10), rnd(n, 50, seed=10).to(DEV)
        plain_ops.moe_combine(rows, want[1], rank_want, offsets, want[2], o_want)
        ops.moe_combine(rows.to(DEV), got[1], rank, offsets.to(DEV), got[2], o)
        assert (o.cpu() - o_want).abs().max() < 1e-5


def test_half_rotation_tables_and_kernel():
    from minfer_amd.kernels import ops
    from minfer_amd.parts.rotary import blended_frequencies
    sc = dict(factor=4.0, original=64, fast=8.0, slow=2.0)
    freqs, mag = blended_frequencies(12, 500.0, sc)
    f_plain, mag_plain = pl.yarn_frequencies(12, 500.0, sc)
    assert np.allclose(freqs, f_plain) and mag == pytest.approx(mag_plain)
    cos, sin = ops.rope_table_freqs(300, freqs, mag, DEV)
    rows = rnd(7, 5 * 20, seed=1)
    pos = torch.tensor([0, 1, 63, 64, 200, 299, 7], dtype=torch.int32)
    got = rows.clone().to(DEV)
    ops.rope_half_inplace(got, cos, sin, pos.to(DEV), 3, 5, 20)
    x = rows.double().numpy().reshape(7, 5, 20)
    want = x.copy()
    want[:, :3] = pl.rotate_half(x[:, :3], pos.numpy(), 12, 500.0, sc)
    assert np.abs(got.cpu().numpy().reshape(7, 5, 20) - want).max() < 1e-5


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("lagedra")
    return {name: write_lagedra(str(tmp / name), raw, seed=i) for i, (name, raw) in enumerate(LG.items())}


@pytest.fixture(scope="module")
def plains(folders):
    return {name: pl.PlainLagedra.from_folder(f) for name, f in folders.items()}


def engine_for(folder, dtype, max_tokens=64 * 16, **kw):
    from minfer_amd import Engine, load_model
    return Engine(load_model(folder, dtype=dtype, device="cuda:0"), max_tokens=max_tokens, poison_cache=True, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(LG))
def test_replays_agree_with_plain(folders, plains, name, dtype):
    """Whole; the last tokens one by one (the windows pass over decoded tokens); unequal batches one after
    another (slots, pages and states used again); prompts in portions down to two tokens and one, alone
    and in mixed batches."""
    reqs = requests_for(LG[name]["vocab"], (1, 7, 64, 150, 65, 33, 290), seed=3)
    ids = list(reqs)
    eng = engine_for(folders[name], dtype)
    plain = plains[name]
    check(eng, whole_steps(reqs), plain, reqs, dtype, f"{name} whole")
    check(eng, tail_steps(reqs, tail=80), plain, reqs, dtype, f"{name} last 80 one by one")
    check(eng, batch_steps(reqs, [ids[:4], ids[4:]]), plain, reqs, dtype, f"{name} unequal batches")
    check(eng, chunk_steps(reqs, [ids[:3], ids[3:]]), plain, reqs, dtype, f"{name} portions in batches")
    check(eng, chunk_steps(reqs, [[r] for r in ids], sizes=(2,)), plain, reqs, dtype, f"{name} portions of 2")
    check(eng, chunk_steps(reqs, [[r] for r in ids], sizes=(129, 3, 64)), plain, reqs, dtype, f"{name} portions of 129")
    assert not eng.cache.live_slots()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_more_sequences_than_one_launch_of_the_experts_takes(folders, plains, dtype):
    """Twenty sequences that start and decode together: the routed layers' few-token form runs in slices."""
    reqs = requests_for(LG["A"]["vocab"], tuple(3 + (7 * i) % 11 for i in range(20)), seed=12)
    eng = engine_for(folders["A"], dtype, max_tokens=64 * 24)
    check(eng, batch_steps(reqs, [list(reqs)], prompt_frac=0.4), plains["A"], reqs, dtype, "twenty together")
    assert not eng.cache.live_slots()


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whatever config.json may say: sizes, orders and options drawn at random, both run types, whole, one
    by one, in batches and in portions."""
    raw = random_config(np.random.default_rng(3000 + seed))
    folder = write_lagedra(str(tmp_path / "m"), raw, seed=seed)
    plain = pl.PlainLagedra.from_folder(folder)
    reqs = requests_for(raw["vocab"], (1, 9, 70, 200, 131), seed=seed)
    ids = list(reqs)
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(folder, dtype)
        what = f"random configuration {seed} ({json.dumps(raw)[:300]})"
        check(eng, whole_steps(reqs), plain, reqs, dtype, what + " whole", SHARP)
        check(eng, tail_steps(reqs, tail=33), plain, reqs, dtype, what + " one by one", SHARP)
        check(eng, batch_steps(reqs, [ids[:3], ids[3:]]), plain, reqs, dtype, what + " batches", SHARP)
        check(eng, chunk_steps(reqs, [ids[:2], ids[2:]]), plain, reqs, dtype, what + " portions", SHARP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_windows_and_long_decoding(tmp_path, dtype):
    """Queries scaled so that the softmax picks single keys (a key that a window wrongly holds or drops
    then moves a row by its whole size): a prompt of 400 tokens whole, then as 250 + 150 one by one, with
    windows of 17 and 70 passing over decoded tokens and page edges, and without a window."""
    raw = dict(LG_A, layers=list(LG_A["layers"]) + [dict(attention(2, 1, 16, 24, 0.5, rot_dims=8, base=100.0), mlp=dense(64))])
    folder = write_lagedra(str(tmp_path / "sharp"), raw, seed=21, sharpen=4.0 if dtype == "float32" else 2.0)
    plain = pl.PlainLagedra.from_folder(folder)
    reqs = {"long": random_tokens(300, 400, 77)}
    eng = engine_for(folder, dtype, max_tokens=64 * 16)
    check(eng, whole_steps(reqs), plain, reqs, dtype, "sharp whole", SHARP, 1e-3)
    check(eng, tail_steps(reqs, tail=150), plain, reqs, dtype, "sharp 250 + 150 one by one", SHARP, 1e-3)


def test_greedy_generation_through_the_entry_point(folders, plains):
    """`LLM.generate`: the scheduler, slots used again (more prompts than slots), the captured decode step;
    70 new tokens so that every sequence crosses a page edge and the windows while decoding."""
    from minfer_amd import LLM
    llm = LLM(folders["A"], dtype="float32", n_ctx=256, n_slots=2)
    prompts = [random_tokens(300, n, 30 + i) for i, n in enumerate((5, 60, 1, 17))]
    res = llm.generate(prompts, max_new=70, temp=0.0, repeat_penalty=1.0, stop_tokens=[])
    eager = llm.generate(prompts, max_new=70, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False)
    assert res.tokens == eager.tokens
    for p, toks in zip(prompts, res.tokens):
        assert len(toks) == 70
        logits = plains["A"].forward(list(p) + toks)
        for i, t in enumerate(toks):
            row = logits[len(p) + i - 1]
            top = np.sort(row)[-2:]
            assert t == pl.greedy(row) or top[1] - top[0] < 1e-4, f"token {i}"
    bf = LLM(folders["A"], dtype="bfloat16", n_ctx=256, n_slots=4)
    a = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[]).tokens
    b = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False).tokens
    assert a == b


def test_programs(folders, plains, tmp_path):
    """bin/minfer generates greedily from a Lagedra folder; bin/trace_run replays a batch."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "minfer"), folders["C"], "--prompt-tokens", "5,6,7;9",
                        "--greedy", "--repeat-penalty", "1.0", "-n", "4", "--dtype", "float32", "--n-ctx", "64",
                        "--stop-token", "100000"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.strip().splitlines() if l]
    for line, prompt in zip(lines, ([5, 6, 7], [9])):
        seq = list(prompt)
        for t in (int(x) for x in line.split(",")):
            assert t == pl.greedy(plains["C"].forward(seq)[-1])
            seq.append(t)
    reqs = requests_for(97, (3, 70, 20), seed=9)
    ref = {rid: plains["C"].forward(toks) for rid, toks in reqs.items()}
    steps = batch_steps(reqs, [list(reqs)])
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["C"], "--dtype",
                          "float32", "--out", out, "--max-tokens", "93"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                         text=True, bufsize=1)
    rows, pos = {}, {}
    try:
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            assert p.stdout.readline().strip() == f"done {st['step']}"
            arr = np.fromfile(os.path.join(out, f"{st['step']}.f32"), dtype="<f4").reshape(-1, 97)
            i = 0
            for e in st["entries"]:
                for w in e["want"]:
                    rows[(e["id"], pos.get(e["id"], 0) + w)] = arr[i]
                    i += 1
                pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()
    for (rid, p), got in rows.items():
        assert np.abs(got - ref[rid][p]).max() <= F32_ABS * max(1.0, ref[rid][p].std()), f"trace_run: request {rid} position {p}"
