"""Katarax on the GPU: each new or extended kernel alone against the plain stand-ins, keys just inside and outside
a window, among and behind the kept first positions and far back, the bias by distance by hand, the engine against
the plain implementation under every way of cutting requests into steps, long decoding through the captured step,
and the programs."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_katarax as pk
import plain_ops
from katarax_tiny import KT, KT_B, attention, latent, moe, random_config, unit, write_katarax
from paged_cases import DEV, attention_case, pages, rnd, run_logged, step_context
from replays import batch_steps, chunk_steps, requests_for, tail_steps, whole_steps
from tiny import random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# bfloat16 logits against the 64-bit plain implementation, as fractions of the logits' standard deviation, at three
# layers and growing with the root of their number beyond; 32-bit in absolute terms (times the logits' standard
# deviation where that is above one)
BF16_RMS, BF16_MAX, F32_ABS = 0.04, 0.2, 2e-4
SHARP = 3.0
# a router decides a token between two experts (or two groups) whose choice scores differ by less than this
# differently in bfloat16 than in 64 bits now and then: a bfloat16 run is compared with the plain implementation
# taking the run's own choices, which must be the plain router's wherever its margin is at least this
CLOSE_CALL = 0.02


def check(engine, steps, plain, reqs, dtype, what, loosen=1.0, f32_abs=F32_ABS):
    runs = plain.routed_runs()
    loosen = loosen * max(1.0, len(plain.cfg["layers"]) / 3.0) ** 0.5
    rows, routes = run_logged(engine, steps, runs)
    assert rows, "nothing was produced"
    for rid, toks in reqs.items():
        if not any(k[0] == rid for k in rows):
            continue
        forced = None
        if dtype != "float32" and runs:
            forced = {l: np.stack([routes[rid][l][p] for p in range(len(toks))]) for l in runs}
        margins, choices = [], []
        want_all = plain.forward(toks, routes=forced, margins=margins, choices=choices)
        for l, m, c in zip(runs, margins, choices):
            for p in range(len(toks)):
                if (rid, p) in rows and (dtype == "float32" or m[p] >= CLOSE_CALL):
                    assert sorted(routes[rid][l][p].tolist()) == sorted(c[p].tolist()), \
                        f"{what} [{dtype}]: request {rid} position {p} layer {l}: experts {routes[rid][l][p]} for {c[p]} (margin {m[p]:.4f})"
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
def _attend(form, q, kc, vc, table, pos, seq, lens, new, H, G, D, V, scale, window, keep_first, bias):
    """One launch of the attention in one of its forms; the result on the host."""
    from minfer_amd.kernels import ops
    if form == "stand-in":
        out = torch.empty(sum(new), H * V, dtype=q.dtype)
        plain_ops.capped_attn(q, kc, vc, table, pos, seq, torch.ones(H), out, H, G, D, V, scale, 0.0, window, max(lens),
                              keep_first=keep_first, bias=bias)
        return out.float()
    out = torch.empty(sum(new), H * V, dtype=q.dtype, device=DEV)
    ones = torch.ones(H, device=DEV)
    b = None if bias is None else bias.to(DEV)
    if form == "matrix cores":
        ops.capped_attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), step_context(lens, new, table, pos, seq), ones,
                                out, H, G, D, V, scale, 0.0, window, keep_first=keep_first, bias=b)
    else:
        ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), ones, out, H, G, D, V, scale,
                        0.0, window, max(lens), keep_first=keep_first, bias=b)
    return out.float().cpu()


_WANT = {}


@pytest.mark.parametrize("form, dtype", [("plain", torch.float32), ("plain", torch.bfloat16), ("matrix cores", torch.bfloat16)])
@pytest.mark.parametrize("H, G, D, V, window, keep, n_bias", [
    (6, 3, 32, 48, 17, 3, 9), (8, 2, 96, 48, 0, 0, 40), (4, 4, 16, 16, 64, 64, 0), (8, 2, 128, 64, 70, 5, 300),
    (7, 7, 48, 16, 1, 33, 2), (6, 2, 48, 48, 100, 1, 1), (6, 2, 128, 128, 65, 70, 0), (2, 1, 64, 128, 33, 32, 500),
    (9, 1, 10, 6, 5, 2, 7), (3, 3, 20, 12, 40, 130, 11), (4, 2, 256, 256, 40, 3, 50), (4, 4, 192, 80, 100, 0, 9)])
@pytest.mark.parametrize("new", [(1, 130, 3, 1, 40), (1, 64, 64, 300, 65), (1, 1, 1, 1, 1)])
def test_window_kept_first_positions_and_bias_in_both_attention_kernels(form, dtype, H, G, D, V, window, keep, n_bias, new):
    """Prompts, portions on held tokens and single tokens in one launch, over shuffled pages of a poisoned pool."""
    if form == "matrix cores" and (D % 16 or V % 16):
        pytest.skip("sizes the plain kernel takes")
    lens = (1, 130, 64, 300, 65)
    q, kc, vc, table, pos, seq, _ = attention_case(dtype, H, G, D, V, lens, new, 0, 0.0, 3)
    bias = rnd(H, n_bias, seed=9, scale=1.5) if n_bias else None
    case = (dtype, H, G, D, V, window, keep, n_bias, new)
    if case not in _WANT:            # the stand-in walks every (token, head, key) on the host: once per case
        _WANT[case] = _attend("stand-in", q, kc, vc, table, pos, seq, lens, new, H, G, D, V, 0.2, window, keep, bias)
    want = _WANT[case]
    got = _attend(form, q, kc, vc, table, pos, seq, lens, new, H, G, D, V, 0.2, window, keep, bias)
    err = (got - want).abs().max()
    assert torch.isfinite(got).all() and err < (2e-5 if dtype == torch.float32 else 4e-2), float(err)


# the last query stands at position 299: (window, kept first positions, the key's position, seen or not)
EDGES = [(17, 0, 283, True), (17, 0, 282, False), (64, 4, 236, True), (64, 4, 235, False), (64, 4, 3, True), (64, 4, 4, False),
         (65, 1, 0, True), (65, 1, 1, False), (100, 64, 63, True), (100, 64, 64, False), (100, 70, 69, True), (100, 70, 70, False),
         (40, 33, 32, True), (40, 33, 33, False), (1, 2, 299, True), (1, 2, 298, False), (1, 2, 1, True), (300, 0, 0, True),
         (299, 0, 0, False), (0, 0, 0, True), (236, 130, 129, True), (236, 0, 63, False)]


@pytest.mark.parametrize("form", ["plain float32", "plain bfloat16", "matrix cores"])
@pytest.mark.parametrize("window, keep, key, inside", EDGES)
def test_a_key_at_an_edge_decides_or_is_not_seen(form, window, keep, key, inside):
    """A key made to win the softmax with a value row of 50s: it decides the result where the query's window or
    the kept first positions hold it (also 299 positions back, across page edges and with a bias on every
    distance), and leaves no trace one position further; at the end of a prompt, of a portion, and for a single
    token."""
    H, G, D, V = 4, 2, 16, 16
    dtype = torch.float32 if form == "plain float32" else torch.bfloat16
    for lens, new in (((300, 90), (300, 20)), ((300, 90), (45, 1)), ((300, 90), (1, 1))):
        for bias in (None, rnd(H, 50, seed=2, scale=0.5)):
            q, kc, vc, table, pos, seq, _ = attention_case(dtype, H, G, D, V, lens, new, 0, 0.0, 5, needle=(0, key, 1))
            got = _attend("plain" if form.startswith("plain") else form, q, kc, vc, table, pos, seq, lens, new, H, G, D, V, 1.0,
                          window, keep, bias)
            row = got[new[0] - 1].view(H, V)
            if inside:
                assert (row[2:] - 50.0).abs().max() < 0.5, (lens, new, bias is not None)
            else:
                assert row[2:].abs().max() < 10.0, (lens, new, bias is not None)


def test_the_bias_by_distance_by_hand():
    """Two equal keys with different values, one 1 and one 200 positions back, and the other keys far below them:
    the farther one weighs exp(bias[far] - bias[1]) of the nearer; distances beyond the table take its last column."""
    from minfer_amd.kernels import ops
    H, G, D, V = 2, 1, 16, 16
    lens, new = (201,), (1,)
    table = pages(lens, 1)
    kc, vc = torch.zeros(40, G, 64, D), torch.zeros(40, G, 64, V)
    key = torch.zeros(D)
    key[3] = 2.0
    for p, val in ((0, 1.0), (199, 3.0)):
        kc[int(table[0, p // 64]), 0, p % 64] = key
        vc[int(table[0, p // 64]), 0, p % 64] = val
    for p in list(range(1, 199)) + [200]:
        kc[int(table[0, p // 64]), 0, p % 64] = -20.0 * key
    q = torch.cat([key, key]).view(1, H * D)
    bias = torch.zeros(H, 120)
    bias[0, 1], bias[0, 119], bias[1, 1], bias[1, 119] = 0.3, -0.9, -1.0, 0.5
    pos, seq = torch.tensor([200], dtype=torch.int32), torch.tensor([0], dtype=torch.int32)
    got = torch.empty(1, H * V, device=DEV)
    ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), torch.ones(H, device=DEV), got,
                    H, G, D, V, 1.0, 0.0, 0, 201, bias=bias.to(DEV))
    for h in range(H):
        ratio = float(torch.exp(bias[h, 119] - bias[h, 1]))
        assert abs(float(got[0, h * V]) - (ratio * 1.0 + 3.0) / (ratio + 1.0)) < 1e-4, h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, normed, rot, halves, q_only", [
    (6, 3, 24, 40, True, 16, True, False), (9, 1, 10, 10, False, 0, False, False), (2, 1, 12, 6, True, 2, True, False),
    (4, 4, 16, 16, True, 16, True, True), (2, 2, 64, 32, False, 64, True, False), (6, 2, 128, 64, True, 32, True, True),
    (3, 1, 130, 20, False, 0, False, True)])
def test_queries_and_keys_rotated_in_halves_and_queries_alone(dtype, H, G, D, V, normed, rot, halves, q_only):
    """Sequences that bring 1, 2, 70 and 5 tokens onto 0, 3, 60 and 127 held ones, into shuffled pages; a layer
    without keys and values of its own leaves the pages as they are."""
    from minfer_amd.cache.paged import v_page_shape
    from minfer_amd.kernels import ops
    held, new = (0, 3, 60, 127), (1, 2, 70, 5)
    C = H * D if q_only else H * D + G * D + G * V
    n = sum(new)
    qkv = rnd(n, C, seed=1, scale=2.0)
    seq = torch.repeat_interleave(torch.arange(4, dtype=torch.int32), torch.tensor(new)).to(torch.int32)
    pos = torch.cat([torch.arange(h, h + m) for h, m in zip(held, new)]).to(torch.int32)
    table = pages([h + m for h, m in zip(held, new)], 7)
    ang = torch.arange(256, dtype=torch.float64)[:, None]
    rt = None if not rot else tuple(f(ang * (100.0 ** (-2.0 * torch.arange(rot // 2) / rot))).float() for f in (torch.cos, torch.sin))
    outs = []
    for side in ("plain", "gpu"):
        dev = "cpu" if side == "plain" else DEV
        mv = lambda t: None if t is None else (tuple(x.to(dev) for x in t) if isinstance(t, tuple) else t.to(dev))
        kc = torch.full((40, G, 64, D), 7.0, dtype=dtype, device=dev)
        vc = torch.full((40,) + v_page_shape(G, V, dtype), 7.0, dtype=dtype, device=dev)
        q = torch.empty(n, H * D, dtype=dtype, device=dev)
        fn = plain_ops.qk_norm_prep if side == "plain" else ops.qk_norm_prep
        fn(mv(qkv), None, None, 1e-5, normed, mv(seq), mv(pos), mv(rt), None, False, mv(table), q, kc, vc, H, G, D, V, not q_only,
           halves=halves, q_only=q_only)
        outs.append([t.cpu().float() for t in (q, kc, vc)])
    tol = 3e-5 if dtype == torch.float32 else 1e-2
    for name, a, b in zip(("q", "k pages", "v pages"), *outs):
        assert ((a - b).abs() / b.abs().clamp(min=1.0)).max() < tol, name
    if q_only:
        assert bool((outs[1][1] == 7.0).all()) and bool((outs[1][2] == 7.0).all())
    if normed and dtype == torch.float32:       # the norm behind the rotation: every head has a root mean square of one
        rms = outs[1][0].view(n, H, D).pow(2).mean(dim=-1).sqrt()
        assert (rms - 1.0).abs().max() < 1e-4


def test_sigmoid_router_with_corrections_and_group_sums():
    from minfer_amd.kernels import ops
    for E, groups, keep, top, n, gt in ((6, 3, 2, 3, 40, 2), (8, 4, 3, 4, 33, 2), (8, 8, 2, 2, 9, 2), (4, 1, 1, 4, 5, 2), (9, 3, 1, 3, 17, 2),
                                        (12, 2, 1, 5, 64, 3), (1, 1, 1, 1, 2, 2), (16, 4, 2, 1, 21, 1)):
        want = [torch.empty(n, E), torch.empty(n, top, dtype=torch.int32), torch.empty(n, top)]
        got = [t.clone().to(DEV) for t in want]
        corr = rnd(E, seed=E + 2, scale=0.5) - 0.8          # choice scores on both sides of zero
        for xt in (torch.float32, torch.bfloat16):
            xr, wr = rnd(n, 70, seed=E).to(xt), rnd(E, 70, seed=E + 1, scale=0.3)
            kw = dict(score="sigmoid", group_top=gt, weight_scale=1.7)
            plain_ops.moe_route(xr, wr, want[0], want[1], want[2], groups, keep, correction=corr, **kw)
            ops.moe_route(xr.to(DEV), wr.to(DEV), got[0], got[1], got[2], groups, keep, correction=corr.to(DEV), **kw)
            assert torch.equal(got[1].cpu(), want[1]) and (got[2].cpu() - want[2]).abs().max() < 1e-5
            assert (got[0].cpu() - want[0]).abs().max() < 1e-5
            # the weights are the scores themselves over their sum, times the scale: the corrections are not in them
            s = torch.sigmoid(xr.double() @ wr.double().T)
            picked = torch.gather(s, 1, want[1].long())
            assert ((picked / picked.sum(dim=1, keepdim=True) * 1.7).float() - got[2].cpu()).abs().max() < 1e-5
            # every chosen expert lies in one of `keep` groups
            assert all(len({int(e) // (E // groups) for e in row}) <= keep for row in want[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [5, 40, 300])
def test_latent_preparation_with_a_query_latent_and_gates_per_value(dtype, n):
    """The three forms of the per-head matrices (plain, matrix cores from memory, a head's matrix in LDS) with a gate
    for every value; the preparation with queries that come as rows of their own; the norm over a row's front."""
    from minfer_amd.kernels import ops
    H, dn, dr, rank, dv, qr = 3, 16, 8, 40, 24, 24
    proj = rnd(n, qr + rank + dr + H * dv, seed=1, scale=2.0)
    q_rows = rnd(n, H * (dn + dr), seed=2, scale=2.0)
    w, qw = rnd(rank, seed=3) + 1.0, rnd(qr, seed=4) + 1.0
    lens = [n]
    table = pages(lens, 3)
    pos, seq = torch.arange(n, dtype=torch.int32), torch.zeros(n, dtype=torch.int32)
    ang = torch.arange(512, dtype=torch.float64)[:, None] * (100.0 ** (-2.0 * torch.arange(dr // 2) / dr))
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    res = []
    for side in ("plain", "gpu"):
        dev = "cpu" if side == "plain" else DEV
        o = plain_ops if side == "plain" else ops
        cache = torch.zeros(40, 64, rank + dr, dtype=dtype, device=dev)
        q_plain = torch.empty(n, H, dn, dtype=dtype, device=dev)
        q_abs = torch.zeros(n, H, rank + dr, dtype=dtype, device=dev)
        gate = torch.empty(n, H, dv, dtype=torch.float32, device=dev)
        c_q = torch.empty(n, qr, dtype=dtype, device=dev)
        o.rmsnorm(proj.to(dev), qw.to(dev), 1e-5, c_q, cols=qr)
        o.latent_prep(proj.to(dev), qr, qr + rank + dr, w.to(dev), 1e-5, cos.to(dev), sin.to(dev), pos.to(dev), seq.to(dev),
                      table.to(dev), cache, q_plain, q_abs, gate, H, dn, dr, rank, True, q_rows=q_rows.to(dev))
        x = (rnd(n, H, rank, seed=5)).to(dtype).to(dev)
        wt = (rnd(H, rank, dv, seed=6) / 6).to(dtype).to(dev)
        out = torch.empty(n, H, dv, dtype=dtype, device=dev)
        o.headwise_linear(x, rank, wt, out, dv, gate=gate)
        outs = [c_q, cache, q_plain, q_abs[:, :, rank:], gate, out]
        if dtype == torch.bfloat16:
            out2 = torch.empty(n, H, dv, dtype=dtype, device=dev)
            o.headwise_linear_mfma(x, rank, wt.transpose(1, 2).contiguous(), out2, dv, gate=gate)
            outs.append(out2)
        res.append([t.float().cpu() for t in outs])
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    for i, (a, b) in enumerate(zip(*res)):
        assert ((a - b).abs() / a.abs().clamp(min=1.0)).max() < tol, i
    z = rnd(7, 33, seed=8, scale=20.0)
    got = z.clone().to(DEV)
    ops.softcap(got, 12.5)
    assert (got.cpu() - 12.5 * torch.tanh(z / 12.5)).abs().max() < 1e-5


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("katarax")
    return {name: write_katarax(str(tmp / name), raw, seed=i) for i, (name, raw) in enumerate(KT.items())}


@pytest.fixture(scope="module")
def plains(folders):
    return {name: pk.PlainKatarax.from_folder(f) for name, f in folders.items()}


def engine_for(folder, dtype, max_tokens=64 * 16, **kw):
    from minfer_amd import Engine, load_model
    return Engine(load_model(folder, dtype=dtype, device="cuda:0"), max_tokens=max_tokens, poison_cache=True, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(KT))
def test_replays_agree_with_plain(folders, plains, name, dtype):
    """Whole; the last tokens one by one (the windows' edges pass over decoded tokens); unequal batches one after
    another (slots and pages used again over a poisoned pool); prompts in portions down to two tokens and one, alone
    and in mixed batches."""
    reqs = requests_for(KT[name]["vocab"], (1, 7, 64, 150, 65, 33, 290), seed=3)
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
def test_steps_in_which_nothing_or_little_is_wanted(folders, plains, dtype):
    """A prompt step that asks for no logits at all, then single tokens of which one sequence's are wanted."""
    eng = engine_for(folders["A"], dtype)
    toks = random_tokens(300, 100, 5)
    a, b = eng.new_sequence(), eng.new_sequence()
    assert tuple(eng.step([a, b], [toks[:90], toks[:50]], [[], []]).shape) == (0, 300)
    got_a = eng.step([a, b], [toks[90:91], toks[50:51]], [[0], []]).cpu().numpy()
    got_b = eng.step([a, b], [toks[91:92], toks[51:52]], [[], [0]]).cpu().numpy()
    assert got_a.shape == (1, 300) and got_b.shape == (1, 300)
    for got, n in ((got_a, 91), (got_b, 52)):
        want = plains["A"].forward(toks[:n])[-1]
        tol = F32_ABS * max(1.0, want.std()) if dtype == "float32" else SHARP * BF16_MAX * want.std()
        assert np.abs(got[0] - want).max() <= tol
    eng.end_sequence(a)
    eng.end_sequence(b)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_more_sequences_than_one_launch_of_the_experts_takes(folders, plains, dtype):
    """Twenty sequences that start and decode together: the routed layers' few-token form runs in slices."""
    reqs = requests_for(KT["A"]["vocab"], tuple(3 + (7 * i) % 11 for i in range(20)), seed=12)
    eng = engine_for(folders["A"], dtype, max_tokens=64 * 24)
    check(eng, batch_steps(reqs, [list(reqs)], prompt_frac=0.4), plains["A"], reqs, dtype, "twenty together")
    assert not eng.cache.live_slots()


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whatever config.json may say: sizes, orders and options drawn at random, both run types, whole, one by one,
    in batches and in portions."""
    raw = random_config(np.random.default_rng(9000 + seed))
    folder = write_katarax(str(tmp_path / "m"), raw, seed=seed)
    plain = pk.PlainKatarax.from_folder(folder)
    reqs = requests_for(raw["vocab"], (1, 9, 70, 200, 131), seed=seed)
    ids = list(reqs)
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(folder, dtype)
        what = f"random configuration {seed} ({json.dumps(raw)[:600]})"
        check(eng, whole_steps(reqs), plain, reqs, dtype, what + " whole", SHARP)
        check(eng, tail_steps(reqs, tail=33), plain, reqs, dtype, what + " one by one", SHARP)
        check(eng, batch_steps(reqs, [ids[:3], ids[3:]]), plain, reqs, dtype, what + " batches", SHARP)
        check(eng, chunk_steps(reqs, [ids[:2], ids[2:]]), plain, reqs, dtype, what + " portions", SHARP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_windows_and_long_decoding(tmp_path, dtype):
    """Scales and query matrices raised so that the softmax picks single keys (a key that a window wrongly holds or
    drops, a kept position lost, or a distance in the wrong bucket then moves a row by its whole size): a prompt of
    400 tokens whole, then as 250 + 150 one by one, with windows of 17, 64 and 70 whose edges pass over decoded
    tokens and page edges, kept positions of 3 and 65, and the causal layers over all 400."""
    raw = dict(architecture="Katarax", vocab=300, width=96, norm=dict(eps=1e-5), logit_softcap=20.0, layers=[
        dict(attention(4, 2, 32, 16, 0.2, 70, 3, 12, 100), mlp=moe(6, 2, 40, groups=3, keep=2, scale=1.5)),
        dict(latent(3, 16, 8, 24, 40, 24, 0.3, 17, base=1000.0), mlp=None),
        dict(unit(4, 2, 32, 32, 2.0, 16), mlp=moe(4, 1, 56)),
        dict(attention(2, 1, 16, 48, 0.3, 64, 65, 8, 300), mlp=None),
        dict(unit(4, 2, 32, 32, 1.5, 16, kv_from=2), mlp=moe(4, 2, 32, groups=2, keep=1)),
    ])
    folder = write_katarax(str(tmp_path / "sharp"), raw, seed=21, sharpen=4.0 if dtype == "float32" else 2.0)
    plain = pk.PlainKatarax.from_folder(folder)
    reqs = {"long": random_tokens(300, 400, 77)}
    eng = engine_for(folder, dtype, max_tokens=64 * 16)
    check(eng, whole_steps(reqs), plain, reqs, dtype, "sharp whole", SHARP, 1e-3)
    check(eng, tail_steps(reqs, tail=150), plain, reqs, dtype, "sharp 250 + 150 one by one", SHARP, 1e-3)


def test_greedy_generation_through_the_entry_point(folders, plains):
    """`LLM.generate`: the scheduler, slots used again (more prompts than slots), the captured decode step; 70 new
    tokens so that every sequence crosses a page edge and the windows' edges while decoding."""
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
            assert t == pk.greedy(row) or top[1] - top[0] < 1e-4, f"token {i}"
    bf = LLM(folders["A"], dtype="bfloat16", n_ctx=256, n_slots=4)
    a = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[]).tokens
    b = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False).tokens
    assert a == b


def test_programs(folders, plains, tmp_path):
    """bin/minfer generates greedily from a Katarax folder; bin/trace_run replays a batch."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "minfer"), folders["B"], "--prompt-tokens", "5,6,7;9",
                        "--greedy", "--repeat-penalty", "1.0", "-n", "4", "--dtype", "float32", "--n-ctx", "64",
                        "--stop-token", "100000"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.strip().splitlines() if l]
    for line, prompt in zip(lines, ([5, 6, 7], [9])):
        seq = list(prompt)
        for t in (int(x) for x in line.split(",")):
            assert t == pk.greedy(plains["B"].forward(seq)[-1])
            seq.append(t)
    vocab = KT_B["vocab"]
    reqs = requests_for(vocab, (3, 70, 20), seed=9)
    ref = {rid: plains["B"].forward(toks) for rid, toks in reqs.items()}
    steps = batch_steps(reqs, [list(reqs)])
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["B"], "--dtype",
                          "float32", "--out", out, "--max-tokens", "93"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                         text=True, bufsize=1)
    rows, pos = {}, {}
    try:
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            assert p.stdout.readline().strip() == f"done {st['step']}"
            arr = np.fromfile(os.path.join(out, f"{st['step']}.f32"), dtype="<f4").reshape(-1, vocab)
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
