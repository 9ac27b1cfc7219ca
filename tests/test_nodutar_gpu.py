"""Nodutar on the GPU: each new kernel alone against the plain stand-ins, keys just inside and outside a
chunk and far behind under the penalty on distance, the engine against the plain implementation under every
way of cutting requests into steps, long decoding through the captured step, and the programs."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_nodutar as pn
import plain_ops
from nodutar_tiny import ND, ND_A, ND_B, attention, left, moe, parallel, random_config, right, write_nodutar
from paged_cases import DEV, attention_case, pages, rnd, run_logged, step_context
from replays import batch_steps, chunk_steps, requests_for, tail_steps, whole_steps
from tiny import random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# bfloat16 logits against the 64-bit plain implementation, as fractions of the logits' standard deviation, at
# three runs of a layer and growing with the root of their number beyond (every run adds roundings of its own:
# the engine's own composition on host stand-ins that round at the same places and compute in 64 bits in
# between differs from the plain implementation by up to 3.4 % rms at the six runs of "A"); 32-bit in absolute terms (times the logits' standard deviation where that is above one)
BF16_RMS, BF16_MAX, F32_ABS = 0.04, 0.2, 2e-4
SHARP = 3.0
# a router decides a token between two experts whose logits differ by less than this differently in bfloat16
# than in 64 bits now and then (its input is a normed stream that has been through several layers' roundings,
# about one percent of logits of size one): a bfloat16 run is compared with the plain implementation taking the
# run's own choices, which must be the plain router's wherever its margin is at least this
CLOSE_CALL = 0.05


def check(engine, steps, plain, reqs, dtype, what, loosen=1.0, f32_abs=F32_ABS):
    runs = plain.routed_runs()
    loosen = loosen * max(1.0, len(pn.run_order(plain.cfg)) / 3.0) ** 0.5
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
                        f"{what} [{dtype}]: request {rid} position {p} run {l}: experts {routes[rid][l][p]} for {c[p]} (margin {m[p]:.4f})"
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
@pytest.mark.parametrize("heads, dim, vdim, lens", [(3, 20, 12, (1, 5, 200, 64, 129)), (1, 40, 72, (700,)),
                                                    (2, 136, 16, (3, 128, 65)), (3, 5, 7, (1, 1, 1)), (2, 128, 130, (300, 2)),
                                                    (5, 32, 48, (1, 1, 1, 1, 1, 1, 1)), (1, 256, 8, (66,))])
def test_gated_scan_kernels(heads, dim, vdim, lens):
    """Ragged sequences, carried state, shuffled slots; the sequential and the chunked form; the norm per head."""
    from minfer_amd.kernels import ops
    n = sum(lens)
    proj = rnd(n, heads * (2 * dim + vdim), seed=1, scale=1.5)
    lower = torch.tensor(np.random.default_rng(1).uniform(0.0, 0.95, heads * dim), dtype=torch.float32)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    slots = torch.tensor(np.random.default_rng(0).permutation(len(lens) + 2)[:len(lens)], dtype=torch.int32)
    state0 = rnd(len(lens) + 2, heads, dim, vdim, seed=2, scale=0.5)
    want, st_want = torch.empty(n, heads * vdim), state0.clone()
    plain_ops.gated_scan(proj, lower, cu, slots, st_want, want, heads, dim, vdim)
    table, count = ops.gr_chunks(list(lens))
    for chunks in (None, (table.to(DEV), count)):
        got, st = torch.empty(n, heads * vdim, device=DEV), state0.clone().to(DEV)
        ops.gated_scan(proj.to(DEV), lower.to(DEV), cu.to(DEV), slots.to(DEV), st, got, heads, dim, vdim, chunks)
        scale = float(want.abs().max())
        assert (got.cpu() - want).abs().max() < 2e-5 * scale, "outputs" + (" (chunked)" if chunks else "")
        assert (st.cpu() - st_want).abs().max() < 2e-5 * float(st_want.abs().max()), "state"
        untouched = [s for s in range(len(lens) + 2) if s not in slots.tolist()]
        assert torch.equal(st.cpu()[untouched], state0[untouched]), "a state of no sequence of the step was written"
    o, w = rnd(n, heads * vdim, seed=3, scale=4.0), rnd(vdim, seed=4) + 1
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        for weight in (w, None):
            y_want, y = torch.empty(n, heads * vdim, dtype=dtype), torch.empty(n, heads * vdim, dtype=dtype, device=DEV)
            plain_ops.head_rmsnorm(o, weight, 1e-5, y_want, heads, 0.7)
            ops.head_rmsnorm(o.to(DEV), None if weight is None else weight.to(DEV), 1e-5, y, heads, 0.7)
            assert (y.cpu().float() - y_want.float()).abs().max() < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, gains, rot, v_from_k, vrot", [
    (6, 3, 24, 40, True, 16, False, True), (9, 1, 10, 10, False, 0, True, False), (2, 1, 12, 6, True, 2, False, True),
    (4, 4, 16, 16, True, 16, False, False), (2, 2, 64, 32, False, 64, False, True), (3, 1, 130, 130, False, 0, True, False),
    (6, 2, 128, 64, True, 32, False, True)])
def test_normed_rotated_queries_keys_values_and_the_turn_back(dtype, H, G, D, V, gains, rot, v_from_k, vrot):
    """Sequences that bring 1, 2, 70 and 5 tokens onto 0, 3, 60 and 127 held ones, into shuffled pages."""
    from minfer_amd.cache.paged import v_page_shape
    from minfer_amd.kernels import ops
    held, new = (0, 3, 60, 127), (1, 2, 70, 5)
    C = H * D + G * D + (0 if v_from_k else G * V)
    n = sum(new)
    qkv = rnd(n, C, seed=1, scale=2.0)
    seq = torch.repeat_interleave(torch.arange(4, dtype=torch.int32), torch.tensor(new)).to(torch.int32)
    pos = torch.cat([torch.arange(h, h + m) for h, m in zip(held, new)]).to(torch.int32)
    table = pages([h + m for h, m in zip(held, new)], 7)
    qg = kg = None
    if gains:
        qg, kg = rnd(D, seed=8) + 1.0, rnd(D, seed=9) + 1.0
    ang = torch.arange(256, dtype=torch.float64)[:, None]
    rt = None if not rot else tuple(f(ang * (100.0 ** (-2.0 * torch.arange(rot // 2) / rot))).float() for f in (torch.cos, torch.sin))
    vt = None if not vrot else tuple(f(ang * (100.0 ** (-2.0 * torch.arange(V // 2) / V))).float() for f in (torch.cos, torch.sin))
    outs = []
    for side in ("plain", "gpu"):
        dev = "cpu" if side == "plain" else DEV
        mv = lambda t: None if t is None else (tuple(x.to(dev) for x in t) if isinstance(t, tuple) else t.to(dev))
        kc = torch.zeros(40, G, 64, D, dtype=dtype, device=dev)
        vc = torch.zeros((40,) + v_page_shape(G, V, dtype), dtype=dtype, device=dev)
        q = torch.empty(n, H * D, dtype=dtype, device=dev)
        fn = plain_ops.qk_norm_prep if side == "plain" else ops.qk_norm_prep
        fn(mv(qkv), mv(qg), mv(kg), 1e-5, True, mv(seq), mv(pos), mv(rt), mv(vt), v_from_k, mv(table), q, kc, vc, H, G, D, V, True)
        o = (rnd(n, H * V, seed=11) * 3).to(dtype).to(dev)
        (plain_ops.unrotate if side == "plain" else ops.unrotate)(o, mv(vt), mv(pos), H, 1.3)
        outs.append([t.cpu().float() for t in (q, kc, vc, o)])
    tol = 3e-5 if dtype == torch.float32 else 1e-2          # bfloat16: a rounding apart, relative to the value
    for name, a, b in zip(("q", "k pages", "v pages", "rotated back"), *outs):
        assert ((a - b).abs() / b.abs().clamp(min=1.0)).max() < tol, name
    if vt is not None and dtype == torch.float32:        # turning back undoes the turn
        x = (rnd(n, H * V, seed=12)).to(DEV)
        y = x.clone()
        ops.unrotate(y, tuple(t.to(DEV) for t in vt), pos.to(DEV), H, 1.0)
        ops.unrotate(y, (vt[0].to(DEV), -vt[1].to(DEV)), pos.to(DEV), H, 1.0)
        assert (x - y).abs().max() < 1e-5


def _far(H, seed):
    rng = np.random.default_rng(seed)
    return (torch.tensor(rng.uniform(0.1, 1.5, H), dtype=torch.float32), torch.tensor(rng.uniform(0.05, 2.0, H), dtype=torch.float32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, chunk, far", [(6, 3, 24, 40, 17, False), (9, 1, 8, 24, 0, True), (2, 1, 12, 5, 1, False),
                                                    (4, 4, 16, 16, 64, True), (16, 2, 128, 64, 70, False), (6, 2, 48, 48, 0, True),
                                                    (3, 3, 10, 10, 100, False)])
def test_chunks_and_distance_in_the_plain_attention_kernel(dtype, H, G, D, V, chunk, far):
    """Prompts, portions on held tokens and single tokens in one launch, over shuffled pages."""
    from minfer_amd.kernels import ops
    lens, new = (1, 130, 64, 300, 65), (1, 130, 3, 1, 40)
    q, kc, vc, table, pos, seq, _ = attention_case(dtype, H, G, D, V, lens, new, 0, 0.0, 3)
    ones = torch.ones(H)
    fr = _far(H, 5) if far else None
    want = torch.empty(sum(new), H * V, dtype=dtype)
    plain_ops.capped_attn(q, kc, vc, table, pos, seq, ones, want, H, G, D, V, 0.2, 0.0, 0, max(lens), chunk=chunk, far=fr)
    got = torch.empty(sum(new), H * V, dtype=dtype, device=DEV)
    ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), ones.to(DEV), got, H, G, D, V,
                    0.2, 0.0, 0, max(lens), chunk=chunk, far=None if fr is None else tuple(t.to(DEV) for t in fr))
    err = (got.cpu().float() - want.float()).abs().max()
    assert torch.isfinite(got).all() and err < (2e-5 if dtype == torch.float32 else 4e-2), float(err)


@pytest.mark.parametrize("H, G, D, V, chunk, far", [(6, 3, 32, 48, 17, False), (8, 2, 96, 48, 0, True), (4, 4, 16, 16, 64, True),
                                                    (16, 2, 128, 64, 70, False), (7, 7, 48, 16, 1, False), (6, 2, 48, 48, 0, True),
                                                    (6, 2, 128, 128, 65, False), (2, 1, 64, 128, 100, True)])
@pytest.mark.parametrize("new", [(1, 130, 3, 1, 40), (1, 64, 64, 300, 65), (1, 1, 1, 2, 17), (1, 1, 1, 1, 1)])
def test_chunks_and_distance_in_the_matrix_core_attention_kernel(H, G, D, V, chunk, far, new):
    """Blocks of 16 tokens that lie across a chunk's edge, and a decode step whose keys split over waves."""
    from minfer_amd.kernels import ops
    lens = (1, 130, 64, 300, 65)
    q, kc, vc, table, pos, seq, _ = attention_case(torch.bfloat16, H, G, D, V, lens, new, 0, 0.0, 4)
    ones = torch.ones(H)
    fr = _far(H, 6) if far else None
    want = torch.empty(sum(new), H * V, dtype=torch.bfloat16)
    plain_ops.capped_attn(q, kc, vc, table, pos, seq, ones, want, H, G, D, V, 0.2, 0.0, 0, max(lens), chunk=chunk, far=fr)
    got = torch.empty(sum(new), H * V, dtype=torch.bfloat16, device=DEV)
    ops.capped_attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), step_context(lens, new, table, pos, seq),
                            ones.to(DEV), got, H, G, D, V, 0.2, 0.0, 0, chunk=chunk,
                            far=None if fr is None else tuple(t.to(DEV) for t in fr))
    err = (got.cpu().float() - want.float()).abs().max()
    assert torch.isfinite(got).all() and err < 4e-2, float(err)


# the last query stands at position 299: (chunk, the key's position, seen or not)
EDGES = [(17, 289, True), (17, 288, False), (64, 256, True), (64, 255, False), (65, 260, True), (65, 259, False),
         (70, 280, True), (70, 279, False), (100, 200, True), (100, 199, False), (300, 0, True), (1, 299, True), (1, 298, False),
         (0, 0, True)]


@pytest.mark.parametrize("form", ["plain float32", "plain bfloat16", "matrix cores"])
@pytest.mark.parametrize("chunk, key, inside", EDGES)
def test_a_key_at_the_chunk_edge_decides_or_is_not_seen(form, chunk, key, inside):
    """A key made to win the softmax with a value row of 50s: it decides the result where the query's chunk
    holds it (also 299 positions back, across page edges, and under the penalty on distance), and leaves no
    trace one position earlier; at the end of a prompt, of a portion, and for a single token."""
    from minfer_amd.kernels import ops
    H, G, D, V = 4, 2, 16, 16
    dtype = torch.float32 if form == "plain float32" else torch.bfloat16
    for lens, new in (((300, 90), (300, 20)), ((300, 90), (45, 1)), ((300, 90), (1, 1))):
        for fr in (None, _far(H, 2)):
            q, kc, vc, table, pos, seq, _ = attention_case(dtype, H, G, D, V, lens, new, 0, 0.0, 5, needle=(0, key, 1))
            got = torch.empty(sum(new), H * V, dtype=dtype, device=DEV)
            ones = torch.ones(H, device=DEV)
            far = None if fr is None else tuple(t.to(DEV) for t in fr)
            if form == "matrix cores":
                ops.capped_attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), step_context(lens, new, table, pos, seq),
                                        ones, got, H, G, D, V, 1.0, 0.0, 0, chunk=chunk, far=far)
            else:
                ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), ones, got, H, G, D, V,
                                1.0, 0.0, 0, 300, chunk=chunk, far=far)
            row = got[new[0] - 1].float().cpu().view(H, V)
            if inside:
                assert (row[2:] - 50.0).abs().max() < 0.5, (lens, new, fr is not None)
            else:
                assert row[2:].abs().max() < 10.0, (lens, new, fr is not None)


def test_the_penalty_on_distance_by_hand():
    """Two equal keys with different values, one 1 and one 200 positions back, and the query's own key far
    below them: the farther one weighs ((1 + b) / (1 + 200 b))^a of the nearer."""
    from minfer_amd.kernels import ops
    H, G, D, V = 2, 1, 16, 16
    lens, new = (201,), (1,)
    table = pages(lens, 1)
    kc = torch.zeros(40, G, 64, D)
    vc = torch.zeros(40, G, 64, V)
    key = torch.zeros(D)
    key[3] = 2.0
    for p, val in ((0, 1.0), (199, 3.0)):
        kc[int(table[0, p // 64]), 0, p % 64] = key
        vc[int(table[0, p // 64]), 0, p % 64] = val
    for p in list(range(1, 199)) + [200]:
        kc[int(table[0, p // 64]), 0, p % 64] = -20.0 * key
    q = torch.cat([key, key]).view(1, H * D)
    a, b = torch.tensor([1.0, 0.5]), torch.tensor([0.25, 2.0])
    pos, seq = torch.tensor([200], dtype=torch.int32), torch.tensor([0], dtype=torch.int32)
    got = torch.empty(1, H * V, device=DEV)
    ops.capped_attn(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq.to(DEV), torch.ones(H, device=DEV), got,
                    H, G, D, V, 1.0, 0.0, 0, 201, far=(a.to(DEV), b.to(DEV)))
    for h in range(H):
        ratio = ((1.0 + float(b[h])) / (1.0 + 200.0 * float(b[h]))) ** float(a[h])
        want = (ratio * 1.0 + 3.0) / (ratio + 1.0)
        assert abs(float(got[0, h * V]) - want) < 1e-4, h


def test_biased_router_silu_experts_and_rows_added():
    from minfer_amd.kernels import ops
    for E, top, n in ((6, 2, 40), (8, 8, 5), (4, 1, 3), (12, 3, 33), (1, 1, 2)):
        want = [torch.empty(n, E), torch.empty(n, top, dtype=torch.int32), torch.empty(n, top)]
        got = [t.clone().to(DEV) for t in want]
        bias = rnd(E, seed=E + 2, scale=2.0)
        for xt in (torch.float32, torch.bfloat16):
            xr, wr = rnd(n, 70, seed=E).to(xt), rnd(E, 70, seed=E + 1, scale=0.3)
            plain_ops.moe_route(xr, wr, want[0], want[1], want[2], 1, 1, bias=bias)
            ops.moe_route(xr.to(DEV), wr.to(DEV), got[0], got[1], got[2], 1, 1, bias=bias.to(DEV))
            assert torch.equal(got[1].cpu(), want[1]) and (got[2].cpu() - want[2]).abs().max() < 1e-5
            # the weights are the softmax over the chosen logits (with their biases) alone
            z = xr.double() @ wr.double().T + bias.double()
            assert (torch.softmax(torch.gather(z, 1, want[1].long()), dim=1).float() - got[2].cpu()).abs().max() < 1e-5
        F, K, N = 24, 72, 40
        gu = rnd(n, E * 2 * F, seed=2, scale=2.0)
        silu = ops.MOE_ACTS["silu"]
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
            y_want, y = torch.empty(n, E * F, dtype=dtype), torch.empty(n, E * F, dtype=dtype, device=DEV)
            plain_ops.moe_act(gu, want[0], y_want, 0.0, silu)
            ops.moe_act(gu.to(DEV), got[0], y, 0.0, silu)
            assert (y.cpu().float() - y_want.float()).abs().max() < tol
            x, w1, w2 = rnd(n, K, seed=3).to(dtype), (rnd(E, 2 * F, K, seed=4) / 8).to(dtype), (rnd(E, N, F, seed=5) / 5).to(dtype)
            o_want, o = rnd(n, N, seed=6), rnd(n, N, seed=6).to(DEV)
            few = min(n, 16)
            plain_ops.moe_sparse(x[:few], w1, w2, want[1][:few], want[2][:few], o_want[:few], E, 0.0, silu)
            ops.moe_sparse(x[:few].contiguous().to(DEV), w1.to(DEV), w2.to(DEV), got[1][:few].contiguous(),
                           got[2][:few].contiguous(), o[:few], E, 0.0, silu)
            assert (o.cpu()[:few] - o_want[:few]).abs().max() < (1e-4 if dtype == torch.float32 else 5e-2)
    h, x = rnd(7, 100, seed=1), rnd(7, 100, seed=2)
    got = h.clone().to(DEV)
    ops.add_rows(got, x.to(DEV))
    assert torch.equal(got.cpu(), h + x)


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("nodutar")
    return {name: write_nodutar(str(tmp / name), raw, seed=i) for i, (name, raw) in enumerate(ND.items())}


@pytest.fixture(scope="module")
def plains(folders):
    return {name: pn.PlainNodutar.from_folder(f) for name, f in folders.items()}


def engine_for(folder, dtype, max_tokens=64 * 16, **kw):
    from minfer_amd import Engine, load_model
    return Engine(load_model(folder, dtype=dtype, device="cuda:0"), max_tokens=max_tokens, poison_cache=True, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ND))
def test_replays_agree_with_plain(folders, plains, name, dtype):
    """Whole; the last tokens one by one (the chunks' edges pass under decoded tokens); unequal batches one
    after another (slots, pages and states used again); prompts in portions down to two tokens and one, alone
    and in mixed batches."""
    reqs = requests_for(ND[name]["vocab"], (1, 7, 64, 150, 65, 33, 290), seed=3)
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
    """Twenty sequences that start and decode together: the routed layers' few-token form runs in slices, and
    the recurrence carries twenty states side by side."""
    reqs = requests_for(ND["A"]["vocab"], tuple(3 + (7 * i) % 11 for i in range(20)), seed=12)
    eng = engine_for(folders["A"], dtype, max_tokens=64 * 24)
    check(eng, batch_steps(reqs, [list(reqs)], prompt_frac=0.4), plains["A"], reqs, dtype, "twenty together")
    assert not eng.cache.live_slots()


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whatever config.json may say: sizes, orders and options drawn at random, both run types, whole, one by
    one, in batches and in portions."""
    raw = random_config(np.random.default_rng(7000 + seed))
    folder = write_nodutar(str(tmp_path / "m"), raw, seed=seed)
    plain = pn.PlainNodutar.from_folder(folder)
    reqs = requests_for(raw["vocab"], (1, 9, 70, 200, 131), seed=seed)
    ids = list(reqs)
    for dtype in ("float32", "bfloat16"):
        eng = engine_for(folder, dtype)
        what = f"random configuration {seed} ({json.dumps(raw)[:400]})"
        check(eng, whole_steps(reqs), plain, reqs, dtype, what + " whole", SHARP)
        check(eng, tail_steps(reqs, tail=33), plain, reqs, dtype, what + " one by one", SHARP)
        check(eng, batch_steps(reqs, [ids[:3], ids[3:]]), plain, reqs, dtype, what + " batches", SHARP)
        check(eng, chunk_steps(reqs, [ids[:2], ids[2:]]), plain, reqs, dtype, what + " portions", SHARP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_chunks_and_long_decoding(tmp_path, dtype):
    """Query gains and scales raised so that the softmax picks single keys (a key that a chunk wrongly holds
    or drops, or a distance counted one off, then moves a row by its whole size): a prompt of 400 tokens whole,
    then as 250 + 150 one by one, with chunks of 17, 64 and 70 whose edges pass under decoded tokens and page
    edges, and the penalised attention over all 400."""
    raw = dict(vocab=300, width=96, architecture="Nodutar", norm=dict(eps=1e-5), loop=dict(start=0, stop=2, times=2), layers=[
        dict(parallel(left(4, 2, 32, 16, 0.6, 17, 16, base=1000.0), right(3, 20, 12), 0.7, 1.3), mlp=moe(6, 2, 40)),
        dict(attention(6, 3, 16, 2.5), mlp=None),
        dict(parallel(left(2, 2, 16, 48, 1.0, 70, 16, base=50.0), right(1, 40, 72), 1.1, 0.4), mlp=moe(4, 1, 56)),
        dict(parallel(left(2, 1, 32, 32, 0.5, 64, 8, base=200.0), right(2, 8, 8), 1.0, 1.0), mlp=None),
    ])
    folder = write_nodutar(str(tmp_path / "sharp"), raw, seed=21, sharpen=4.0 if dtype == "float32" else 2.0)
    plain = pn.PlainNodutar.from_folder(folder)
    reqs = {"long": random_tokens(300, 400, 77)}
    eng = engine_for(folder, dtype, max_tokens=64 * 16)
    check(eng, whole_steps(reqs), plain, reqs, dtype, "sharp whole", SHARP, 1e-3)
    check(eng, tail_steps(reqs, tail=150), plain, reqs, dtype, "sharp 250 + 150 one by one", SHARP, 1e-3)


def test_greedy_generation_through_the_entry_point(folders, plains):
    """`LLM.generate`: the scheduler, slots used again (more prompts than slots), the captured decode step;
    70 new tokens so that every sequence crosses a page edge and the chunks' edges while decoding."""
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
            assert t == pn.greedy(row) or top[1] - top[0] < 1e-4, f"token {i}"
    bf = LLM(folders["A"], dtype="bfloat16", n_ctx=256, n_slots=4)
    a = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[]).tokens
    b = bf.generate(prompts, max_new=20, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False).tokens
    assert a == b


def test_programs(folders, plains, tmp_path):
    """bin/minfer generates greedily from a Nodutar folder; bin/trace_run replays a batch."""
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "minfer"), folders["B"], "--prompt-tokens", "5,6,7;9",
                        "--greedy", "--repeat-penalty", "1.0", "-n", "4", "--dtype", "float32", "--n-ctx", "64",
                        "--stop-token", "100000"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.strip().splitlines() if l]
    for line, prompt in zip(lines, ([5, 6, 7], [9])):
        seq = list(prompt)
        for t in (int(x) for x in line.split(",")):
            assert t == pn.greedy(plains["B"].forward(seq)[-1])
            seq.append(t)
    vocab = ND_B["vocab"]
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
