"""Katarax without a GPU: the configuration, the plain implementation's own mechanisms against hand-made cases,
and the real engine, cache and generation loop driven through the plain stand-ins for the kernels against the
plain implementation."""
import copy
import json
import math
import os

import numpy as np
import pytest
import torch

import plain_katarax as pk
import plain_ops
from katarax_tiny import KT, KT_A, KT_B, KT_C, random_config, write_katarax, written_config
from replays import batch_steps, chunk_steps, requests_for, run_steps, tail_steps, whole_steps


# ------------------------------------------------------------------ configuration
def test_configuration_reads_writes_and_describes():
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    cfg = config_from_dict(KT_A)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.model_spec()
    assert [b.kind for b in spec.blocks] == ["parallel_shared_norm"] * 6
    # layer 4 reads layer 2's keys and values: it runs on that cache entry and writes nothing
    assert [(e.block, e.cache, e.writes_cache) for e in spec.schedule] == \
        [(0, 0, True), (1, 1, True), (2, 2, True), (3, 3, True), (4, 2, False), (5, 5, True)]
    names = expected_tensors(spec)
    assert names["l0.mix.dq"].shape == (24, 96) and names["l0.mix.uq"].shape == (3 * 24, 24)
    assert names["l0.mix.dkv"].shape == (48, 96) and names["l0.mix.dkv.norm"].shape == (40,)
    assert names["l0.mix.uv"].shape == (72, 40) and names["l0.mix.g"].shape == (72, 96) and names["l0.mix.o"].shape == (96, 72)
    assert names["l1.mix.rel"].shape == (12, 4) and names["l1.mix.v"].shape == (32, 96) and names["l1.mix.o"].shape == (96, 64)
    assert "l4.mix.k" not in names and "l4.mix.v" not in names and names["l4.mix.q"].shape == (128, 96)
    assert "l2.mlp.router" not in names and names["l0.mlp.correction"].shape == (6,) and names["l3.mlp.e2.down"].shape == (96, 24)
    assert names["head"].shape == (300, 96) and names["l5.norm1"].shape == (96,) and "l5.norm2" not in names
    assert spec.head.kind == "capped_linear_head" and config_from_dict(KT_B).model_spec().head.kind == "linear_head"


def test_the_rows_of_a_bias_table_come_from_the_file():
    from minfer_amd import ConfigError, config_from_dict
    cfg = config_from_dict(written_config(KT_A))
    with pytest.raises(ConfigError, match="bias_rows"):
        cfg.model_spec()
    with pytest.raises(ConfigError, match="l1.mix.rel"):
        cfg.adopt_tensor_shapes({"l3.mix.rel": (6, 6)})
    cfg.adopt_tensor_shapes({"l1.mix.rel": (12, 4), "l3.mix.rel": (6, 6)})
    assert cfg.to_dict() == config_from_dict(KT_A).to_dict()


@pytest.mark.parametrize("change, word", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "dims"),
    (lambda c: c["layers"][0]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("bias_max"), "bias_max"),
    (lambda c: c["layers"][1]["mixer"].update(bias_max=5), "bias_max"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=5), "kv_from"),
    (lambda c: c["layers"][4]["mixer"].update(dim=16), "dim"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "router"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c.pop("width"), "width"),
])
def test_configuration_rejections_name_the_key(change, word):
    from minfer_amd import ConfigError, config_from_dict
    raw = copy.deepcopy(KT_A)
    change(raw)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(raw).model_spec()


# ------------------------------------------------------------------ the plain mechanisms by hand
def test_plain_norms_rotations_and_buckets_by_hand():
    x = np.array([[3.0, 4.0, 0.0, 0.0]])
    assert np.allclose(pk.offset_norm(x, np.array([0.5, -0.5, 0.0, 1.0]), 0.0), [[1.5 * 3 / 2.5, 0.5 * 4 / 2.5, 0, 0]])
    assert np.allclose(pk.plain_norm(x, np.array([0.5, -0.5, 0.0, 1.0]), 0.0), [[0.5 * 3 / 2.5, -0.5 * 4 / 2.5, 0, 0]])
    # dims 4, base 100: frequencies 1 and 0.1; position 2; the fifth value passes
    v = np.array([[[1.0, 0.0, 0.0, 2.0, 7.0]]])
    assert np.allclose(pk.rotate_pairs(v, [2], 100.0, 4)[0, 0],
                       [math.cos(2.0), math.sin(2.0), -2 * math.sin(0.2), 2 * math.cos(0.2), 7.0])
    # in halves value 0 turns with value 2 and value 1 with value 3
    assert np.allclose(pk.rotate_halves(v, [2], 100.0, 4)[0, 0],
                       [math.cos(2.0), -2 * math.sin(0.2), math.sin(2.0), 2 * math.cos(0.2), 7.0])
    # 8 rows reaching to 64: below 4 a row a distance, then four rows for the factors 2^(k) of 4
    assert [pk.bucket(n, 8, 64.0) for n in (0, 3, 4, 7, 9, 15, 17, 31, 33, 64, 1000)] == [0, 3, 4, 4, 5, 5, 6, 6, 7, 7, 7]
    from minfer_amd.parts.normed_attention import distance_buckets
    for rows, far in ((8, 64.0), (7, 30.0), (16, 1000.0), (2, 1.5), (4, 3.0)):
        table = distance_buckets(rows, far)
        assert table == [pk.bucket(n, rows, far) for n in range(len(table))] and table[-1] == rows - 1
        assert pk.bucket(len(table) + 50, rows, far) == rows - 1 and (len(table) < 2 or table[-2] < rows - 1)


def test_plain_router_and_expert_by_hand():
    # six experts in three groups; scores 0.5 everywhere except expert 4; corrections decide
    z = np.zeros((1, 6))
    z[0, 4] = math.log(3.0)                                       # sigmoid = 0.75
    corr = np.array([0.3, 0.1, -0.9, 0.45, 0.0, -0.2])            # choice scores 0.8 0.6 | -0.4 0.95 | 0.75 0.3
    r = dict(experts=6, top=2, scale=2.0, groups=dict(count=3, keep=2))
    chosen, w, margins = pk.route(z, corr, r)
    # group sums 1.4, 0.55, 1.05: groups 0 and 2 are kept, so expert 3, the best of all, cannot be chosen
    assert list(chosen[0]) == [0, 4] and np.allclose(w[0], [2.0 * 0.5 / 1.25, 2.0 * 0.75 / 1.25])
    assert np.isclose(margins[0], 0.75 - 0.6)                     # the last one chosen over the first one left out
    # one group kept of three: the experts of the others count as minus infinity, not as zero
    corr = np.array([-2.0, -3.0, -1.0, -2.0, -1.0, -1.5])         # every choice score is negative; group sums -4, -2, -1.25
    chosen, w, _ = pk.route(z, corr, dict(r, top=2, groups=dict(count=3, keep=1)))
    assert sorted(chosen[0]) == [4, 5] and np.allclose(sorted(w[0]), [2.0 * 0.5 / 1.25, 2.0 * 0.75 / 1.25])
    h = np.array([[1.0, 2.0]])
    g, u, d = np.array([[2.0, 0.0], [0.0, -1.0]]), np.array([[1.0, 1.0], [0.5, 0.0]]), np.eye(2)
    # gate sums 2 and -2, up sums 3 (clamped to 1.5) and 0.5; the gate is clamped from above only
    want = [1.5 / (1 + math.exp(-1.702 * 1.5)) * 2.5, -2 / (1 + math.exp(1.702 * 2)) * 1.5]
    assert np.allclose(pk.expert(h, g, u, d, 1.5), [want])


def test_plain_attentions_by_hand():
    eye = np.eye(2)
    # a window of two with one kept position: position 3 sees 0 (kept), 2 and 3, not 1
    w = {"q": eye * 0.0, "k": eye, "v": eye, "o": eye, "rel": np.zeros((4, 1))}
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, bias_max=4, mask=dict(size=2, keep_first=1))
    h = np.array([[1.0, 0.0], [0.0, 100.0], [0.0, 1.0], [1.0, 1.0]])
    out = pk.biased_window_attention(h, w, "", m)
    assert np.allclose(out[3], (h[0] + h[2] + h[3]) / 3) and np.allclose(out[1], (h[0] + h[1]) / 2)
    # the bias alone decides: rows 0, 1, 2 for distances 0, 1, 2; row 3 from distance 3 on (4 rows reaching to 4:
    # 2 + floor(2 ln(3 / 2) / ln 2) = 3)
    w["rel"] = np.log(np.array([[1.0], [2.0], [3.0], [5.0]]))
    m["mask"] = dict(size=100, keep_first=0)
    h = np.vstack([h, [[2.0, 2.0]]])
    out = pk.biased_window_attention(h, w, "", m)
    assert np.allclose(out[4], (5 * h[0] + 5 * h[1] + 3 * h[2] + 2 * h[3] + 1 * h[4]) / 16)
    # a reader takes the owner's keys and values and its own queries
    wq = {"q": eye, "k": eye, "v": eye * 2, "o": eye}
    mu = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, rot=dict(base=10.0, dims=2))
    hh = np.array([[1.0, 0.0], [0.0, 1.0]])
    kv = pk.unit_keys_values(hh, wq, "", mu, 0.0)
    assert np.allclose(np.linalg.norm(kv[0], axis=-1), math.sqrt(2.0))          # unit root mean square over two values
    own = pk.unit_attention(hh, wq, "", mu, 0.0, kv)
    other = pk.unit_attention(hh, dict(wq, q=-eye), "", mu, 0.0, kv)
    assert np.allclose(own[0], other[0]) and not np.allclose(own[1], other[1])   # one key: the query does not matter


def test_plain_latent_attention_against_the_absorbed_form():
    """The explicit per-head keys and values against queries taken to the latent's side, for one token."""
    rng = np.random.default_rng(0)
    m = dict(heads=2, dim=3, rot_dim=2, vdim=4, kv_rank=5, q_rank=3, scale=0.7, rot=dict(base=10.0, dims=2), mask=dict(size=3))
    w = {k: rng.standard_normal(s) for k, s in dict(dq=(3, 6), uq=(10, 3), dkv=(7, 6), uk=(6, 5), uv=(8, 5), g=(8, 6), o=(6, 8)).items()}
    w["dq.norm"], w["dkv.norm"] = rng.uniform(0.5, 1.5, 3), rng.uniform(0.5, 1.5, 5)
    h = rng.standard_normal((5, 6))
    out = pk.latent_attention(h, w, "", m, 1e-5)
    t = 4                                                      # sees positions 2, 3, 4
    pos = np.arange(5)
    dkv = h @ w["dkv"].T
    c = pk.plain_norm(dkv[:, :5], w["dkv.norm"], 1e-5)
    kr = pk.rotate_pairs(dkv[:, None, 5:], pos, 10.0, 2)[:, 0]
    q = (pk.plain_norm(h @ w["dq"].T, w["dq.norm"], 1e-5) @ w["uq"].T).reshape(5, 2, 5)
    qr = pk.rotate_pairs(q[:, :, 3:], pos, 10.0, 2)
    heads = []
    for hd in range(2):
        q_lat = w["uk"][hd * 3:(hd + 1) * 3].T @ q[t, hd, :3]
        s = np.array([(q_lat @ c[j] + qr[t, hd] @ kr[j]) * 0.7 for j in (2, 3, 4)])
        p = np.exp(s - s.max())
        p /= p.sum()
        heads.append(w["uv"][hd * 4:(hd + 1) * 4] @ (p @ c[2:5]))
    want = (np.concatenate(heads) * pk.sigmoid(h[t] @ w["g"].T)) @ w["o"].T
    assert np.allclose(out[t], want)


# ------------------------------------------------------------------ the engine on the stand-ins
def _rel(rows, ref):
    worst = 0.0
    for (rid, p), got in rows.items():
        want = ref[rid][p]
        worst = max(worst, float(np.abs(got - want).max() / max(1e-9, want.std())))
    return worst


@pytest.mark.parametrize("name", list(KT))
def test_engine_on_stand_ins_agrees_with_plain(tmp_path, monkeypatch, name):
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, load_model
    folder = write_katarax(str(tmp_path / name), KT[name], seed=5)
    assert "bias_rows" not in open(os.path.join(folder, "config.json")).read()
    plain = pk.PlainKatarax.from_folder(folder)
    reqs = requests_for(KT[name]["vocab"], (1, 7, 70, 33, 140), seed=2)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 12)
    ids = list(reqs)
    for what, steps in (("whole", whole_steps(reqs)), ("one by one", tail_steps(reqs, tail=9)),
                        ("batches", batch_steps(reqs, [ids[:3], ids[3:]])),
                        ("portions", chunk_steps(reqs, [ids[:2], ids[2:]], sizes=(2, 50, 64, 1, 17)))):
        assert _rel(run_steps(eng, steps), ref) < 1e-4, what
    assert not eng.cache.live_slots()


def test_engine_on_stand_ins_random_configuration(tmp_path, monkeypatch):
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, load_model
    raw = random_config(np.random.default_rng(11))
    folder = write_katarax(str(tmp_path / "r"), raw, seed=6)
    plain = pk.PlainKatarax.from_folder(folder)
    reqs = requests_for(raw["vocab"], (3, 40, 90), seed=4)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 8)
    assert _rel(run_steps(eng, chunk_steps(reqs, [list(reqs)], sizes=(2, 31, 1))), ref) < 1e-4, json.dumps(raw)


@pytest.mark.parametrize("name", ["B", "A"])
def test_greedy_generation_on_stand_ins(tmp_path, monkeypatch, name):
    """`generate` with its scheduler, slots and decode sessions, tokens against the plain model."""
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, generate, load_model
    from minfer_amd.sampling import SamplingParams
    folder = write_katarax(str(tmp_path / "gen"), KT[name], seed=8)
    plain = pk.PlainKatarax.from_folder(folder)
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 6, max_seqs=2)
    prompts = [[5, 9, 20, 7], [11], [25, 3, 3, 3, 8, 1, 44]]
    res = generate(eng, prompts, SamplingParams(temp=0.0, repeat_penalty=1.0), max_new=5, stop_tokens=[])
    for p, toks in zip(prompts, res.tokens):
        seq = list(p)
        for t in toks:
            assert t == pk.greedy(plain.forward(seq)[-1])
            seq.append(t)
    assert not eng.cache.live_slots()


def test_a_windowed_entry_keeps_the_pages_of_its_first_positions():
    """Pages of 64 positions, a window of 100 with 70 kept positions: the first two pages stay, the pages between
    them and the window go back to the pool and are taken again by the next sequence."""
    from minfer_amd.cache.paged import Cache, KVRequest
    cache = Cache({0: KVRequest(1, 8, window=100, keep_first=70), 1: KVRequest(1, 8, window=100), 2: KVRequest(1, 8)},
                  max_tokens=64 * 16, max_seqs=2, dtype=torch.float32, device="cpu")
    kept, plain_window = cache.group_of[0], cache.group_of[1]
    s = cache.alloc_slot()
    for length, gone_kept, gone_plain in ((99, 0, 0), (227, 0, 2), (228, 0, 2), (291, 1, 3), (420, 3, 5), (600, 5, 7)):
        cache.reserve({s: length})
        cache.commit({s: length})
        assert [p < 0 for p in kept.pages[s]].count(True) == gone_kept, length
        assert all(p >= 0 for p in kept.pages[s][:2]) and [p < 0 for p in plain_window.pages[s]].count(True) == gone_plain
        assert all(p >= 0 for p in cache.group_of[2].pages[s])
        cache.check_invariants()
    t = cache.alloc_slot()
    cache.reserve({t: 64 * 5})          # the pages given back serve another sequence
    cache.commit({t: 64 * 5})
    cache.check_invariants()
    cache.free_slot(s)
    cache.free_slot(t)
    assert kept.pool.free_pages == 16 and plain_window.pool.free_pages == 16
