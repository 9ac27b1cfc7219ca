"""Nodutar without a GPU: the configuration, the plain implementation's own mechanisms against hand-made
cases, and the real engine, cache and generation loop driven through the plain stand-ins for the kernels
against the plain implementation."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_nodutar as pn
import plain_ops
from nodutar_tiny import ND, ND_A, ND_B, ND_C, random_config, write_nodutar
from replays import batch_steps, chunk_steps, requests_for, run_steps, tail_steps, whole_steps


# ------------------------------------------------------------------ configuration
def test_configuration_reads_writes_and_describes():
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    cfg = config_from_dict(ND_A)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.model_spec()
    assert [b.kind for b in spec.blocks] == ["sandwich"] * 4
    # layers 1 and 2 are passed twice, every run with a cache entry of its own; the second pass takes the embedding in
    assert [(e.block, e.cache, e.adds_embedding) for e in spec.schedule] == \
        [(0, 0, False), (1, 1, False), (2, 2, False), (1, 3, True), (2, 4, False), (3, 5, False)]
    names = expected_tensors(spec)
    assert names["l0.mix.left.q"].shape == (4 * 32, 96) and names["l0.mix.left.v"].shape == (2 * 16, 96)
    assert names["l0.mix.left.q.norm"].shape == (32,) and names["l0.mix.left.o"].shape == (96, 4 * 16)
    assert names["l0.mix.right.f.b"].shape == (60,) and names["l0.mix.right.lower"].shape == (60,)
    assert names["l0.mix.right.norm"].shape == (12,) and names["l0.mix.right.o"].shape == (96, 36)
    assert names["l1.mix.k"].shape == (3 * 16, 96) and "l1.mix.v" not in names and names["l1.mix.r2"].shape == (6,)
    assert "l1.norm2" not in names and "l1.mlp.router" not in names and names["l1.norm1b"].shape == (96,)
    assert names["l3.mlp.router.b"].shape == (3,) and names["l3.mlp.e2.down"].shape == (96, 24)
    assert "head" not in names and names["final.norm"].shape == (96,)
    assert [e.adds_embedding for e in config_from_dict(ND_C).model_spec().schedule] == [False, False, True, False, True, False]
    once = copy.deepcopy(ND_C)
    once["loop"]["times"] = 1
    assert [e.block for e in config_from_dict(once).model_spec().schedule] == [0, 1]
    assert pn.run_order(ND_A) == config_from_dict(ND_A).run_order() and pn.run_order(ND_B) == [(0, False), (1, False), (2, False)]


@pytest.mark.parametrize("change, word", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=34), "dims"),
    (lambda c: c["layers"][0]["mixer"]["left"].pop("mask"), "size"),
    (lambda c: c["layers"][0]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "router"),
    (lambda c: c["loop"].update(stop=5), "loop"),
    (lambda c: c.pop("width"), "width"),
])
def test_configuration_rejections_name_the_key(change, word):
    from minfer_amd import ConfigError, config_from_dict
    raw = copy.deepcopy(ND_A)
    change(raw)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(raw)


# ------------------------------------------------------------------ the plain mechanisms by hand
def test_plain_norm_rotation_and_router_by_hand():
    x = np.array([[3.0, 4.0, 0.0, 0.0]])
    assert np.allclose(pn.offset_norm(x, np.array([0.5, -0.5, 0.0, 1.0]), 0.0), [[1.5 * 3 / 2.5, 0.5 * 4 / 2.5, 0, 0]])
    # dims 4, base 100: frequencies 1 and 0.1; position 2; the fifth value passes
    v = np.array([[[1.0, 0.0, 0.0, 2.0, 7.0]]])
    r = pn.rotate_pairs(v, [2], 100.0, 4)
    assert np.allclose(r[0, 0], [math.cos(2.0), math.sin(2.0), -2 * math.sin(0.2), 2 * math.cos(0.2), 7.0])
    assert np.allclose(pn.rotate_pairs(r, [2], 100.0, 4, sign=-1.0), v)
    # the three largest of logits + bias, weighted by the softmax over them alone
    h, router, bias = np.array([[1.0, 2.0]]), np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [-1.0, 0.0]]), np.array([0.0, 0.5, -2.0, 4.0])
    chosen, w = pn.route(h, router, bias, 3)          # logits 1, 2.5, 1, 3
    assert list(chosen[0]) == [3, 1, 0]
    e = np.exp(np.array([3.0, 2.5, 1.0]))
    assert np.allclose(w[0], e / e.sum())
    g, u, d = np.array([[2.0, 0.0], [0.0, -1.0]]), np.array([[1.0, 1.0], [0.5, 0.0]]), np.eye(2)
    assert np.allclose(pn.expert(h, g, u, d), [[2 / (1 + math.exp(-2)) * 3, -2 / (1 + math.exp(2)) * 0.5]])


def test_plain_recurrence_by_hand_and_carried():
    # one head, two key channels, one value; lower bounds 0 and 0.5; the gates' sigmoid is 0.5 with zero projections
    w = {"q": np.array([[1.0], [0.0]]), "f": np.zeros((2, 1)), "f.b": np.zeros(2), "lower": np.array([0.0, 0.5]),
         "v": np.array([[2.0]]), "norm": np.array([1.0]), "o": np.array([[1.0]])}
    m = dict(heads=1, dim=2, vdim=1)
    h = np.array([[1.0], [1.0]])
    st = np.zeros((1, 2, 1))
    pn.gated_recurrence(h[:1], w, "", m, 0.0, state=st)
    assert np.allclose(st[0, :, 0], [0.5 * 2.0, 0.25 * 2.0])              # (1 - f) v with f = 0.5, 0.75
    pn.gated_recurrence(h[1:], w, "", m, 0.0, state=st)
    assert np.allclose(st[0, :, 0], [0.5 * 1.0 + 1.0, 0.75 * 0.5 + 0.5])
    both = np.zeros((1, 2, 1))
    out = pn.gated_recurrence(h, w, "", m, 0.0, state=both)
    assert np.allclose(both, st) and np.allclose(np.abs(out), 1.0)      # a head of one value norms to its sign


def test_plain_attentions_by_hand():
    # one head, keys of two values; the chunked form: a token at position 2 with chunks of 2 sees itself only
    eye = np.eye(2)
    w = {"q": eye, "k": eye, "v": eye, "o": eye, "q.norm": np.ones(2), "k.norm": np.ones(2)}
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, mask=dict(size=2), rot=dict(base=10.0, dims=2))
    h = np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]])
    out = pn.chunked_rotary_attention(h, w, "", m, 0.0)
    assert np.allclose(out[2], h[2]) and np.allclose(out[0], h[0])        # turned by its position and back
    assert not np.allclose(out[1], h[1])                                   # position 1 also sees position 0
    # the distance form: values are the keys as projected; two equal keys, the farther one weighs 1 / (1 + r2)^r1 less
    w = {"q": eye, "k": eye, "o": eye, "r1": np.array([2.0]), "r2": np.array([3.0])}
    m = dict(heads=1, kv_heads=1, dim=2, scale=5.0)
    h = np.array([[2.0, 0.0], [4.0, 0.0]])
    out = pn.distance_attention(h, w, "", m, 0.0)
    p_far = (1.0 / 16.0) / (1.0 + 1.0 / 16.0)
    assert np.allclose(out[1], [p_far * 2.0 + (1 - p_far) * 4.0, 0.0])


# ------------------------------------------------------------------ the engine on the stand-ins
def _rel(rows, ref):
    worst = 0.0
    for (rid, p), got in rows.items():
        want = ref[rid][p]
        worst = max(worst, float(np.abs(got - want).max() / max(1e-9, want.std())))
    return worst


@pytest.mark.parametrize("name", list(ND))
def test_engine_on_stand_ins_agrees_with_plain(tmp_path, monkeypatch, name):
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, load_model
    folder = write_nodutar(str(tmp_path / name), ND[name], seed=5)
    plain = pn.PlainNodutar.from_folder(folder)
    reqs = requests_for(ND[name]["vocab"], (1, 7, 70, 33, 140), seed=2)
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
    folder = write_nodutar(str(tmp_path / "r"), raw, seed=6)
    plain = pn.PlainNodutar.from_folder(folder)
    reqs = requests_for(raw["vocab"], (3, 40, 90), seed=4)
    ref = {rid: plain.forward(toks) for rid, toks in reqs.items()}
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 8)
    assert _rel(run_steps(eng, chunk_steps(reqs, [list(reqs)], sizes=(2, 31, 1))), ref) < 1e-4


@pytest.mark.parametrize("name", ["B", "A"])
def test_greedy_generation_on_stand_ins(tmp_path, monkeypatch, name):
    """`generate` with its scheduler, slots and decode sessions, tokens against the plain model.  In "A" a
    cache group that gives pages back comes before one that does not: the first step of a decode session
    brings the page tables of both."""
    plain_ops.install(monkeypatch)
    from minfer_amd import Engine, generate, load_model
    from minfer_amd.sampling import SamplingParams
    folder = write_nodutar(str(tmp_path / "gen"), ND[name], seed=8)
    plain = pn.PlainNodutar.from_folder(folder)
    eng = Engine(load_model(folder, dtype="float32", device="cpu"), max_tokens=64 * 6, max_seqs=2)
    prompts = [[5, 9, 20, 7], [11], [25, 3, 3, 3, 8, 1, 44]]
    res = generate(eng, prompts, SamplingParams(temp=0.0, repeat_penalty=1.0), max_new=5, stop_tokens=[])
    for p, toks in zip(prompts, res.tokens):
        seq = list(p)
        for t in toks:
            assert t == pn.greedy(plain.forward(seq)[-1])
            seq.append(t)
    assert not eng.cache.live_slots()


def test_a_file_may_hold_the_norms_of_a_feed_forward_that_is_not_there(tmp_path, monkeypatch):
    plain_ops.install(monkeypatch)
    from minfer_amd import load_model
    from minfer_amd.weights.safetensors_io import open_model_files, write_safetensors
    folder = write_nodutar(str(tmp_path / "m"), ND_B, seed=3)
    files = open_model_files(folder)
    have = {n: f.tensor(n).clone() for n, f in files.items()}
    have["l1.norm2"] = torch.zeros(64, dtype=torch.bfloat16)
    have["l1.norm2b"] = torch.zeros(64, dtype=torch.bfloat16)
    del files
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), [(n, tuple(t.shape), t.dtype) for n, t in have.items()],
                      lambda n: have[n])
    with pytest.warns(UserWarning, match="not used"):
        load_model(folder, dtype="float32", device="cpu")


def test_a_chunked_entry_gives_back_the_pages_of_chunks_gone_by():
    """Pages of 64 positions, chunks of 100: once a sequence holds 200 positions, later ones read from 200 on."""
    from minfer_amd.cache.paged import Cache, KVRequest, StateRequest
    cache = Cache({0: (KVRequest(1, 8, chunk=100), StateRequest((2, 3))), 1: KVRequest(1, 8)}, max_tokens=64 * 8, max_seqs=2,
                  dtype=torch.float32, device="cpu")
    chunked = cache.group_of[0]
    s = cache.alloc_slot()
    for length, gone in ((99, 0), (100, 1), (199, 1), (200, 3), (260, 3), (300, 4)):
        cache.reserve({s: length})
        cache.commit({s: length})
        assert [p < 0 for p in chunked.pages[s]].count(True) == gone, length
        assert all(p >= 0 for p in cache.group_of[1].pages[s])
        cache.check_invariants()
    cache.free_slot(s)
    assert chunked.pool.free_pages == 8
