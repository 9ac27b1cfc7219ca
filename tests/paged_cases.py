"""Shared pieces of the GPU tests of paged attention kernels and routed models: random tensors, shuffled
page tables, attention cases over a poisoned pool with a key made to stand out, step contexts made by hand,
and replays that log the routed layers' choices."""
from __future__ import annotations

import numpy as np
import torch

import plain_ops

DEV = torch.device("cuda:0")


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def run_logged(engine, steps, routed_layers):
    """`replays.run_steps` with the routed layers' choices: ({(request, position): logits row},
    {request: {layer: [position] -> chosen experts}}).  Every step asks for all of its positions."""
    slots, pos, rows, routes = {}, {}, {}, {}
    for st in steps:
        ents = st["entries"]
        for e in ents:
            assert e["want"] == list(range(len(e["tokens"])))
            if e["id"] not in slots:
                slots[e["id"]] = engine.new_sequence()
                pos[e["id"]] = 0
        ctx = engine.build_context([slots[e["id"]] for e in ents], [e["tokens"] for e in ents], [e["want"] for e in ents])
        log = ctx._memo["route_log"] = []
        logits = engine.model.forward(ctx).cpu().numpy()
        engine.cache.commit(ctx.new_lengths)
        assert len(log) == len(routed_layers)
        chosen = [c.cpu().numpy() for c in log]
        r = 0
        for e in ents:
            for w in e["want"]:
                rows[(e["id"], pos[e["id"]] + w)] = logits[r]
                for layer, c in zip(routed_layers, chosen):
                    routes.setdefault(e["id"], {}).setdefault(layer, {})[pos[e["id"]] + w] = c[r]
                r += 1
            pos[e["id"]] += len(e["tokens"])
        assert r == logits.shape[0]
        for rid in st["end"]:
            engine.end_sequence(slots.pop(rid))
        engine.cache.check_invariants()
    return rows, routes


def pages(lens, seed, n_pages=40):
    """Shuffled page tables for sequences of the given lengths."""
    rng = np.random.default_rng(seed)
    order = rng.permutation(n_pages)
    cols = max((l + 63) // 64 for l in lens)
    table = torch.full((len(lens), cols), -1, dtype=torch.int32)
    at = 0
    for b, l in enumerate(lens):
        for c in range((l + 63) // 64):
            table[b, c] = int(order[at])
            at += 1
    return table


def attention_case(dtype, H, G, D, V, lens, new, window, cap, seed, needle=None):
    """Random pages of a NaN-poisoned pool; `needle` = (sequence, key position, kv head): that key is made
    to stand out for the sequence's last query, and its value row is large."""
    from minfer_amd.cache.paged import v_page_shape
    rng = np.random.default_rng(seed)
    table = pages(lens, seed)
    kc = torch.full((40, G, 64, D), float("nan"), dtype=dtype)
    vc = torch.full((40,) + v_page_shape(G, V, dtype), float("nan"), dtype=dtype)
    for b, l in enumerate(lens):
        for p in range(l):
            page = int(table[b, p // 64])
            kc[page, :, p % 64] = rnd(G, D, seed=seed * 1000 + b * 100 + p).to(dtype)
            for g in range(G):
                plain_ops._store_v(vc, page, p % 64, g, rnd(V, seed=seed * 777 + b * 100 + p + g))
    n = sum(new)
    q = rnd(n, H * D, seed=seed + 5).to(dtype)
    pos = torch.cat([torch.arange(l - m, l) for l, m in zip(lens, new)]).to(torch.int32)
    seq = torch.repeat_interleave(torch.arange(len(lens), dtype=torch.int32), torch.tensor(new)).to(torch.int32)
    if needle is not None:
        b, p, g = needle
        page = int(table[b, p // 64])
        row = int(np.cumsum(new)[b]) - 1
        key = kc[page, g, p % 64].float()
        for h in range(g * (H // G), (g + 1) * (H // G)):
            q[row, h * D:(h + 1) * D] = (key * 6.0).to(dtype)          # q . k = 6 |k|^2 for this key
        plain_ops._store_v(vc, page, p % 64, g, torch.full((V,), 50.0))
    temp = torch.tensor(rng.uniform(0.7, 1.4, H), dtype=torch.float32)
    return q, kc, vc, table, pos, seq, temp


def step_context(lens, new, table, pos, seq):
    from minfer_amd.engine.batch import StepContext
    n = sum(new)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return StepContext(cache=None, n_tokens=n, n_seqs=len(lens), token_ids=i32([0] * n), positions=pos.to(DEV),
                       seq_of_tok=seq.to(DEV), cu_seqlens=i32(np.concatenate([[0], np.cumsum(new)]).tolist()),
                       start_pos=i32([l - m for l, m in zip(lens, new)]), slot_ids=i32(list(range(len(lens)))),
                       logit_rows=None, page_tables={}, max_len=max(lens), max_new=max(new), all_decode=all(m == 1 for m in new),
                       host_new=list(new), host_start=[l - m for l, m in zip(lens, new)])


