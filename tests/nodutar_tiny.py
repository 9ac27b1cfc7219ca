"""Small Nodutar configurations that differ in every size and option, a writer of model folders with random
weights whose gains, bounds, penalties and biases are not the trivial ones, and configurations drawn at
random."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, scale):
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale))


def parallel(left, right, left_scale=1.0, right_scale=1.0):
    return dict(type="parallel", mixer=dict(left=left, right=right, left_scale=left_scale, right_scale=right_scale))


def left(heads, kv_heads, dim, vdim, scale, chunk, rot_dims, base=10000.0):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, mask=dict(size=chunk),
                rot=dict(base=base, dims=rot_dims))


def right(heads, dim, vdim):
    return dict(heads=heads, dim=dim, vdim=vdim)


def moe(experts, top, ff):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


# sizes the matrix-core attention takes; the middle two layers are passed twice; a chunk of 17 and one of 70;
# a rotation over half a head and one over a whole head; values narrower and wider than keys; a layer without
# feed-forward; all experts chosen in the last layer
ND_A = dict(architecture="Nodutar", vocab=300, width=96, norm=dict(eps=1e-5), loop=dict(start=1, stop=3, times=2), layers=[
    dict(parallel(left(4, 2, 32, 16, 0.2, 17, 16, base=1000.0), right(3, 20, 12), 0.7, 1.3), mlp=moe(6, 2, 40)),
    dict(attention(6, 3, 16, 0.9), mlp=None),
    dict(parallel(left(2, 2, 16, 48, 0.3, 70, 16, base=50.0), right(1, 40, 72), 1.1, 0.4), mlp=moe(4, 1, 56)),
    dict(attention(4, 1, 32, 1.5), mlp=moe(3, 3, 24)),
])

# sizes that are multiples of nothing; no repeated passes; nine query heads on one kv head; a chunk of one (a
# token sees itself only) and one of a page; a rotation over two values; a recurrence wider than 128
ND_B = dict(architecture="Nodutar", vocab=97, width=64, norm=dict(eps=1e-4), layers=[
    dict(attention(9, 1, 10, 0.7), mlp=moe(8, 8, 20)),
    dict(parallel(left(3, 1, 12, 6, 0.4, 1, 2, base=20.0), right(2, 5, 7), 1.0, 1.0), mlp=None),
    dict(parallel(left(4, 4, 6, 10, 0.5, 64, 6, base=500.0), right(2, 136, 16), 0.5, 2.0), mlp=moe(5, 2, 33)),
])

# every layer passed three times; a chunk one longer than a page; one expert of two
ND_C = dict(architecture="Nodutar", vocab=400, width=128, norm=dict(eps=1e-6), loop=dict(start=0, stop=2, times=3), layers=[
    dict(parallel(left(8, 2, 64, 64, 0.125, 65, 32), right(4, 64, 64), 1.2, 0.8), mlp=moe(4, 2, 64)),
    dict(attention(2, 2, 64, 0.25), mlp=moe(2, 1, 100)),
])

ND = {"A": ND_A, "B": ND_B, "C": ND_C}


def _bf16(a) -> torch.Tensor:
    return torch.tensor(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)


def write_nodutar(folder: str, raw: dict, seed: int = 0, sharpen: float = 1.0) -> str:
    """config.json and model.safetensors (bfloat16).  Matrices N(0, 1/inputs); the layers' norm weights around
    zero (they stand for gains around one), the gains of the q, k and head norms around one, lower bounds between
    0.05 and 0.9, the distance penalty's numbers positive, biases N(0, 0.5).  `sharpen` multiplies the gains of
    the chunked attention's query norm (its scores grow with it)."""
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    from minfer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    expected = expected_tensors(config_from_dict(raw).model_spec())
    rng = np.random.default_rng(seed)
    made = {}
    for name, ts in expected.items():
        shape = tuple(ts.shape)
        last = name.split(".", 1)[1] if "." in name else name
        if last in ("norm1", "norm1b", "norm2", "norm2b") or name == "final.norm":
            a = rng.uniform(-0.4, 0.4, shape)
        elif name.endswith("q.norm"):
            a = rng.uniform(0.6, 1.4, shape) * sharpen
        elif name.endswith("k.norm") or name.endswith("right.norm"):
            a = rng.uniform(0.6, 1.4, shape)
        elif name.endswith(".lower"):
            a = rng.uniform(0.05, 0.9, shape)
        elif name.endswith(".r1"):
            a = rng.uniform(0.1, 1.5, shape)
        elif name.endswith(".r2"):
            a = rng.uniform(0.05, 2.0, shape)
        elif name.endswith(".b"):
            a = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[1])
        made[name] = _bf16(a)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(n, tuple(t.shape), torch.bfloat16) for n, t in made.items()], lambda n: made[n])
    return folder


def random_config(rng) -> dict:
    """A configuration drawn at random: one to four layers of either kind in any order, with and without
    feed-forward, odd head sizes and counts, chunks from one to beyond the prompts, partial and whole
    rotations, any run of layers passed one to three times."""
    width = int(rng.choice([48, 64, 100, 128, 136]))
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        mlp = None
        if rng.random() > 0.2:
            experts = int(rng.choice([1, 2, 3, 6, 9]))
            mlp = moe(experts, int(rng.integers(1, experts + 1)), int(rng.choice([16, 40, 64, 72])))
        kv = int(rng.choice([1, 2, 3]))
        heads = kv * int(rng.choice([1, 2, 3, 10]))
        dim = int(rng.choice([6, 8, 16, 24, 32, 64, 96]))
        if rng.random() < 0.4:
            layers.append(dict(attention(heads, kv, dim, float(rng.choice([0.3, 1.0, 2.0]))), mlp=mlp))
            continue
        rot = int(rng.choice([d for d in (2, 4, 6, 8, 16, 32, 64, 96) if d <= dim]))
        vdim = int(rng.choice([6, 8, 16, 24, 64, 10]))
        lt = left(heads, kv, dim, vdim, float(rng.choice([0.05, 0.125, 0.3])), int(rng.choice([1, 2, 31, 64, 65, 100, 1000])),
                  rot, float(rng.choice([100.0, 10000.0, 500000.0])))
        rt = right(int(rng.choice([1, 2, 3, 5])), int(rng.choice([4, 16, 24, 64, 130])), int(rng.choice([8, 16, 40, 64, 100])))
        layers.append(dict(parallel(lt, rt, float(rng.choice([0.5, 1.0, 1.7])), float(rng.choice([0.3, 1.0, 1.4]))), mlp=mlp))
    raw = dict(architecture="Nodutar", vocab=int(rng.choice([64, 300, 1000])), width=width,
               norm=dict(eps=float(rng.choice([1e-6, 1e-5]))), layers=layers)
    if rng.random() < 0.7:
        start = int(rng.integers(0, len(layers)))
        raw["loop"] = dict(start=start, stop=int(rng.integers(start, len(layers) + 1)), times=int(rng.integers(1, 4)))
    return raw
