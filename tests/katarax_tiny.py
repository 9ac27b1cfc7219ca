"""Small Katarax configurations that differ in every size and option, a writer of model folders with random
weights whose gains, bias tables and corrections are not the trivial ones, and configurations drawn at random."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, scale, window, keep_first, rows, far):
    """`rows` (the bias table's) goes into the tensor's shape, not into the written config.json."""
    mask = None if window is None else dict(size=window, keep_first=keep_first)
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, bias_max=far,
                                             bias_rows=rows, mask=mask))


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, window, rot_dims=None, base=10000.0):
    return dict(type="latent_attention", mixer=dict(
        heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale,
        rot=dict(base=base, dims=rot_dim if rot_dims is None else rot_dims), mask=None if window is None else dict(size=window)))


def unit(heads, kv_heads, dim, vdim, scale, rot_dims, base=10000.0, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=dict(base=base, dims=rot_dims))
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="attention_2", mixer=m)


def moe(experts, top, ff, groups=1, keep=None, scale=1.0, limit=2.0):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit),
                router=dict(experts=experts, top=top, scale=scale, groups=dict(count=groups, keep=groups if keep is None else keep)))


# sizes the matrix-core kernels take; a window of 17 and one of 70 with three kept positions; a bias table of 12
# rows reaching to 100; a reader two layers behind its owner, then an owner of other sizes; a layer without
# feed-forward; groups of two experts of which two of three are kept
KT_A = dict(architecture="Katarax", vocab=300, width=96, norm=dict(eps=1e-5), logit_softcap=12.0, layers=[
    dict(latent(3, 16, 8, 24, 40, 24, 0.3, 17, base=1000.0), mlp=moe(6, 3, 40, groups=3, keep=2, scale=1.5)),
    dict(attention(4, 2, 32, 16, 0.2, 70, 3, 12, 100), mlp=moe(4, 1, 56, scale=0.7)),
    dict(unit(4, 2, 32, 32, 0.4, 16), mlp=None),
    dict(attention(6, 3, 16, 48, 0.3, 33, 0, 6, 40), mlp=moe(3, 3, 24)),
    dict(unit(4, 2, 32, 32, 0.6, 16, kv_from=2), mlp=moe(4, 2, 32, groups=2, keep=1, scale=2.0)),
    dict(unit(2, 1, 16, 64, 0.5, 16, base=50.0), mlp=moe(2, 1, 48)),
])

# sizes that are multiples of nothing; nine query heads on one kv head; an odd number of table rows; a window of
# one with five kept positions; a rotation over two values; a reader right behind its owner; groups of one expert;
# no cap on the logits
KT_B = dict(architecture="Katarax", vocab=97, width=64, norm=dict(eps=1e-4), layers=[
    dict(attention(9, 1, 10, 6, 0.7, 1, 5, 7, 30), mlp=moe(8, 2, 20, groups=4, keep=1, scale=1.2, limit=0.8)),
    dict(unit(3, 3, 12, 7, 0.9, 4, base=20.0), mlp=moe(5, 5, 33)),
    dict(unit(3, 3, 12, 7, 0.5, 4, base=20.0, kv_from=1), mlp=None),
    dict(latent(2, 6, 4, 10, 20, 5, 0.4, 64, rot_dims=2, base=500.0), mlp=moe(2, 1, 16, groups=2, keep=2)),
])

# a window one longer than a page with a page of kept positions; a latent attention that sees everything; kept
# positions beyond a page; every expert chosen
KT_C = dict(architecture="Katarax", vocab=400, width=128, norm=dict(eps=1e-6), logit_softcap=50.0, layers=[
    dict(attention(8, 2, 64, 64, 0.125, 65, 64, 32, 128), mlp=moe(4, 2, 64, groups=2, keep=2, scale=2.5)),
    dict(latent(4, 32, 16, 48, 64, 48, 0.15, None), mlp=moe(2, 2, 100)),
    dict(attention(2, 2, 16, 16, 0.25, 40, 70, 4, 3), mlp=None),
    dict(unit(8, 8, 16, 16, 1.0, 8), mlp=moe(9, 4, 24, groups=3, keep=2)),
])

KT = {"A": KT_A, "B": KT_B, "C": KT_C}


def _bf16(a) -> torch.Tensor:
    return torch.tensor(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)


def written_config(raw: dict) -> dict:
    """config.json as a folder holds it: the rows of the bias tables are the tensors' business."""
    out = copy.deepcopy(raw)
    for layer in out["layers"]:
        layer["mixer"].pop("bias_rows", None)
    return out


def write_katarax(folder: str, raw: dict, seed: int = 0, sharpen: float = 1.0) -> str:
    """config.json and model.safetensors (bfloat16).  Matrices N(0, 1/inputs); the layers' norm weights around
    zero (they stand for gains around one), the latents' norm weights around one, bias tables N(0, 1),
    corrections N(0, 0.3) (they change choices and can take a choice score below zero).  `sharpen` multiplies
    the query matrices of the layers whose queries are not normed (their scores grow with it)."""
    from minfer_amd import config_from_dict
    from minfer_amd.engine.model import expected_tensors
    from minfer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(written_config(raw), f)
    expected = expected_tensors(config_from_dict(raw).model_spec())
    rng = np.random.default_rng(seed)
    made = {}
    for name, ts in expected.items():
        shape = tuple(ts.shape)
        if name.endswith(".norm1") or name == "final.norm":
            a = rng.uniform(-0.4, 0.4, shape)
        elif name.endswith(".norm"):
            a = rng.uniform(0.6, 1.4, shape)
        elif name.endswith(".rel"):
            a = rng.standard_normal(shape)
        elif name.endswith(".correction"):
            a = 0.3 * rng.standard_normal(shape)
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[1])
            if name.endswith("mix.uq") or (name.endswith("mix.q") and (name[:-1] + "rel") in expected):
                a = a * sharpen
        made[name] = _bf16(a)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(n, tuple(t.shape), torch.bfloat16) for n, t in made.items()], lambda n: made[n])
    return folder


def random_config(rng) -> dict:
    """A configuration drawn at random: one to five layers of the three kinds in any order, readers behind
    owners, with and without feed-forward, odd head sizes and counts, windows from one to beyond the prompts, kept
    positions from none to beyond a page, any grouping of the experts."""
    width = int(rng.choice([48, 64, 100, 128, 136]))
    layers, owners = [], []
    for i in range(int(rng.integers(1, 6))):
        mlp = None
        if rng.random() > 0.2:
            groups = int(rng.choice([1, 2, 3]))
            per = int(rng.choice([1, 2, 3]))
            keep = int(rng.integers(1, groups + 1))
            mlp = moe(groups * per, int(rng.integers(1, keep * per + 1)), int(rng.choice([16, 40, 64, 72])), groups=groups,
                      keep=keep, scale=float(rng.choice([0.5, 1.0, 2.5])), limit=float(rng.choice([0.5, 2.0, 7.0])))
        kind = int(rng.integers(0, 3))
        kv = int(rng.choice([1, 2, 3]))
        heads = kv * int(rng.choice([1, 2, 3, 10]))
        dim = int(rng.choice([6, 8, 16, 24, 32, 64, 96]))
        vdim = int(rng.choice([6, 8, 16, 24, 64, 10]))
        window = int(rng.choice([1, 2, 31, 64, 65, 100, 1000]))
        if kind == 0:
            rows = int(rng.choice([2, 4, 7, 16, 32]))
            layer = attention(heads, kv, dim, vdim, float(rng.choice([0.1, 0.3, 1.0])), window if rng.random() < 0.8 else None,
                              int(rng.choice([0, 1, 4, 64, 70])), rows, float(rows // 2 + rng.choice([1, 10, 200])))
        elif kind == 1:
            rot_dim = int(rng.choice([2, 4, 8, 16]))
            layer = latent(int(rng.choice([1, 2, 3, 5])), dim, rot_dim, vdim, int(rng.choice([8, 20, 40, 64])),
                           int(rng.choice([5, 16, 24])), float(rng.choice([0.05, 0.125, 0.3])),
                           window if rng.random() < 0.7 else None, rot_dims=int(rng.choice([d for d in (2, 4, 8, 16) if d <= rot_dim])),
                           base=float(rng.choice([100.0, 10000.0, 500000.0])))
        elif owners and rng.random() < 0.5:
            j = int(rng.choice(owners))
            layer = copy.deepcopy(dict(type="attention_2", mixer=layers[j]["mixer"]))
            layer["mixer"].update(kv_from=j, scale=float(rng.choice([0.3, 1.0])))
        else:
            rot = int(rng.choice([d for d in (2, 4, 6, 8, 16, 32, 64, 96) if d <= dim]))
            layer = unit(heads, kv, dim, vdim, float(rng.choice([0.3, 1.0, 2.0])), rot, base=float(rng.choice([100.0, 10000.0])))
            owners.append(i)
        layers.append(dict(layer, mlp=mlp))
    raw = dict(architecture="Katarax", vocab=int(rng.choice([64, 300, 1000])), width=width,
               norm=dict(eps=float(rng.choice([1e-6, 1e-5]))), layers=layers)
    if rng.random() < 0.6:
        raw["logit_softcap"] = float(rng.choice([5.0, 30.0]))
    return raw
