"""A plain, slow implementation of the Nodutar decoder in numpy float64, one function per
mechanism, written from the design's equations and sharing no code with the product path.

The design: x = table[token]; layers x <- x + N1b(mixer(N1(x))), x <- x + N2b(ff(N2(x))) with
N(x) = x / sqrt(mean(x^2) + eps) (1 + w); a run of consecutive layers may be passed several times with
the same weights (every pass with a cache and state of its own), the embedding output being added to
the stream in front of every pass but the first.  A mixer is softmax attention whose values are its
keys as projected, with unit-normed queries and keys and a logarithmic penalty on distance; or two
mixers on one input, scaled and summed: chunked softmax attention with normed, partly rotated queries
and keys and values that are rotated by their own position and rotated back by the query's, beside a
gated linear recurrence whose input gate is one minus its forget gate.  A feed-forward is a mixture
of silu-gated experts; the router's weights are the softmax over the chosen logits.  The head is the
embedding table.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ------------------------------------------------------------------ file reading
def read_safetensors(path: str):
    """name -> float64 array: header length, JSON header, raw data."""
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        head = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, e in head.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = data[lo:hi]
        if e["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif e["dtype"] == "F32":
            a = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif e["dtype"] == "I32":
            a = np.frombuffer(raw, dtype="<i4").copy()
        else:
            raise ValueError(f"{name}: dtype {e['dtype']}")
        out[name] = a.reshape(e["shape"])
    return out


# ------------------------------------------------------------------ small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def unit_rms(x, eps: float):
    """x over its root mean square, eps inside the root."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps: float):
    """The design's norm: the gain is one plus the stored weight."""
    return unit_rms(x, eps) * (1.0 + w)


def softmax(z):
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def rotate_pairs(x, positions, base: float, dims: int, sign: float = 1.0):
    """Values 2i and 2i + 1, i < dims / 2, of the last axis turn by sign * position * base^(-2i/dims);
    the values from `dims` on pass.  x [tokens][...][width], positions [tokens]."""
    out = x.copy()
    i = np.arange(dims // 2)
    freq = base ** (-2.0 * i / dims)
    ang = sign * np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------ feed-forward
def expert(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h, router, bias, top: int):
    """(chosen [tokens][top], weights [tokens][top]): the largest logits, softmax over them alone."""
    z = h @ router.T + bias
    chosen = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(z, chosen, axis=-1)
    return chosen, softmax(picked)


def moe(h, w, prefix: str, n_experts: int, top: int, forced=None, margins=None, own=None):
    """`forced`: the choices to take instead of the router's own (the weights are still the softmax of
    the chosen logits).  `margins`, a list, gets per token the gap between the last logit chosen and the
    first one left out (infinite where all experts are chosen); `own`, a list, the router's own choices."""
    z = h @ w[prefix + "router"].T + w[prefix + "router.b"]
    chosen, weights = route(h, w[prefix + "router"], w[prefix + "router.b"], top)
    if margins is not None:
        ranked = -np.sort(-z, axis=-1)
        margins.append(ranked[:, top - 1] - ranked[:, top] if top < n_experts else np.full(h.shape[0], np.inf))
    if own is not None:
        own.append(chosen)
    if forced is not None:
        chosen = np.asarray(forced)
        weights = softmax(np.take_along_axis(z, chosen, axis=-1))
    out = np.zeros((h.shape[0], w[prefix + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(chosen[t, k])
            out[t] += weights[t, k] * expert(h[t:t + 1], w[f"{prefix}e{e}.gate"], w[f"{prefix}e{e}.up"],
                                             w[f"{prefix}e{e}.down"])[0]
    return out, chosen


# ------------------------------------------------------------------ mixers
def distance_attention(h, w, prefix: str, m, eps: float):
    """Causal attention over one whole sequence from position 0: values are the keys as projected; queries
    and keys over their root mean square per head; score = q . k scale - r1 ln(1 + r2 (i - j))."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[prefix + "q"].T).reshape(T, H, D)
    k = (h @ w[prefix + "k"].T).reshape(T, G, D)
    v = k.copy()
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    pos = np.arange(T)
    dist = (pos[:, None] - pos[None, :]).astype(np.float64)
    seen = dist >= 0
    out = np.zeros((T, H, D))
    for hd in range(H):
        g = hd // (H // G)
        s = q[:, hd] @ k[:, g].T * m["scale"]
        s = s - w[prefix + "r1"][hd] * np.log1p(w[prefix + "r2"][hd] * np.where(seen, dist, 0.0))
        s = np.where(seen, s, -np.inf)
        out[:, hd] = softmax(s) @ v[:, g]
    return out.reshape(T, H * D) @ w[prefix + "o"].T


def chunked_rotary_attention(h, w, prefix: str, m, eps: float):
    """Softmax attention inside chunks of mask.size positions counted from 0, over one whole sequence:
    normed (weighted) queries and keys, rotation in pairs over the first rot.dims values, values rotated
    by their own position over all their pairs and the head's sum rotated back by the query's."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    base, dims, size = m["rot"]["base"], m["rot"]["dims"], m["mask"]["size"]
    pos = np.arange(T)
    q = (h @ w[prefix + "q"].T).reshape(T, H, D)
    k = (h @ w[prefix + "k"].T).reshape(T, G, D)
    v = (h @ w[prefix + "v"].T).reshape(T, G, V)
    q = unit_rms(q, eps) * w[prefix + "q.norm"]
    k = unit_rms(k, eps) * w[prefix + "k.norm"]
    q, k = rotate_pairs(q, pos, base, dims), rotate_pairs(k, pos, base, dims)
    v = rotate_pairs(v, pos, base, V)
    seen = (pos[:, None] >= pos[None, :]) & (pos[:, None] // size == pos[None, :] // size)
    out = np.zeros((T, H, V))
    for hd in range(H):
        g = hd // (H // G)
        s = np.where(seen, q[:, hd] @ k[:, g].T * m["scale"], -np.inf)
        out[:, hd] = softmax(s) @ v[:, g]
    out = rotate_pairs(out, pos, base, V, sign=-1.0)
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def gated_recurrence(h, w, prefix: str, m, eps: float, state=None):
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t per head, from S = 0 (or `state`
    [heads][dim][vdim], which is updated in place); f = l + (1 - l) sigmoid(Wf h + b)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[prefix + "q"].T).reshape(T, H, D)
    v = (h @ w[prefix + "v"].T).reshape(T, H, V)
    low = w[prefix + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ w[prefix + "f"].T + w[prefix + "f.b"])).reshape(T, H, D)
    S = np.zeros((H, D, V)) if state is None else state
    o = np.zeros((T, H, V))
    for t in range(T):
        S *= f[t][:, :, None]
        S += (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps) * w[prefix + "norm"]
    return o.reshape(T, H * V) @ w[prefix + "o"].T


def side_by_side(h, w, prefix: str, m, eps: float):
    left = chunked_rotary_attention(h, w, prefix + "left.", m["left"], eps)
    right = gated_recurrence(h, w, prefix + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ------------------------------------------------------------------ the model
def run_order(cfg):
    """[(layer, first of a repeated pass or not)] as the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] <= 1:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        order += [(i, p > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg, w, tokens, forced=None, keep_layers: bool = False, margins=None, own=None):
    """Logits [tokens][vocab] of one whole sequence from position 0.  `forced`: per run of a layer with a
    feed-forward, the experts to take (None: the router's own).  Returns (logits, streams after every
    layer run, choices taken per routed layer run).  `own` (a list) gets what every router would have
    chosen itself, given what was taken before it."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    first = x.copy()
    streams, choices = [], []
    for i, again in run_order(cfg):
        layer = cfg["layers"][i]
        p = f"l{i}."
        if again:
            x = x + first
        hin = offset_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            y = distance_attention(hin, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            y = side_by_side(hin, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        x = x + offset_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            r = layer["mlp"]["router"]
            f = None if forced is None else forced[len(choices)]
            y, chosen = moe(offset_norm(x, w[p + "norm2"], eps), w, p + "mlp.", r["experts"], r["top"], f, margins, own)
            choices.append(chosen)
            x = x + offset_norm(y, w[p + "norm2b"], eps)
        if keep_layers:
            streams.append(x.copy())
    logits = offset_norm(x, w["final.norm"], eps) @ w["embed"].T
    return logits, streams, choices


def load(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


def greedy(row) -> int:
    return int(np.argmax(row))


class PlainNodutar:
    def __init__(self, cfg, w):
        self.cfg, self.w = cfg, w

    @classmethod
    def from_folder(cls, folder: str):
        return cls(*load(folder))

    def routed_runs(self):
        """The runs of layers (positions of the run order) that have a feed-forward."""
        return [n for n, (i, _) in enumerate(run_order(self.cfg)) if self.cfg["layers"][i].get("mlp") is not None]

    def forward(self, tokens, routes=None, margins=None, choices=None):
        """Logits [tokens][vocab].  `routes`: {run: [tokens][top]} experts to take; `margins` and `choices`
        (lists) get, per routed run, the routers' margins and what they would have chosen themselves given
        the choices taken before them."""
        forced = None if routes is None else [routes[n] for n in self.routed_runs()]
        own = []
        logits, _, _ = forward(self.cfg, self.w, tokens, forced=forced, margins=margins, own=own)
        if choices is not None:
            choices.extend(own)
        return logits
