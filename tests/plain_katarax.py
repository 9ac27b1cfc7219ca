"""A plain, slow implementation of the Katarax decoder in numpy float64, one function per mechanism,
written from the design's equations and sharing no code with the product path.

The design: x = table[token]; a layer reads the stream through one norm and adds both branches,
n = N(x), x <- x + mixer(n) + ff(n), with N(x) = x / sqrt(mean(x^2) + eps) (1 + w).  A mixer is one of
  "attention":        grouped-query softmax attention without rotation; a learned bias per (bucket of the
                      distance, head) joins the scaled score; a token sees the last `mask.size` positions and
                      the sequence's first `mask.keep_first`;
  "latent_attention": queries through a normed latent; keys and values from one normed latent a token plus one
                      rotated key part all heads share; rotation in neighbouring pairs; a sliding window; the
                      heads' results times sigmoid(Wg n), value by value;
  "attention_2":      grouped-query causal attention; rotation in halves over the first rot.dims values, then
                      queries and keys over their root mean square per head (no gain); a layer with `kv_from`
                      has no keys and values of its own and reads those of the layer it names.
A feed-forward is a mixture of clamped gated experts; the router scores with a sigmoid, chooses by score plus
a correction per expert among the experts of the best groups (a group counts its two best), and weighs by the
scores themselves over their sum, times a scale.  The logits pass cap tanh(z / cap).
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ------------------------------------------------------------------ file reading
def read_safetensors(path: str):
    """name -> float64 array (int32 stays): header length, JSON header, raw data."""
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


def unit_rms(x, eps: float):
    """x over its root mean square, eps inside the root."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps: float):
    """The layers' norm: the gain is one plus the stored weight."""
    return unit_rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps: float):
    """The latents' norm: the gain is the stored weight."""
    return unit_rms(x, eps) * w


def softmax_rows(s):
    """Softmax over the last axis; -inf entries weigh nothing."""
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def angles(positions, base: float, dims: int):
    i = np.arange(dims // 2)
    return np.asarray(positions, dtype=np.float64)[:, None] * (base ** (-2.0 * i / dims))[None, :]


def rotate_pairs(x, positions, base: float, dims: int):
    """Values 2i and 2i + 1, i < dims / 2, of the last axis turn by position * base^(-2i/dims); the values
    from `dims` on pass.  x [tokens][heads][width]."""
    out = x.copy()
    a = angles(positions, base, dims)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * np.cos(a) - v * np.sin(a)
    out[..., 1:dims:2] = v * np.cos(a) + u * np.sin(a)
    return out


def rotate_halves(x, positions, base: float, dims: int):
    """Value i turns with value i + dims / 2, i < dims / 2, by position * base^(-2i/dims)."""
    out = x.copy()
    half = dims // 2
    a = angles(positions, base, dims)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * np.cos(a) - v * np.sin(a)
    out[..., half:dims] = v * np.cos(a) + u * np.sin(a)
    return out


def bucket(n: int, rows: int, far: float) -> int:
    """The table row of a distance: itself below half the rows, then logarithmic steps up to `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def attend(q, k, v, seen, scale: float, bias=None, kv_of_head=None):
    """q [T][H][D], k [S][G][D], v [S][G][V], seen [T][S] -> [T][H][V]; bias [H][T][S] joins the scaled scores."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for hd in range(H):
        g = hd // (H // G)
        s = q[:, hd] @ k[:, g].T * scale
        if bias is not None:
            s = s + bias[hd]
        out[:, hd] = softmax_rows(np.where(seen, s, -np.inf)) @ v[:, g]
    return out


# ------------------------------------------------------------------ mixers
def biased_window_attention(h, w, prefix: str, m):
    """"attention": no rotation; score = q . k scale + rel[bucket(i - j)][head]; i sees j <= i with
    i - j < mask.size or j < mask.keep_first."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + "q"].T).reshape(T, H, D)
    k = (h @ w[prefix + "k"].T).reshape(T, G, D)
    v = (h @ w[prefix + "v"].T).reshape(T, G, V)
    rel = w[prefix + "rel"]
    pos = np.arange(T)
    dist = pos[:, None] - pos[None, :]
    seen = dist >= 0
    if m.get("mask") is not None:          # no mask: every earlier position
        seen = seen & ((dist < m["mask"]["size"]) | (pos[None, :] < m["mask"].get("keep_first", 0)))
    rows = np.array([[bucket(int(d), rel.shape[0], m["bias_max"]) if d >= 0 else 0 for d in r] for r in dist])
    bias = np.stack([rel[rows, hd] for hd in range(H)])
    return attend(q, k, v, seen, m["scale"], bias).reshape(T, H * V) @ w[prefix + "o"].T


def latent_attention(h, w, prefix: str, m, eps: float):
    """"latent_attention", with every head's keys and values built explicitly."""
    T = h.shape[0]
    H, D, R, V, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T)
    cq = plain_norm(h @ w[prefix + "dq"].T, w[prefix + "dq.norm"], eps)
    q = (cq @ w[prefix + "uq"].T).reshape(T, H, D + R)
    dkv = h @ w[prefix + "dkv"].T
    c = plain_norm(dkv[:, :rank], w[prefix + "dkv.norm"], eps)
    k_rot = rotate_pairs(dkv[:, None, rank:], pos, m["rot"]["base"], m["rot"]["dims"])      # one part for all heads
    q_rot = rotate_pairs(q[:, :, D:], pos, m["rot"]["base"], m["rot"]["dims"])
    k = np.concatenate([(c @ w[prefix + "uk"].T).reshape(T, H, D), np.repeat(k_rot, H, axis=1)], axis=-1)
    q = np.concatenate([q[:, :, :D], q_rot], axis=-1)
    v = (c @ w[prefix + "uv"].T).reshape(T, H, V)
    dist = pos[:, None] - pos[None, :]
    seen = dist >= 0
    if m.get("mask") is not None:
        seen = seen & (dist < m["mask"]["size"])
    o = attend(q, k, v, seen, m["scale"]).reshape(T, H * V)
    return (o * sigmoid(h @ w[prefix + "g"].T)) @ w[prefix + "o"].T


def unit_keys_values(h, w, prefix: str, m, eps: float):
    """The keys (rotated in halves, then over their root mean square) and values of an "attention_2" layer."""
    T = h.shape[0]
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w[prefix + "k"].T).reshape(T, G, D)
    k = unit_rms(rotate_halves(k, np.arange(T), m["rot"]["base"], m["rot"]["dims"]), eps)
    return k, (h @ w[prefix + "v"].T).reshape(T, G, V)


def unit_attention(h, w, prefix: str, m, eps: float, kv):
    """"attention_2" over the keys and values `kv` (its own, or those of the layer it reads)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + "q"].T).reshape(T, H, D)
    q = unit_rms(rotate_halves(q, np.arange(T), m["rot"]["base"], m["rot"]["dims"]), eps)
    pos = np.arange(T)
    seen = pos[:, None] >= pos[None, :]
    return attend(q, kv[0], kv[1], seen, m["scale"]).reshape(T, H * V) @ w[prefix + "o"].T


# ------------------------------------------------------------------ feed-forward
def expert(h, gate, up, down, limit: float):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(z, correction, r):
    """(chosen [tokens][top], weights, margins) from the router's logits z [tokens][experts]."""
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or dict(count=1, keep=1)
    per = E // groups["count"]
    s = sigmoid(z)
    choice = s + correction
    chosen = np.zeros((z.shape[0], top), dtype=np.int64)
    weights = np.zeros((z.shape[0], top))
    margins = np.full(z.shape[0], np.inf)
    for t in range(z.shape[0]):
        by_group = choice[t].reshape(groups["count"], per)
        group_score = np.sort(by_group, axis=-1)[:, -2:].sum(axis=-1)
        ranked_groups = np.argsort(-group_score, kind="stable")
        kept = ranked_groups[:groups["keep"]]
        if groups["keep"] < groups["count"]:
            margins[t] = group_score[ranked_groups[groups["keep"] - 1]] - group_score[ranked_groups[groups["keep"]]]
        masked = np.full(E, -np.inf)
        for g in kept:
            masked[g * per:(g + 1) * per] = choice[t, g * per:(g + 1) * per]
        order = np.argsort(-masked, kind="stable")
        chosen[t] = order[:top]
        if top < E and np.isfinite(masked[order[top]]):
            margins[t] = min(margins[t], masked[order[top - 1]] - masked[order[top]])
        picked = s[t, chosen[t]]
        weights[t] = picked / (picked.sum() + 1e-20) * r["scale"]
    return chosen, weights, margins


def moe(h, w, prefix: str, mlp, forced=None, margins=None, own=None):
    """`forced`: the choices to take instead of the router's own (weighted as the router weighs them)."""
    r = mlp["router"]
    z = h @ w[prefix + "router"].T
    chosen, weights, gaps = route(z, w[prefix + "correction"], r)
    if margins is not None:
        margins.append(gaps)
    if own is not None:
        own.append(chosen)
    if forced is not None:
        chosen = np.asarray(forced)
        picked = np.take_along_axis(sigmoid(z), chosen, axis=-1)
        weights = picked / (picked.sum(axis=-1, keepdims=True) + 1e-20) * r["scale"]
    out = np.zeros((h.shape[0], w[prefix + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for k in range(r["top"]):
            e = int(chosen[t, k])
            out[t] += weights[t, k] * expert(h[t:t + 1], w[f"{prefix}e{e}.gate"], w[f"{prefix}e{e}.up"],
                                             w[f"{prefix}e{e}.down"], mlp["expert"]["limit"])[0]
    return out, chosen


# ------------------------------------------------------------------ the model
def forward(cfg, w, tokens, forced=None, keep_layers: bool = False, margins=None, own=None):
    """Logits [tokens][vocab] of one whole sequence from position 0.  Returns (logits, streams after every
    layer, choices taken per routed layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    streams, choices, kvs = [], [], {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        n = offset_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            y = biased_window_attention(n, w, p + "mix.", m)
        elif layer["type"] == "latent_attention":
            y = latent_attention(n, w, p + "mix.", m, eps)
        elif layer["type"] == "attention_2":
            if m.get("kv_from") is None:
                kvs[i] = unit_keys_values(n, w, p + "mix.", m, eps)
            y = unit_attention(n, w, p + "mix.", m, eps, kvs[i if m.get("kv_from") is None else m["kv_from"]])
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            f = None if forced is None else forced[len(choices)]
            z, chosen = moe(n, w, p + "mlp.", layer["mlp"], f, margins, own)
            choices.append(chosen)
            y = y + z
        x = x + y
        if keep_layers:
            streams.append(x.copy())
    logits = offset_norm(x, w["final.norm"], eps) @ w["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * np.tanh(logits / cap)
    return logits, streams, choices


def load(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


def greedy(row) -> int:
    return int(np.argmax(row))


class PlainKatarax:
    def __init__(self, cfg, w):
        self.cfg, self.w = cfg, w

    @classmethod
    def from_folder(cls, folder: str):
        return cls(*load(folder))

    def routed_runs(self):
        """The layers that have a feed-forward."""
        return [i for i, layer in enumerate(self.cfg["layers"]) if layer.get("mlp") is not None]

    def forward(self, tokens, routes=None, margins=None, choices=None):
        """Logits [tokens][vocab].  `routes`: {layer: [tokens][top]} experts to take; `margins` and `choices`
        (lists) get, per routed layer, the routers' margins and what they would have chosen themselves given
        the choices taken before them."""
        forced = None if routes is None else [routes[n] for n in self.routed_runs()]
        own = []
        logits, _, _ = forward(self.cfg, self.w, tokens, forced=forced, margins=margins, own=own)
        if choices is not None:
            choices.extend(own)
        return logits
