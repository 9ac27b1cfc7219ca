"""Grouped-query softmax attention with queries and keys RMS-normed per head (or not normed at all), and with a
choice of what else a design asks of its attention, each a parameter:

q = Wq x, k = Wk x (no biases); every q and k head over its root mean square (eps inside the root), times a
gain vector shared by the heads where the design has one -> the rotation in neighbouring pairs over the first
values of a head, where it has one -> values: v = Wv x, or the key heads as projected, before their norm
(`values_from_keys`: there is no Wv then) -> with `value_rotation`, a value row goes into the cache rotated by
its own position over all its pairs (an encoding of the values' own, independent of the keys' rotation), and a
head's weighted sum for the query at position i is rotated by -i -> query head h reads kv head h // (heads / kv_heads); mask: all earlier
positions, the last `window` of them, or (`chunk`) those of the token's own chunk of that many positions
counted from 0 -> s = q . k scale, less a penalty on distance a[h] ln(1 + b[h] (i - j)) where the design has
one -> ordinary softmax, o = sum p_j v_j, times `out_scale` -> Wo.

Further parameters: no norm at all (`qk_norm` False); a rotation in halves instead of pairs (a `position` with
`half_tables`; a norm without gains commutes with either rotation, so a design that norms behind the rotation is
served by the same order); with a window, the sequence's first `keep_first` positions, which stay in sight of
every later token; a learned number per (bucket of the distance, head) that joins the scaled score, with the
buckets of `distance_buckets`; and `shared_kv`: the layer has no key and value matrices and reads the keys and
values another layer's run left in its cache entry (the run order gives it that entry, not written by it).

The attention itself runs in the kernels of the capped attention (temperatures of one, no cap).
"""
from __future__ import annotations

import math

import torch

from ..cache.paged import KVRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, POSITIONS, make_part, register_mixer
from .linear import Linear


def distance_buckets(rows: int, far: float):
    """The row of a bias table for every distance 0, 1, ... up to the first that lands in the last row: a distance
    below half the rows has a row of its own; from there on the rows are equal steps of ln(distance), the last row
    beginning where the distance reaches `far`: row(n) = min(rows - 1, half + floor(ln(n / half) / ln(far / half)
    (rows - half))) with half = rows // 2.  Worked out in double on the host; a kernel looks distances up."""
    half = rows // 2
    if rows < 2 or not far > half:
        raise ValueError(f"distance_buckets: {rows} rows reaching to {far}: at least two rows, and the reach beyond half of them")
    out, n = [], 0
    while True:
        row = n if n < half else min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))
        out.append(row)
        if row == rows - 1:
            return out
        n += 1


@register_mixer("normed_attention")
class NormedAttention(Mixer):
    """params: hidden_size, n_heads, n_kv_heads, dim, v_dim, scale, eps (of the q and k norms), qk_gains (True:
    gain vectors under q_norm and k_norm), position (PartSpec of a rotation in pairs with `pair_tables`, or
    None), values_from_keys, value_rotation (PartSpec of a rotation in pairs over v_dim values, or None), window,
    chunk (None or int each), distance (None, or the names of the penalty's two per-head tensors), out_scale,
    qk_norm (default True), keep_first (None or int; needs a window), distance_bias (None, or dict(table: tensor
    name of `[rows][heads]`, rows, far)), shared_kv (default False), q, k, v, o, q_norm, k_norm (tensor names)."""

    takes_normed = True
    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.nh, self.nk, self.dim, self.vdim = (
            int(p[k]) for k in ("hidden_size", "n_heads", "n_kv_heads", "dim", "v_dim"))
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.out_scale = float(p.get("out_scale", 1.0))
        self.gains = bool(p.get("qk_gains", False))
        self.v_from_k = bool(p.get("values_from_keys", False))
        self.window, self.chunk = p.get("window"), p.get("chunk")
        self.distance = p.get("distance")
        self.normed = bool(p.get("qk_norm", True))
        self.keep_first = int(p.get("keep_first") or 0)
        self.bias_spec = p.get("distance_bias")
        self.shared_kv = bool(p.get("shared_kv", False))
        if self.keep_first and (self.window is None or self.chunk is not None):
            raise ValueError("normed_attention: kept first positions go with a window (and no chunks)")
        if self.gains and not self.normed:
            raise ValueError("normed_attention: gains belong to the q and k norms; there are none")
        if self.shared_kv and (self.v_from_k or p.get("value_rotation") is not None):
            raise ValueError("normed_attention: a layer that reads another layer's keys and values makes none of its own")
        self.bias_rows = None
        if self.bias_spec is not None:
            self.bias_rows = distance_buckets(int(self.bias_spec["rows"]), float(self.bias_spec["far"]))
        if self.nh % self.nk:
            raise ValueError(f"normed_attention: {self.nh} heads are not a multiple of {self.nk} kv heads")
        for name, v in (("window", self.window), ("chunk", self.chunk)):
            if v is not None and int(v) < 1:
                raise ValueError(f"normed_attention: {name} {v} must be >= 1")
        if self.v_from_k and self.vdim != self.dim:
            raise ValueError(f"normed_attention: values taken from keys of {self.dim} cannot have {self.vdim} values")
        if self.dim > 512 or self.vdim > 256:
            raise ValueError(f"normed_attention: keys of {self.dim} (at most 512) and values of {self.vdim} (at most 256)")
        self.names = {k: p.get(k) for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
        self.position = self.value_position = None
        if p.get("position") is not None:
            self.position = make_part(POSITIONS, p["position"], rt, "position encoding")
        if p.get("value_rotation") is not None:
            self.value_position = make_part(POSITIONS, p["value_rotation"], rt, "position encoding")
            if self.vdim % 2 or getattr(self.value_position, "dims", None) != self.vdim:
                raise ValueError(f"normed_attention: the values' rotation must cover all {self.vdim} values in pairs")
        for part in (self.position, self.value_position):
            if part is not None and not (hasattr(part, "pair_tables") or (part is self.position and hasattr(part, "half_tables"))):
                raise ValueError("normed_attention: the position encoding must be a rotation in pairs (pair_tables) or, for "
                                 "queries and keys, in halves (half_tables)")
        self.halves = self.position is not None and not hasattr(self.position, "pair_tables")
        self.qkv = self.o = self.q_gain = self.k_gain = self.far = self.ones = self.bias = None

    def tensor_specs(self):
        n = self.names
        s = {n["q"]: TensorSpec((self.nh * self.dim, self.hidden))}
        if not self.shared_kv:
            s[n["k"]] = TensorSpec((self.nk * self.dim, self.hidden))
        s[n["o"]] = TensorSpec((self.hidden, self.nh * self.vdim))
        if not self.shared_kv and not self.v_from_k:
            s[n["v"]] = TensorSpec((self.nk * self.vdim, self.hidden))
        if self.bias_spec is not None:
            s[self.bias_spec["table"]] = TensorSpec((int(self.bias_spec["rows"]), self.nh))
        if self.gains:
            s[n["q_norm"]] = TensorSpec((self.dim,), init="ones")
            s[n["k_norm"]] = TensorSpec((self.dim,), init="ones")
        if self.distance is not None:
            # random weights: positive numbers, or the logarithm has no value
            s[self.distance[0]] = TensorSpec((self.nh,), init="halves")
            s[self.distance[1]] = TensorSpec((self.nh,), init="halves")
        return s

    def load(self, get):
        n = self.names
        self.qkv = Linear.stacked([get(n[k]) for k in (("q",) if self.shared_kv else ("q", "k") if self.v_from_k
                                                       else ("q", "k", "v"))])
        if self.bias_spec is not None:
            # the table by distance, a row a head: what the kernels look up
            table = get(self.bias_spec["table"]).to(torch.float32)
            rows = torch.tensor(self.bias_rows, dtype=torch.long, device=table.device)
            self.bias = table[rows].t().contiguous()
        self.o = Linear(get(n["o"]))
        if self.gains:
            self.q_gain = get(n["q_norm"]).to(torch.float32).contiguous()
            self.k_gain = get(n["k_norm"]).to(torch.float32).contiguous()
        if self.distance is not None:
            self.far = tuple(get(name).to(torch.float32).contiguous() for name in self.distance)
        self.ones = torch.ones(self.nh, dtype=torch.float32, device=self.o.weight.device)

    def cache_request(self):
        return KVRequest(self.nk, self.dim, None if self.window is None else int(self.window),
                         v_head_dim=None if self.vdim == self.dim else self.vdim,
                         chunk=None if self.chunk is None else int(self.chunk),
                         keep_first=self.keep_first or None)

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.qkv.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length)

    def prepare(self, max_len: int) -> None:
        for part in (self.position, self.value_position):
            if part is not None:
                part.prepare(max_len)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        kc, vc, group = ctx.cache.kv(entry)
        table = ctx.page_table(group)
        qkv = self.qkv(x, out_dtype=torch.float32)
        n, dev = qkv.shape[0], qkv.device
        if self.shared_kv and writes_cache:
            raise ValueError("normed_attention: a layer without keys and values of its own cannot write a cache entry")
        rot = None if self.position is None else (self.position.half_tables if self.halves
                                                  else self.position.pair_tables)(ctx.max_len)
        vrot = None if self.value_position is None else self.value_position.pair_tables(ctx.max_len)
        q = torch.empty((n, self.nh * self.dim), dtype=self.rt.dtype, device=dev)
        ops.qk_norm_prep(qkv, self.q_gain, self.k_gain, self.eps, self.normed, ctx.seq_of_tok, ctx.positions, rot, vrot,
                         self.v_from_k, table, q, kc, vc, self.nh, self.nk, self.dim, self.vdim, writes_cache,
                         halves=self.halves, q_only=self.shared_kv)
        o = torch.empty((n, self.nh * self.vdim), dtype=self.rt.dtype, device=dev)
        window = 0 if self.window is None else int(self.window)
        chunk = 0 if self.chunk is None else int(self.chunk)
        if ops.capped_mfma_takes(self.rt.dtype, self.dim, self.vdim):
            ops.capped_attn_prefill(q, kc, vc, table, ctx, self.ones, o, self.nh, self.nk, self.dim, self.vdim, self.scale,
                                    0.0, window, chunk=chunk, far=self.far, keep_first=self.keep_first, bias=self.bias)
        else:
            ops.capped_attn(q, kc, vc, table, ctx.positions, ctx.seq_of_tok, self.ones, o, self.nh, self.nk, self.dim,
                            self.vdim, self.scale, 0.0, window, ctx.max_len, chunk=chunk, far=self.far,
                            keep_first=self.keep_first, bias=self.bias)
        if vrot is not None or self.out_scale != 1.0:
            ops.unrotate(o, vrot, ctx.positions, self.nh, self.out_scale)
        self.o(o, out=h, accumulate=accumulate)
