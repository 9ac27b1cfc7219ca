"""Linear attention whose forget gate a sets the input gate as well, 1 - a (HGRN2): a fixed-size matrix
state per sequence and head instead of keys and values.

q = silu(Wq x) (heads x dim), v = Wv x (heads x v_dim), a = l + (1 - l) sigmoid(Wf x + b) per head and key
channel, with learned lower bounds l; per head S_t = diag(a_t) S_(t-1) + (1 - a_t) v_t^T from S = 0 at a
sequence's start, o_t = S_t^T q_t, no key and no other scale; every head's o is RMS-normed over its v_dim
values with a gain vector shared by the heads, the heads side by side are multiplied by `out_scale` and
projected by Wo.  The state is float32 `[heads][dim][v_dim]` per cache slot; gates, state, products and sums
are 32-bit in both run types.
"""
from __future__ import annotations

import torch

from ..cache.paged import StateRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, register_mixer
from .linear import Linear

# a step whose longest sequence brings more tokens than this walks its sequences in chunks side by side
CHUNKED_FROM = ops.GR_CHUNK


@register_mixer("gated_recurrence")
class GatedRecurrence(Mixer):
    """params: hidden_size, n_heads, dim, v_dim, eps (of the norm over a head), out_scale, q, f, f_bias, lower, v,
    norm, o (tensor names)."""

    takes_normed = True
    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.nh, self.dim, self.vdim = (int(p[k]) for k in ("hidden_size", "n_heads", "dim", "v_dim"))
        self.eps = float(p["eps"])
        self.out_scale = float(p.get("out_scale", 1.0))
        if self.dim > 256:
            raise ValueError(f"gated_recurrence: key width {self.dim} is beyond what the kernels take (256)")
        self.names = {k: p[k] for k in ("q", "f", "f_bias", "lower", "v", "norm", "o")}
        self.proj = self.o = self.norm_weight = self.lower = None

    def tensor_specs(self):
        n, H = self.names, self.nh
        return {n["q"]: TensorSpec((H * self.dim, self.hidden)), n["f"]: TensorSpec((H * self.dim, self.hidden)),
                n["f_bias"]: TensorSpec((H * self.dim,)), n["lower"]: TensorSpec((H * self.dim,), init="halves"),
                n["v"]: TensorSpec((H * self.vdim, self.hidden)), n["norm"]: TensorSpec((self.vdim,), init="ones"),
                n["o"]: TensorSpec((self.hidden, H * self.vdim))}

    def load(self, get):
        n = self.names
        self.proj = Linear.stacked([get(n["q"]), get(n["f"]), get(n["v"])], [None, get(n["f_bias"]), None])   # one product
        self.o = Linear(get(n["o"]))
        self.norm_weight = get(n["norm"]).to(torch.float32).contiguous()
        self.lower = get(n["lower"]).to(torch.float32).contiguous()

    def cache_request(self):
        return StateRequest((self.nh, self.dim, self.vdim), torch.float32)

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.proj.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        state = ctx.cache.state(entry)
        proj = self.proj(x, out_dtype=torch.float32)
        n, hv = proj.shape[0], self.nh * self.vdim
        o = torch.empty((n, hv), dtype=torch.float32, device=proj.device)
        chunks = None
        if not ctx.all_decode and ctx.max_new > CHUNKED_FROM:
            key = ("gr_chunks",)
            if key not in ctx._memo:
                table, count = ops.gr_chunks(ctx.host_new)
                ctx._memo[key] = (table.to(proj.device), count)
            chunks = ctx._memo[key]
        ops.gated_scan(proj, self.lower, ctx.cu_seqlens, ctx.slot_ids, state, o, self.nh, self.dim, self.vdim, chunks)
        y = torch.empty((n, hv), dtype=self.rt.dtype, device=proj.device)
        ops.head_rmsnorm(o, self.norm_weight, self.eps, y, self.nh, self.out_scale)
        self.o(y, out=h, accumulate=accumulate)
