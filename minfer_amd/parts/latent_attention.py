"""Attention over a shared low-rank latent.

Per token one latent c (rank values, RMS-normed with a weight of its own) and one rotated key
part (rot_dim values) are computed and cached; head h's key is [Wuk_h c | k_rot] and its value
Wuv_h c; the query of a head is [plain (dim) | rotated (rot_dim)]; scores are
(q_plain . k_plain + q_rot . k_rot) * scale over the positions up to the token's own (the last
`window` of them where the design has a window), ordinary softmax; a head's result is multiplied by
sigmoid of a gate computed from the mixer's input, one gate a head or (`gate_per_value`) one for each
of the head's values; the heads are concatenated and projected.  The queries come from the mixer's
input by one matrix, or (`q_rank`) through a latent of their own: c_q = norm(Wdq x) with a weight
vector, q = Wuq c_q.

The per-head keys and values are never built.  Wuk_h is applied to the query instead
((Wuk_h^T q_plain) . c = q_plain . (Wuk_h c)) and Wuv_h to the attention's result over the cached
latents, so the cache holds `rank + rot_dim` values a token whatever the number of heads, and a step's
attention reads each cached row once for all heads.
"""
from __future__ import annotations

import torch

from ..cache.paged import KVRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, POSITIONS, make_part, register_mixer
from .linear import Linear


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """params: hidden_size, n_heads, dim, rot_dim, v_dim, rank, scale, eps (of the latent's norm),
    window (None or int), position (PartSpec of a pairwise rotation over at most rot_dim values),
    gate_per_value (default False), q_rank (None: the queries are one product of the input),
    q, dkv, dkv_norm, uk, uv, gate, o (tensor names; with q_rank, q names the matrix from the queries' latent
    and dq, dq_norm the matrix into it and its norm's weight)."""

    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.nh, self.dn, self.dr, self.dv, self.rank = (
            int(p[k]) for k in ("hidden_size", "n_heads", "dim", "rot_dim", "v_dim", "rank"))
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window = p.get("window")
        if self.window is not None and int(self.window) < 1:
            raise ValueError(f"latent_attention: window {self.window} must be >= 1")
        self.names = {k: p[k] for k in ("q", "dkv", "dkv_norm", "uk", "uv", "gate", "o")}
        self.gate_w = self.dv if p.get("gate_per_value", False) else 1
        self.q_rank = None if p.get("q_rank") is None else int(p["q_rank"])
        if self.q_rank is not None:
            self.names.update(dq=p["dq"], dq_norm=p["dq_norm"])
        self.position = make_part(POSITIONS, p["position"], rt, "position encoding")
        if not hasattr(self.position, "pair_tables"):
            raise ValueError("latent_attention: the position encoding must be a pairwise rotation (pair_tables)")
        self.dk = self.rank + self.dr
        self.proj = self.o = self.uk_t = self.uv_t = self.latent_weight = self.uq = self.q_latent_weight = None

    def tensor_specs(self):
        n, H = self.names, self.nh
        s = {}
        if self.q_rank is None:
            s[n["q"]] = TensorSpec((H * (self.dn + self.dr), self.hidden))
        else:
            s[n["dq"]] = TensorSpec((self.q_rank, self.hidden))
            s[n["dq_norm"]] = TensorSpec((self.q_rank,), init="ones")
            s[n["q"]] = TensorSpec((H * (self.dn + self.dr), self.q_rank))
        s.update({n["dkv"]: TensorSpec((self.dk, self.hidden)),
                  n["dkv_norm"]: TensorSpec((self.rank,), init="ones"),
                  n["uk"]: TensorSpec((H * self.dn, self.rank)),
                  n["uv"]: TensorSpec((H * self.dv, self.rank)),
                  n["gate"]: TensorSpec((H * self.gate_w, self.hidden)),
                  n["o"]: TensorSpec((self.hidden, H * self.dv))})
        return s

    def load(self, get):
        n, H = self.names, self.nh
        # q (or the queries' latent) | dkv | gate over the same input: one product
        first = get(n["q"]) if self.q_rank is None else get(n["dq"])
        self.proj = Linear.stacked([first, get(n["dkv"]), get(n["gate"])])
        self.off_dkv = first.shape[0]
        self.off_gate = self.off_dkv + self.dk
        if self.q_rank is not None:
            self.uq = Linear(get(n["q"]))
            self.q_latent_weight = get(n["dq_norm"]).to(torch.float32).contiguous()
        self.latent_weight = get(n["dkv_norm"]).to(torch.float32).contiguous()
        # per-head matrices: Wuk_h^T takes q_plain to the latent's side, Wuv_h takes the result over
        # the latents to the head's values.  The matrix-core kernel reads them output-major
        # ([rank][dim], [v_dim][rank]), the plain one input-major.
        uk, uv = get(n["uk"]).view(H, self.dn, self.rank), get(n["uv"]).view(H, self.dv, self.rank)
        self.uk_mfma = ops.headwise_mfma_takes(uk.dtype, self.dn, self.dn) and self.rt.is_bf16
        self.uv_mfma = ops.headwise_mfma_takes(uv.dtype, self.rank, self.rank) and self.rt.is_bf16
        self.uk_t = (uk.transpose(1, 2) if self.uk_mfma else uk).contiguous()
        self.uv_t = (uv if self.uv_mfma else uv.transpose(1, 2)).contiguous()
        self.o = Linear(get(n["o"]))

    def cache_request(self):
        # one shared "kv head" of rank + rot_dim values; the values are the rows' first `rank` columns
        return KVRequest(1, self.dk, None if self.window is None else int(self.window), v_head_dim=0)

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.proj.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length) + \
            (0 if self.uq is None else self.uq.decode_copy(make, min_row_length))

    def prepare(self, max_len: int) -> None:
        self.position.prepare(max_len)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        rows, _, group = ctx.cache.kv(entry)
        table = ctx.page_table(group)
        n, H, dev, dt = x.shape[0], self.nh, x.device, self.rt.dtype
        proj = self.proj(x, out_dtype=torch.float32)
        cos, sin = self.position.pair_tables(ctx.max_len)
        q_plain = torch.empty((n, H, self.dn), dtype=dt, device=dev)
        q_abs = torch.empty((n, H, self.dk), dtype=dt, device=dev)
        gate = torch.empty((n, H) if self.gate_w == 1 else (n, H, self.gate_w), dtype=torch.float32, device=dev)
        q_rows = None
        if self.q_rank is not None:
            # the queries' latent: the first columns of the product, normed into the run type, then up to the heads
            c_q = torch.empty((n, self.q_rank), dtype=dt, device=dev)
            ops.rmsnorm(proj, self.q_latent_weight, self.eps, c_q, cols=self.q_rank)
            q_rows = self.uq(c_q, out_dtype=torch.float32)
        ops.latent_prep(proj, self.off_dkv, self.off_gate, self.latent_weight, self.eps, cos, sin, ctx.positions,
                        ctx.seq_of_tok, table, rows, q_plain, q_abs, gate, H, self.dn, self.dr, self.rank, writes_cache,
                        q_rows=q_rows)
        (ops.headwise_linear_mfma if self.uk_mfma else ops.headwise_linear)(q_plain, self.dn, self.uk_t, q_abs, self.rank)
        o_lat = torch.empty((n, H, self.rank), dtype=dt, device=dev)
        ops.latent_attn(q_abs, rows, table, ctx.positions, ctx.seq_of_tok, o_lat, self.rank, self.scale,
                        0 if self.window is None else int(self.window), ctx.max_len, ctx=ctx)
        o = torch.empty((n, H, self.dv), dtype=dt, device=dev)
        (ops.headwise_linear_mfma if self.uv_mfma else ops.headwise_linear)(o_lat, self.rank, self.uv_t, o, self.dv,
                                                                             gate=gate)
        self.o(o.view(n, H * self.dv), out=h, accumulate=accumulate)
