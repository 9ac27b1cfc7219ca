"""Mixture-of-experts feed-forward with a router that first keeps the best groups of experts.

Router: z = Wr x in 32-bit, scores = softmax(z) over all experts; the experts form `groups` equal
groups of neighbours, a group's score is its best expert's, and only experts of the `keep` best groups
can be among the `top` chosen; the chosen experts' scores over their sum are the weights.
With one group (and so all of it kept) the weights are the softmax over the chosen logits alone.  A router may
add a bias per expert to its logits.  A router may also score with sigmoid(z) instead of the softmax, choose
groups and experts by score plus a correction per expert while weighing by the scores themselves, count a group
by the sum of its `group_top` best (corrected) scores, and multiply the weights by a scale.
Expert (no biases): g = min(Wg x, limit), u = clamp(Wu x, -limit, limit), y = g sigmoid(1.702 g) (u + 1),
output Wd y; or, with `act` "silu", the plain gated form y = silu(Wg x) (Wu x).  The result is the weighted sum
of the chosen experts' outputs.

Two forms, both of which read or multiply only what was chosen.  Steps of few tokens and decode steps (which
may be captured, so nothing may wait for the host): `ops.moe_sparse`, up to 16 tokens a launch, reads every
chosen expert's matrices once.  Steps of many tokens: the (token, choice) pairs are grouped by expert
(`ops.moe_group`; the host reads the experts' counts, the one wait of the step), the tokens' rows are put side by
side expert by expert, every expert with tokens runs its two products over its rows, and the rows' results are
added into the stream with the tokens' weights, a token's choices in their order.

A step whose context carries a list under `_memo["route_log"]` gets every routed layer's choices
(`[rows][top]` expert numbers, on the device) appended to it, in run order.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, register_feed_forward
from .linear import Linear

# steps of at most this many tokens read only the chosen experts' matrices
SPARSE_UP_TO = ops.MOE_SPARSE_TOKENS


@register_feed_forward("grouped_moe")
class GroupedMoE(FeedForward):
    """params: hidden_size, intermediate_size (of one expert), n_experts, top, groups and keep (default 1: no
    groups), act ("clamped_swish", the default, with `limit`; or "silu"), router (tensor name), router_bias
    (tensor name, or None), score ("softmax", the default, or "sigmoid"), correction (tensor name, or None),
    group_top (default 1), weight_scale (default 1.0), expert (format of an expert's tensor stem, e.g. "mlp.e{}";
    its matrices are stem + ".gate", ".up", ".down")."""

    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter, self.ne, self.top = (
            int(p[k]) for k in ("hidden_size", "intermediate_size", "n_experts", "top"))
        self.groups, self.keep = int(p.get("groups", 1)), int(p.get("keep", p.get("groups", 1)))
        act = p.get("act", "clamped_swish")
        if act not in ops.MOE_ACTS:
            raise ValueError(f"grouped_moe: activation {act!r} is not one of {sorted(ops.MOE_ACTS)}")
        self.act = ops.MOE_ACTS[act]
        self.limit = float(p["limit"]) if act == "clamped_swish" else 0.0
        self.router_name, self.expert_name = p["router"], p["expert"]
        self.bias_name = p.get("router_bias")
        self.correction_name = p.get("correction")
        self.score, self.group_top = p.get("score", "softmax"), int(p.get("group_top", 1))
        self.weight_scale = float(p.get("weight_scale", 1.0))
        if self.score not in ops.MOE_SCORES or self.group_top < 1:
            raise ValueError(f"grouped_moe: scores {self.score!r} (one of {sorted(ops.MOE_SCORES)}), group_top {self.group_top}")
        per = self.ne // max(1, self.groups)
        if self.ne % self.groups or not 1 <= self.keep <= self.groups or not 1 <= self.top <= min(64, self.keep * per) \
                or self.ne > ops.MOE_MAX_EXPERTS:
            raise ValueError(f"grouped_moe: {self.ne} experts in {self.groups} groups, {self.keep} kept, {self.top} chosen")
        self.router = self.router_bias = self.correction = self.gate_up = self.down = None

    def tensor_specs(self):
        s = {self.router_name: TensorSpec((self.ne, self.hidden))}
        if self.bias_name is not None:
            s[self.bias_name] = TensorSpec((self.ne,))
        if self.correction_name is not None:
            s[self.correction_name] = TensorSpec((self.ne,))
        for e in range(self.ne):
            stem = self.expert_name.format(e)
            s[stem + ".gate"] = TensorSpec((self.inter, self.hidden))
            s[stem + ".up"] = TensorSpec((self.inter, self.hidden))
            s[stem + ".down"] = TensorSpec((self.hidden, self.inter))
        return s

    def load(self, get):
        self.router = get(self.router_name).to(torch.float32).contiguous()   # the router's product is 32-bit
        if self.bias_name is not None:
            self.router_bias = get(self.bias_name).to(torch.float32).contiguous()
        if self.correction_name is not None:
            self.correction = get(self.correction_name).to(torch.float32).contiguous()
        stems = [self.expert_name.format(e) for e in range(self.ne)]
        # [experts][gate | up][hidden] and [experts][hidden][inter]: an expert's matrices are contiguous slices
        self.gate_up = torch.stack([torch.cat([get(s + ".gate"), get(s + ".up")], dim=0) for s in stems]).contiguous()
        self.down = torch.stack([get(s + ".down") for s in stems]).contiguous()
        self.experts = [(Linear(self.gate_up[e]), Linear(self.down[e])) for e in range(self.ne)]

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return 0

    def forward(self, x, h, ctx, accumulate: bool = True) -> None:
        n, dev = x.shape[0], x.device
        chosen = torch.empty((n, self.top), dtype=torch.int32, device=dev)
        weights = torch.empty((n, self.top), dtype=torch.float32, device=dev)
        ops.moe_route(x, self.router, None, chosen, weights, self.groups, self.keep, bias=self.router_bias,
                      score=self.score, correction=self.correction, group_top=self.group_top,
                      weight_scale=self.weight_scale)
        log = ctx._memo.get("route_log") if ctx is not None else None
        if log is not None:                  # a caller that wants to know: every routed layer's choices, in run order
            log.append(chosen)
        if n == 0:
            return
        few = min(SPARSE_UP_TO, max(1, ops.MOE_SPARSE_PAIRS // self.top))
        if (n <= few or (ctx is not None and ctx.all_decode)) and x.dtype == self.gate_up.dtype:
            if not accumulate:
                h.zero_()
            for t0 in range(0, n, few):      # (slices of a contiguous tensor's rows are contiguous)
                ops.moe_sparse(x[t0:t0 + few], self.gate_up, self.down, chosen[t0:t0 + few], weights[t0:t0 + few],
                               h[t0:t0 + few], self.ne, self.limit, self.act)
            return
        rank = torch.empty_like(chosen)
        counts = torch.empty(self.ne, dtype=torch.int32, device=dev)
        ops.moe_group(chosen, self.ne, rank, counts)
        per_expert = [int(c) for c in counts.cpu()]          # the step waits for the host here
        starts = [0]
        for c in per_expert:
            starts.append(starts[-1] + c)
        offsets = torch.tensor(starts[:-1], dtype=torch.int32).to(dev)
        pairs = n * self.top
        xs = torch.empty((pairs, self.hidden), dtype=x.dtype, device=dev)
        ops.moe_gather(x, chosen, rank, offsets, xs)
        gu = torch.empty((pairs, 2 * self.inter), dtype=torch.float32, device=dev)
        for e, (gate_up, _) in enumerate(self.experts):
            if per_expert[e]:
                gate_up(xs[starts[e]:starts[e + 1]], out=gu[starts[e]:starts[e + 1]])
        y = torch.empty((pairs, self.inter), dtype=self.rt.dtype, device=dev)
        ops.moe_act(gu, self._ones(pairs, dev), y, self.limit, self.act)
        rows = torch.empty((pairs, self.hidden), dtype=torch.float32, device=dev)
        for e, (_, down) in enumerate(self.experts):
            if per_expert[e]:
                down(y[starts[e]:starts[e + 1]], out=rows[starts[e]:starts[e + 1]])
        ops.moe_combine(rows, chosen, rank, offsets, weights, h, accumulate=accumulate)

    def _ones(self, n: int, dev) -> torch.Tensor:
        """[n][1] ones: the activation kernel's weights where the weighting happens later."""
        have = getattr(self, "_ones_buf", None)
        if have is None or have.shape[0] < n:
            have = self._ones_buf = torch.ones((max(n, 4096), 1), dtype=torch.float32, device=dev)
        return have[:n]
