"""The two ends of the model: the embedding table (rows copied, no scaling,
src/graph/builder.rs:60-76, src/graph/cpu_backend.rs:269-285 of yusiwen/minfer) and the output
matrix, which is the embedding table itself when the model ties them (the same storage, no
second copy: src/models/qwen2/loader.rs:260).  Another architecture's scaled embedding, head
bias or logit capping is another registered part, not a change to the model's step."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import NORMS, Runtime, Embedding, Head, make_part, register_embedding, register_head
from .linear import Linear


@register_embedding("token_embedding")
class TokenEmbedding(Embedding):
    """params: name (tensor), vocab_size, hidden_size."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.name = spec.params["name"]
        self.vocab, self.hidden = int(spec.params["vocab_size"]), int(spec.params["hidden_size"])
        self.weight = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.vocab, self.hidden))}

    def load(self, get):
        self.weight = get(self.name).contiguous()

    def table(self):
        return self.weight

    def forward(self, token_ids, out, ctx=None) -> None:
        ops.embed(self.weight, token_ids, out)


@register_embedding("normed_token_embedding")
class NormedTokenEmbedding(TokenEmbedding):
    """The table's row, then a norm of its own over it before anything else reads the stream.
    params: name (tensor), vocab_size, hidden_size, norm (PartSpec of a registered norm)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.norm = make_part(NORMS, spec.params["norm"], Runtime(torch.float32, rt.device), "norm")

    def tensor_specs(self):
        return dict(super().tensor_specs(), **self.norm.tensor_specs())

    def load(self, get):
        super().load(get)
        self.norm.load(get)

    def forward(self, token_ids, out, ctx=None) -> None:
        ops.embed(self.weight, token_ids, out)
        self.norm.forward(out, out=out)       # in place, 32-bit rows


@register_head("linear_head")
class LinearHead(Head):
    """params: name (tensor; None: tied to the embedding's table), vocab_size, hidden_size."""

    takes_normed = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.name = spec.params.get("name")
        self.vocab, self.hidden = int(spec.params["vocab_size"]), int(spec.params["hidden_size"])
        self.linear = None

    def tensor_specs(self):
        return {} if self.name is None else {self.name: TensorSpec((self.vocab, self.hidden))}

    def load(self, get):
        if self.name is not None:
            self.linear = Linear(get(self.name))

    def tie(self, embedding) -> None:
        if self.name is None:
            table = embedding.table()
            if table is None or tuple(table.shape) != (self.vocab, self.hidden):
                raise ValueError("linear_head: tied to an embedding that has no [vocab][hidden] table")
            self.linear = Linear(table)

    @property
    def weight(self) -> torch.Tensor:
        return self.linear.weight

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.linear.decode_copy(make, min_row_length)

    def forward(self, x, ctx=None) -> torch.Tensor:
        return self.linear(x, out_dtype=torch.float32)


@register_head("capped_linear_head")
class CappedLinearHead(LinearHead):
    """The linear head with capped logits: z <- cap tanh(z / cap), in 32-bit.  params: those of `linear_head`, and cap."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.cap = float(spec.params["cap"])
        if not self.cap > 0:
            raise ValueError(f"capped_linear_head: cap {self.cap} must be positive")

    def forward(self, x, ctx=None) -> torch.Tensor:
        logits = super().forward(x, ctx)
        ops.softcap(logits, self.cap)
        return logits


@register_embedding("token_position_embedding")
class TokenPositionEmbedding(TokenEmbedding):
    """The table's row plus a learned row for the token's position (not scaled), added in 32-bit.
    params: name, positions (tensors), vocab_size, hidden_size, max_positions."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.pos_name, self.max_positions = spec.params["positions"], int(spec.params["max_positions"])
        self.pos = None

    def tensor_specs(self):
        return dict(super().tensor_specs(), **{self.pos_name: TensorSpec((self.max_positions, self.hidden))})

    def load(self, get):
        super().load(get)
        self.pos = get(self.pos_name).to(self.weight.dtype).contiguous()

    def forward(self, token_ids, out, ctx=None) -> None:
        ops.embed_pos(self.weight, self.pos, token_ids, ctx.positions, out)
