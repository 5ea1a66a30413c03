"""The two ends of the model: the embedding table (rows copied, no scaling,
src/graph/builder.rs:60-76, src/graph/cpu_backend.rs:269-285 of yusiwen/minfer) and the output
matrix, which is the embedding table itself when the model ties them (the same storage, no
second copy: src/models/qwen2/loader.rs:260).  Another architecture's scaled embedding, head
bias or logit capping is another registered part, not a change to the model's step."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Embedding, Head, register_embedding, register_head
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
