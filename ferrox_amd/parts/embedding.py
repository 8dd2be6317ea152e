"""Token embedding (the reference's has no scale, ferrox-models/src/decoder.rs:1279-1284; `scale` multiplies the rows
of a design that has one) and the output
head, applied to the wanted rows only (decoder.rs:2994-3009); a tied head shares
the embedding table (ferrox-models/src/loader.rs:1433-1436)."""
from __future__ import annotations

import math

from .. import ops
from .base import EMBEDDINGS, HEADS, ParamSpec, Part
from .linear import matmul


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Part):
    kernel_libraries = ("elementwise",)

    def __init__(self, vocab_size: int, hidden_size: int, name: str = "weight", scale: float = 1.0,
                 position_table: str | None = None, max_positions: int = 0):
        """`scale`: a constant that every embedding row is multiplied by on its way into the float32 stream.
        `position_table`: the name of a learned [max_positions, hidden] table; row p of it is added (unscaled) to
        the row of a token at position p."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.name = name
        self.scale = float(scale)
        if not math.isfinite(self.scale):
            raise ValueError(f"an embedding scale of {scale}")
        self.position_table, self.max_positions = position_table or None, int(max_positions)
        if self.position_table and self.max_positions < 1:
            raise ValueError("a table of positions needs `max_positions`")
        self.uses_positions = self.position_table is not None       # forward then takes positions=
        self.weight = self.positions = None

    def param_specs(self):
        specs = {self.name: ParamSpec((self.vocab_size, self.hidden_size))}
        if self.position_table:
            specs[self.position_table] = ParamSpec((self.max_positions, self.hidden_size))
        return specs

    def load(self, fetch):
        self.weight = fetch(self.name).contiguous()
        if self.position_table:
            self.positions = fetch(self.position_table).to(self.weight.dtype).contiguous()

    def forward(self, token_ids, positions=None):
        if self.position_table:
            return ops.embed(self.weight, token_ids, scale=self.scale, position_table=self.positions, positions=positions)
        return ops.embed(self.weight, token_ids, scale=self.scale)


@HEADS.register("linear_head")
class LinearHead(Part):
    kernel_libraries = ("gemm",)

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: str | None = None, name: str = "weight"):
        """`name`: what the head's own matrix is called behind the part's prefix.  `tied_to`: the full name of another part's [vocab, hidden] tensor that serves as this head's matrix (the
        embedding table of a model with tied embeddings); the head then has no tensor of its own."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to or None
        self.name = name
        self.weight = None

    def param_specs(self):
        return {} if self.tied_to else {self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def borrows(self):
        return [self.tied_to] if self.tied_to else []

    def load(self, fetch):
        self.weight = (fetch.shared(self.tied_to) if self.tied_to else fetch(self.name)).contiguous()
        if tuple(self.weight.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"the head's matrix {self.tied_to or self.name} has shape {tuple(self.weight.shape)}, "
                             f"not [{self.vocab_size}, {self.hidden_size}]")

    def forward(self, x):
        """float32 logits [rows, vocab]."""
        return matmul(x, self.weight, epilogue=ops.EPI_STORE_F32)
