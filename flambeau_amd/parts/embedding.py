"""Token embedding and output head.  Both are parts like the others: a model's description names
them by registry key (``EMBEDDINGS``, ``HEADS``), so a scaled embedding or a head with a soft cap is
another registered class, not a change to the model's code.  An embedding must offer ``weight``
(the table, for a tied head) and ``forward(tokens, out)``; a head ``bind(weights, rt,
embedding_table=...)`` and ``forward(x, max_rows) -> float32 logits``.

h0[i,:] = E[token[i],:], no scaling (crates/forward/src/core/composites/embed.rs:26-62);
logits = norm_f(x) Wlm^T in 32-bit, a tied head being the embedding table again
(crates/forward/src/core/composites/output_head.rs:41-100,
crates/models/qwen35-v2/src/loader.rs:218-223)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, NORMS, Part, TensorSpec


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Part):
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size

    def tensors(self):
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size), "table")}

    def bind(self, weights, rt):
        self.rt = rt
        self.weight = weights["weight"]

    def forward(self, tokens, out):
        return ops.embed(self.weight, tokens, out)


@HEADS.register("linear_head")
class OutputHead(Part):
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied

    def tensors(self):
        return {} if self.tied else {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, weights, rt, embedding_table=None):
        self.rt = rt
        table = embedding_table if self.tied else weights["weight"]
        if table is None:
            raise ValueError("a tied output head needs the embedding table")
        # a tied head packs its own copy: the embedding keeps the row-major table for its gather
        self.weight = rt.prepare_weight(table)

    def forward(self, x, max_rows):
        logits = self.rt.buffer("logits", x.shape[0], self.vocab_size, torch.float32, max_rows=max_rows)
        self.rt.gemm(x, self.weight, logits)
        return logits


@EMBEDDINGS.register("scaled_token_embedding")
class ScaledTokenEmbedding(TokenEmbedding):
    """h0[i, :] = E[token[i], :] * scale, the product taken in 32-bit."""

    def __init__(self, vocab_size: int, hidden_size: int, scale: float):
        super().__init__(vocab_size, hidden_size)
        self.scale = float(scale)

    def forward(self, tokens, out):
        return ops.embed_scaled(self.weight, tokens, out, self.scale)


@EMBEDDINGS.register("positional_token_embedding")
class PositionalTokenEmbedding(TokenEmbedding):
    """h0[i, :] = E[token[i], :] + P[position[i], :] (a learned row per position, not scaled), then an optional
    norm (any registered one).  ``wants_step``: ``forward`` is given the step, whose positions it reads."""
    wants_step = True

    def __init__(self, vocab_size: int, hidden_size: int, max_positions: int, norm=None):
        super().__init__(vocab_size, hidden_size)
        self.max_positions = max_positions
        self.norm = NORMS.create(norm) if norm is not None else None

    def subparts(self):
        return [self.norm] if self.norm is not None else []

    def tensors(self):
        t = {"weight": TensorSpec((self.vocab_size, self.hidden_size), "table"),
             "positions": TensorSpec((self.max_positions, self.hidden_size), "table")}
        if self.norm is not None:
            t.update({"norm." + k: v for k, v in self.norm.tensors().items()})
        return t

    def bind(self, weights, rt):
        self.rt = rt
        self.weight, self.positions = weights["weight"], weights["positions"]
        if self.norm is not None:
            self.norm.bind({k[5:]: v for k, v in weights.items() if k.startswith("norm.")}, rt)

    def forward(self, tokens, out, step=None):
        if step is None:
            raise RuntimeError("positional_token_embedding: the step (its positions) is needed")
        ops.embed_positions(self.weight, self.positions, tokens, step.positions, out)
        if self.norm is not None:
            self.norm.forward(out, out)
        return out


@HEADS.register("capped_linear_head")
class CappedOutputHead(OutputHead):
    """logits = cap * tanh((x W^T) / cap), applied to the 32-bit products; ``softcap=None`` leaves them as they are."""

    def __init__(self, vocab_size: int, hidden_size: int, softcap: float | None = None, tied: bool = False):
        super().__init__(vocab_size, hidden_size, tied)
        self.softcap = float(softcap) if softcap else None

    def forward(self, x, max_rows):
        logits = super().forward(x, max_rows)
        return ops.softcap_inplace(logits, self.softcap) if self.softcap is not None else logits


@HEADS.register("scaled_linear_head")
class ScaledOutputHead(OutputHead):
    """logits = (x W^T) * scale, the factor applied to the 32-bit products."""

    def __init__(self, vocab_size: int, hidden_size: int, scale: float, tied: bool = False):
        super().__init__(vocab_size, hidden_size, tied)
        self.scale = float(scale)

    def forward(self, x, max_rows):
        logits = super().forward(x, max_rows)
        return ops.scale_inplace(logits, self.scale) if self.scale != 1.0 else logits
