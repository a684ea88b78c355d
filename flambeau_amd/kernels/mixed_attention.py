"""The kernel set of attention whose heads' scores are mixed before the softmax (distance bias, mixing
matrix, sink): every block of the kernel takes all heads of a query token.  The plain form gives a token
to one block; the tuned form deals the keys of a step of few rows out to several blocks per token, as
the split-K decode kernel of plain attention does, and joins the parts afterwards."""
from __future__ import annotations

import torch

from . import ops
from .sets import register_kernel_set

PART_KEYS = 128       # keys per part (a multiple of the kernel's chunk), aligned to absolute positions
FEW_ROWS = 64         # steps of up to this many rows deal their keys out


class PlainMixedAttention:
    def __init__(self, rt):
        self.rt = rt

    def signature(self, batch, window: int):
        """What the kernels decide from the contexts' lengths (part of a recorded step's key)."""
        return 0

    def attention(self, q, out, kv, step, table, n_heads, scale, window, slopes, talk, sink):
        return ops.attn_mixed(q, out, kv, step.positions, step.tok_seq, table, n_heads, scale, window, slopes, talk, sink)


class TunedMixedAttention(PlainMixedAttention):
    def signature(self, batch, window: int):
        """The number of parts a token's keys are dealt out to (0: one block per token)."""
        ctx = batch.ctx_bound or batch.max_ctx_len
        keys = min(window, ctx) if window else ctx
        if batch.n_tokens > FEW_ROWS or keys <= 2 * PART_KEYS:
            return 0
        parts = (keys - 1) // PART_KEYS + 2          # (a run of keys may begin anywhere inside its first part)
        return 1 << (parts - 1).bit_length()

    def attention(self, q, out, kv, step, table, n_heads, scale, window, slopes, talk, sink):
        parts = self.signature(step.host, window)
        if not parts:
            return super().attention(q, out, kv, step, table, n_heads, scale, window, slopes, talk, sink)
        n, rt = q.shape[0], self.rt
        acc = rt.buffer("amix_part_acc", n, parts * n_heads * kv.head_dim, torch.float32)
        ml = rt.buffer("amix_part_ml", n, parts * n_heads * 2, torch.float32)
        return ops.attn_mixed(q, out, kv, step.positions, step.tok_seq, table, n_heads, scale, window, slopes, talk, sink,
                              part_keys=PART_KEYS, n_parts=parts, part_acc=acc, part_ml=ml)


register_kernel_set("mixed_heads_attention", PlainMixedAttention, TunedMixedAttention)
