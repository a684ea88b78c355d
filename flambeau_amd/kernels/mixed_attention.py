"""The kernel set of attention whose heads' scores are mixed before the softmax (distance bias, mixing
matrix, sink): every block of the kernels takes all heads of its query tokens.  The plain form gives a token
to one block.  The tuned form runs bfloat16 caches on the matrix cores, 16 rows of a request per block, and deals
the keys of a step of few rows out to several blocks per tile, as the split-K decode kernel of plain attention
does, joining the parts afterwards; sizes the matrix-core kernel does not take go the plain way, with parts."""
from __future__ import annotations

import torch

from . import ops
from .sets import register_kernel_set

PART_KEYS = 64        # keys per part of a step of few rows (a multiple of the kernels' chunk), aligned to absolute positions
FEW_ROWS = 64         # steps of up to this many rows deal their keys out that finely
TILE_ROWS = 16        # rows of a request that a block of the matrix-core kernel takes
PROMPT_PART_KEYS = 512    # keys per part of a larger step whose tiles alone do not fill the chip
FULL_CHIP_TILES = 512     # from this many tiles on nothing is dealt out


class PlainMixedAttention:
    def __init__(self, rt):
        self.rt = rt

    def signature(self, batch, window: int):
        """What the kernels decide from the contexts' lengths (part of a recorded step's key)."""
        return 0

    def attention(self, q, out, kv, step, table, n_heads, scale, window, slopes, talk, sink, keep_first=0, chunk=0):
        return ops.attn_mixed(q, out, kv, step.positions, step.tok_seq, table, n_heads, scale, window, slopes, talk, sink,
                              keep_first=keep_first, chunk=chunk)


class TunedMixedAttention(PlainMixedAttention):
    def signature(self, batch, window: int):
        """``(keys per part, parts)`` a tile's keys are dealt out to; ``(0, 0)``: one block finishes a tile.  ``window``:
        how far back a row's own run of keys can reach (its window, or the length of its chunk of positions; 0: to
        the start).  Kept first tokens are not dealt out: the first part's block takes them."""
        ctx = batch.ctx_bound or batch.max_ctx_len
        keys = min(window + TILE_ROWS - 1, ctx) if window else ctx          # (what the rows of a tile see together)
        if batch.n_tokens <= FEW_ROWS:
            part_keys = PART_KEYS
        elif sum(-(-rows // TILE_ROWS) for rows in batch.q_lens) < FULL_CHIP_TILES:
            part_keys = PROMPT_PART_KEYS
        else:
            return (0, 0)
        if keys <= 2 * part_keys:
            return (0, 0)
        parts = (keys - 1) // part_keys + 2          # (a run of keys may begin anywhere inside its first part)
        return (part_keys, 1 << (parts - 1).bit_length())

    def attention(self, q, out, kv, step, table, n_heads, scale, window, slopes, talk, sink, keep_first=0, chunk=0):
        part_keys, parts = self.signature(step.host, window or chunk)
        n, rt = q.shape[0], self.rt
        split = {}
        if parts:
            split = dict(part_keys=part_keys, n_parts=parts,
                         part_acc=rt.buffer("amix_part_acc", n, parts * n_heads * kv.head_dim, torch.float32),
                         part_ml=rt.buffer("amix_part_ml", n, parts * n_heads * 2, torch.float32))
        if kv.pool.dtype == torch.bfloat16 and ops.attn_mixed_tiled_fits(n_heads, kv.head_dim, kv.page_size):
            n_tiles = sum(-(-rows // TILE_ROWS) for rows in step.host.q_lens)
            return ops.attn_mixed_tiled(q, out, kv, step.positions, table, step.seq_q_start, step.seq_q_len, n_tiles, n_heads, scale,
                                        window, slopes, talk, sink, keep_first=keep_first, chunk=chunk, **split)
        return ops.attn_mixed(q, out, kv, step.positions, step.tok_seq, table, n_heads, scale, window, slopes, talk, sink,
                              keep_first=keep_first, chunk=chunk, **split)


register_kernel_set("mixed_heads_attention", PlainMixedAttention, TunedMixedAttention)
