"""Typed wrappers of the plain kernels.

Each wrapper checks on the host that the tensors have the device, dtype, contiguity
and shape the kernel and its grid assume, and only then launches on torch's current
stream.  (The reference keeps the same split: typed, bounds-checked leaf functions
above raw launches, crates/model-ops/src/lib.rs:47-82.)
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .library import KernelError, call

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {dtype}: the kernels take float32 and bfloat16") from None


_pinned_stream = None


def stream_handle() -> int:
    """The stream kernels are launched on: torch's current one, or the one pinned for a forward pass."""
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class pinned_stream:
    """``with pinned_stream():`` every launch inside goes to the stream that is current on entry.
    Asking torch for its current stream at each of a step's two hundred launches costs more than
    the launches; nothing inside a forward pass changes the stream."""

    def __enter__(self):
        global _pinned_stream
        self.prev = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self.prev


def _check(t: torch.Tensor, name: str, dtype=None, shape=None):
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}, the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None:
        have = t.shape
        ok = len(have) == len(shape)
        if ok:
            for s, e in zip(have, shape):
                if e is not None and e != s:
                    ok = False
                    break
        if not ok:
            raise KernelError(f"{name}: shape {tuple(have)}, expected {tuple(shape)}")
    return t.data_ptr()


@dataclass
class PagedLayerCache:
    """The key/value pool of one layer: ``pool[n_pages, 2, n_kv_heads, page_size, head_dim]``."""
    pool: torch.Tensor

    @property
    def n_pages(self): return self.pool.shape[0]
    @property
    def n_kv_heads(self): return self.pool.shape[2]
    @property
    def page_size(self): return self.pool.shape[3]
    @property
    def head_dim(self): return self.pool.shape[4]


def embed(table, tokens, out):
    V, H = table.shape
    n = tokens.shape[0]
    call("fl_embed", _check(table, "embed.table"), dtype_code(table.dtype),
         _check(tokens, "embed.tokens", torch.int32, (n,)),
         _check(out, "embed.out", torch.float32, (n, H)), n, H, V, stream_handle())
    return out


def gather_rows(src, rows, out):
    """``out[r] = src[rows[r]]`` for a float32 ``src`` (the embedding kernel over a table of rows)."""
    return embed(src, rows, out)


def rmsnorm(x, weight, out, eps, delta=None, store_sum=False, rows=None):
    """``out = rmsnorm(x (+ delta)) * weight``; ``store_sum`` writes x + delta back into x;
    ``rows`` (int32) picks the rows of x that are normed, one output row each."""
    n, H = x.shape
    px = _check(x, "rmsnorm.x", torch.float32, (n, H))
    pd = _check(delta, "rmsnorm.delta", torch.float32, (n, H)) if delta is not None else None
    pr = _check(rows, "rmsnorm.rows", torch.int32) if rows is not None else None
    n_out = rows.shape[0] if rows is not None else n
    if store_sum and delta is None:
        store_sum = False
    call("fl_rmsnorm", px, pd, px if store_sum else None, pr,
         _check(weight, "rmsnorm.weight", torch.float32, (H,)),
         _check(out, "rmsnorm.out", None, (n_out, H)), dtype_code(out.dtype), n_out, H, float(eps),
         stream_handle())
    return out


def add_inplace(x, delta):
    if x.shape != delta.shape:
        raise KernelError(f"add: shapes {tuple(x.shape)} and {tuple(delta.shape)} differ")
    call("fl_add_inplace", _check(x, "add.x", torch.float32), _check(delta, "add.delta", torch.float32),
         x.numel(), stream_handle())
    return x


def gemm_plain(x, w, out):
    """``out[m, n] = sum_k x[m, k] w[n, k]``."""
    M, K = x.shape
    N = w.shape[0]
    call("fl_gemm_plain", _check(x, "gemm.x", w.dtype, (M, K)), _check(w, "gemm.w", None, (N, K)),
         _check(out, "gemm.out", None, (M, N)), dtype_code(x.dtype), dtype_code(out.dtype), M, N, K,
         stream_handle())
    return out


def rope_table(positions, rotated_dims, theta, out):
    """``out[n, rotated_dims / 2, 2]`` = (cos, sin)(position * theta^(-2 i / rotated_dims)), float32."""
    n = positions.shape[0]
    call("fl_rope_table", _check(positions, "rope.positions", torch.int32, (n,)), n, int(rotated_dims), float(theta),
         _check(out, "rope.table", torch.float32, (n, rotated_dims // 2, 2)), stream_handle())
    return out


def rope_table_ladder(positions, rotated_dims, inv_freq, out, magnitude: float = 1.0):
    """``rope_table`` from frequencies of the caller's own: ``out[n, rotated_dims / 2, 2]`` = ``magnitude`` *
    (cos, sin)(position * inv_freq[i]); ``inv_freq``: float64 ``[rotated_dims / 2]`` on the device."""
    n = positions.shape[0]
    call("fl_rope_table_ladder", _check(positions, "rope.positions", torch.int32, (n,)), n, int(rotated_dims),
         _check(inv_freq, "rope.inv_freq", torch.float64, (rotated_dims // 2,)), float(magnitude),
         _check(out, "rope.table", torch.float32, (n, rotated_dims // 2, 2)), stream_handle())
    return out


def rope_kv_write(qkv, positions, tok_seq, block_table, q_out, cache: PagedLayerCache, n_heads,
                  rotated_dims, theta, write_cache=True, table=None, paired=False, parts: int = 1):
    """Rotate q and k, store q and the cache rows.  ``table``: the step's ``rope_table`` (else the
    angles are computed here); ``paired``: the projection's rows come in the order of
    ``rotary_paired_rows``.  With ``parts`` > 1 ``qkv`` is ``[parts, n, ld]``: partial sums of a
    product that split K, added here."""
    if parts > 1 or qkv.dim() == 3:
        if qkv.dim() != 3 or qkv.shape[0] != parts or not qkv.is_contiguous():
            raise KernelError(f"rope_kv_write: {parts} parts want a contiguous [{parts}, n, ld] tensor")
        part_stride = qkv.shape[1] * qkv.shape[2]
        n, ld = qkv.shape[1:]
    else:
        part_stride = 0
        n, ld = qkv.shape
    nkv, hd = cache.n_kv_heads, cache.head_dim
    if ld != (n_heads + 2 * nkv) * hd:
        raise KernelError(f"rope_kv_write: row of {ld} values, expected {(n_heads + 2 * nkv) * hd}")
    call("fl_rope_kv_write", _check(qkv, "rope.qkv"), dtype_code(qkv.dtype), ld,
         _check(positions, "rope.positions", torch.int32, (n,)),
         _check(tok_seq, "rope.tok_seq", torch.int32, (n,)),
         _check(block_table, "rope.block_table", torch.int32, (None, None)), block_table.shape[1],
         _check(q_out, "rope.q_out", cache.pool.dtype, (n, n_heads * hd)),
         _check(cache.pool, "rope.cache"), dtype_code(cache.pool.dtype), n, n_heads, nkv, hd,
         cache.page_size, cache.n_pages, int(rotated_dims), float(theta), int(bool(write_cache)),
         _check(table, "rope.table", torch.float32, (n, rotated_dims // 2, 2)) if table is not None and rotated_dims else None,
         int(bool(paired)), int(parts), int(part_stride), stream_handle())
    return q_out


def attn_plain(q, out, cache: PagedLayerCache, positions, tok_seq, block_table, n_heads, scale, window, softcap: float = 0.0):
    """``softcap`` > 0: scores are capped, ``softcap * tanh(score / softcap)``, before the softmax."""
    n = q.shape[0]
    hd = cache.head_dim
    dt = cache.pool.dtype
    call("fl_attn_plain_capped" if softcap else "fl_attn_plain", _check(q, "attn.q", dt, (n, n_heads * hd)),
         _check(out, "attn.out", dt, (n, n_heads * hd)), _check(cache.pool, "attn.cache"),
         dtype_code(dt), _check(positions, "attn.positions", torch.int32, (n,)),
         _check(tok_seq, "attn.tok_seq", torch.int32, (n,)),
         _check(block_table, "attn.block_table", torch.int32, (None, None)), block_table.shape[1],
         n, n_heads, cache.n_kv_heads, hd, cache.page_size, cache.n_pages, float(scale), int(window),
         *((float(softcap),) if softcap else ()), stream_handle())
    return out


def attention_max_head_dim() -> int:
    """The largest head size the attention kernels take (a host function: no GPU needed)."""
    from .library import load
    return load().fl_attn_max_head_dim()


def silu_mul(gu, out):
    n, two_i = gu.shape
    I = two_i // 2
    call("fl_silu_mul", _check(gu, "silu_mul.gu"), dtype_code(gu.dtype),
         _check(out, "silu_mul.out", None, (n, I)), dtype_code(out.dtype), n, I, stream_handle())
    return out


def feed_tokens(tokens, ids, src):
    """``tokens[i] = ids[src[i]]`` where ``src[i] >= 0``: ids drawn on the device in the step before."""
    n = tokens.shape[0]
    call("fl_feed_tokens", _check(tokens, "feed.tokens", torch.int32, (n,)), _check(ids, "feed.ids", torch.int32),
         _check(src, "feed.src", torch.int32, (n,)), n, stream_handle())
    return tokens


def argmax(logits, out):
    R, V = logits.shape
    call("fl_argmax", _check(logits, "argmax.logits", torch.float32), _check(out, "argmax.out", torch.int32, (R,)),
         R, V, stream_handle())
    return out


def _counts(counts, V):
    if counts.dtype != torch.int16 or counts.dim() != 2 or counts.shape[1] != V or not counts.is_contiguous() or not counts.is_cuda:
        raise KernelError(f"sample.counts: {counts.dtype} {tuple(counts.shape)}, want int16 [slots, {V}] on the device")
    return counts.data_ptr()


def sample_penalise(logits, counts, slot, repetition, presence, frequency):
    """Repetition, presence and frequency penalties in place on ``logits`` [R, V] for the rows with a
    history (``slot`` >= 0 as a float: row of ``counts``, int16 [slots, V], how often each token was
    generated)."""
    R, V = logits.shape
    f = lambda t, name: _check(t, "sample_penalise." + name, torch.float32, (R,))
    call("fl_sample_penalise", _check(logits, "sample_penalise.logits", torch.float32), R, V, _counts(counts, V),
         f(slot, "slot"), f(repetition, "repetition"), f(presence, "presence"), f(frequency, "frequency"), stream_handle())
    return logits


def sample_bias(logits, rows, tokens, values):
    """``logits[rows[j], tokens[j]] += values[j]`` (all float32 [n]; a pair occurs once)."""
    V, n = logits.shape[1], rows.shape[0]
    f = lambda t, name: _check(t, "sample_bias." + name, torch.float32, (n,))
    call("fl_sample_bias", _check(logits, "sample_bias.logits", torch.float32), V, n, f(rows, "rows"), f(tokens, "tokens"),
         f(values, "values"), stream_handle())
    return logits


def sample_count(counts, slot, ids):
    """The tokens ``ids`` drawn for the rows with a history join it: ``counts[slot[r], ids[r]] += 1``."""
    R, V = ids.shape[0], counts.shape[1]
    call("fl_sample_count", _counts(counts, V), V, R, _check(slot, "sample_count.slot", torch.float32, (R,)),
         _check(ids, "sample_count.ids", torch.int32, (R,)), stream_handle())


def sample_history(counts, slot: int, tokens):
    """Row ``slot`` of ``counts`` is zeroed and the ``tokens`` (int32 [n], may be empty) are counted."""
    V, n = counts.shape[1], tokens.shape[0]
    call("fl_sample_history", _counts(counts, V), V, int(slot),
         _check(tokens, "sample_history.tokens", torch.int32, (n,)) if n else None, n, stream_handle())


def sample_filtered(logits, inv_temp, uniform, top_k, top_p, min_p, out, stash=None):
    """The temperature draw through top-k, top-p and min-p for the rows that ask for them (``top_k``
    >= 1 as a float, 0 < ``top_p`` < 1, ``min_p`` > 0); other rows of ``out`` are not touched.
    ``stash`` (int32 or float32, at least R * V values): scratch that spares a vocabulary beyond 32,768
    the forming of its probabilities in every pass."""
    R, V = logits.shape
    if stash is not None and (stash.numel() < R * V or stash.element_size() != 4 or not stash.is_contiguous()):
        raise KernelError(f"sample_filtered.stash: {stash.numel()} values of {stash.element_size()} bytes, {R * V} of 4 wanted")
    f = lambda t, name: _check(t, "sample_filtered." + name, torch.float32, (R,))
    call("fl_sample_filtered", _check(logits, "sample_filtered.logits", torch.float32), f(inv_temp, "inv_temp"),
         f(uniform, "uniform"), f(top_k, "top_k"), f(top_p, "top_p"), f(min_p, "min_p"),
         _check(out, "sample_filtered.out", torch.int32, (R,)), R, V,
         stash.data_ptr() if stash is not None else None, stream_handle())
    return out


def sample(logits, inv_temp, uniform, out):
    R, V = logits.shape
    call("fl_sample", _check(logits, "sample.logits", torch.float32),
         _check(inv_temp, "sample.inv_temp", torch.float32, (R,)),
         _check(uniform, "sample.uniform", torch.float32, (R,)),
         _check(out, "sample.out", torch.int32, (R,)), R, V, stream_handle())
    return out


# ---------------------------------------------------------------- latent rows, recurrences, routed experts
@dataclass
class LatentLayerCache:
    """The pool of one layer that keeps one row per token: ``pool[n_pages, 2, page_size, width]``, every
    page's rows as they are and, in its second half, transposed (``[width, page_size]``)."""
    pool: torch.Tensor

    @property
    def n_pages(self): return self.pool.shape[0]
    @property
    def page_size(self): return self.pool.shape[2]
    @property
    def width(self): return self.pool.shape[3]


def norm_slice(x, col0, width, weight, eps, out):
    """``out[n, width] = rmsnorm(x[:, col0 : col0 + width]) * weight`` for float32 rows ``x``."""
    n, ld = x.shape
    call("fl_norm_slice", _check(x, "norm_slice.x", torch.float32), ld, int(col0), int(width),
         _check(weight, "norm_slice.weight", torch.float32, (width,)) if weight is not None else None, float(eps),
         _check(out, "norm_slice.out", None, (n, width)), dtype_code(out.dtype), n, None, None, None, 0, 0, 0, stream_handle())
    return out


def norm_slice_to_pages(x, col0, width, weight, eps, cache: LatentLayerCache, positions, tok_seq, block_table):
    """The same norm, stored into the page row of each token's position."""
    n, ld = x.shape
    if cache.width != width:
        raise KernelError(f"norm_slice: rows of {width} values into a pool of rows {cache.width} wide")
    call("fl_norm_slice", _check(x, "norm_slice.x", torch.float32), ld, int(col0), int(width),
         _check(weight, "norm_slice.weight", torch.float32, (width,)) if weight is not None else None, float(eps),
         _check(cache.pool, "norm_slice.pool"), dtype_code(cache.pool.dtype), n,
         _check(positions, "norm_slice.positions", torch.int32, (n,)), _check(tok_seq, "norm_slice.tok_seq", torch.int32, (n,)),
         _check(block_table, "norm_slice.block_table", torch.int32, (None, None)), block_table.shape[1],
         cache.page_size, cache.n_pages, stream_handle())


def heads_matmul(x, w, out, n_heads, transposed, gate=None, gate_col0=0):
    """One small product per head.  ``x`` float32 ``[n, H * K]``; ``w`` ``[H * K, J]`` (``transposed`` false:
    ``out[t, h] = x[t, h] @ w_h``) or ``[H * J, K]`` (true: ``x[t, h] @ w_h.T``); ``out`` ``[n, H * J]``.
    ``gate``: float32 rows whose columns ``gate_col0 + h`` hold a logit per head; the head's output is
    multiplied by its sigmoid."""
    n, HK = x.shape
    H = int(n_heads)
    K = HK // H
    J = out.shape[1] // H
    want = (H * J, K) if transposed else (H * K, J)
    call("fl_heads_matmul", _check(x, "heads_matmul.x", torch.float32, (n, H * K)), HK,
         _check(w, "heads_matmul.w", None, want), dtype_code(w.dtype),
         _check(out, "heads_matmul.out", None, (n, H * J)), dtype_code(out.dtype), n, H, K, J, int(bool(transposed)),
         _check(gate, "heads_matmul.gate", torch.float32, (n, None)) if gate is not None else None,
         gate.shape[1] if gate is not None else 0, int(gate_col0), stream_handle())
    return out


def latent_max_width() -> int:
    from .library import load
    return load().fl_latent_max_width()


def latent_attention(qa, z, cache: LatentLayerCache, positions, tok_seq, block_table, n_heads, scale, window=0):
    """``z[t, h] = sum_j softmax_j(scale * qa[t, h] . c_j) c_j`` over the cached rows of the token's request."""
    n = qa.shape[0]
    R = cache.width
    call("fl_latent_attention", _check(qa, "latent_attention.qa", torch.float32, (n, n_heads * R)),
         _check(z, "latent_attention.z", torch.float32, (n, n_heads * R)), _check(cache.pool, "latent_attention.pool"),
         dtype_code(cache.pool.dtype), _check(positions, "latent_attention.positions", torch.int32, (n,)),
         _check(tok_seq, "latent_attention.tok_seq", torch.int32, (n,)),
         _check(block_table, "latent_attention.block_table", torch.int32, (None, None)), block_table.shape[1],
         n, int(n_heads), R, cache.page_size, cache.n_pages, float(scale), int(window), stream_handle())
    return z


def mlstm_max_dim() -> int:
    from .library import load
    return load().fl_mlstm_max_dim()


def mlstm_state_floats(dim: int, vdim: int) -> int:
    from .library import load
    import ctypes
    lib = load()
    lib.fl_mlstm_state_floats.restype = ctypes.c_long
    lib.fl_mlstm_state_floats.argtypes = [ctypes.c_int, ctypes.c_int]
    return int(lib.fl_mlstm_state_floats(int(dim), int(vdim)))


def mlstm_scan(proj, cols, bias_i, bias_f, cap, q_scale, state, seq_q_start, seq_q_len, seq_slots, out, factors, n_heads, dim, vdim):
    """The recurrence over the step's tokens, request by request, from and into ``state``
    ``[slots, heads, mlstm_state_floats]``.  ``proj``: float32 rows with q, k, v and the two gates'
    pre-activations at the columns ``cols = (q, k, v, i, f)``; ``out`` float32 ``[n, heads * vdim]``; ``factors``
    float32 ``[n, heads * 3]``: room for the three factors per token and head that the gates' kernel leaves."""
    n, ld = proj.shape
    S = seq_q_start.shape[0]
    rec = mlstm_state_floats(dim, vdim)
    if state.dim() != 3 or state.shape[1] != n_heads or state.shape[2] != rec:
        raise KernelError(f"mlstm_scan.state: shape {tuple(state.shape)}, expected [slots, {n_heads}, {rec}]")
    call("fl_mlstm_scan", _check(proj, "mlstm_scan.proj", torch.float32), ld, *(int(c) for c in cols),
         _check(bias_i, "mlstm_scan.bias_i", torch.float32, (n_heads,)) if bias_i is not None else None,
         _check(bias_f, "mlstm_scan.bias_f", torch.float32, (n_heads,)) if bias_f is not None else None,
         float(cap), float(q_scale), _check(state, "mlstm_scan.state", torch.float32),
         _check(seq_q_start, "mlstm_scan.seq_q_start", torch.int32, (S,)), _check(seq_q_len, "mlstm_scan.seq_q_len", torch.int32, (S,)),
         _check(seq_slots, "mlstm_scan.seq_slots", torch.int32, (S,)),
         _check(out, "mlstm_scan.out", torch.float32, (n, n_heads * vdim)),
         _check(factors, "mlstm_scan.factors", torch.float32, (n, n_heads * 3)), S, int(n_heads), int(dim), int(vdim), stream_handle())
    return out


def headnorm_gate(x, weight, gate, gate_col0, out, n_heads, eps, gate_kind: str = "sigmoid"):
    """Every head's slice of ``x`` (float32 ``[n, H * Dv]``) divided by its root mean square, times ``weight``
    ``[H * Dv]``, times the sigmoid (or, ``gate_kind`` "silu", the silu) of ``gate[:, gate_col0 : gate_col0 + H * Dv]``."""
    n, HD = x.shape
    Dv = HD // n_heads
    call("fl_headnorm_gate", _check(x, "headnorm_gate.x", torch.float32),
         _check(weight, "headnorm_gate.weight", torch.float32, (HD,)) if weight is not None else None,
         _check(gate, "headnorm_gate.gate", torch.float32, (n, None)) if gate is not None else None,
         gate.shape[1] if gate is not None else 0, int(gate_col0), _check(out, "headnorm_gate.out", None, (n, HD)),
         dtype_code(out.dtype), n, int(n_heads), Dv, float(eps), {"sigmoid": 1, "silu": 2}[gate_kind], stream_handle())
    return out


ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu2": 3}


def activation(x, out, kind: str, bias=None):
    """``out = act(x (+ bias))`` for float32 ``x``: ``gelu`` (with the error function), ``gelu_tanh``, ``silu``,
    ``relu2`` (the square of relu); ``bias``: float32, one value per column."""
    if x.shape != out.shape:
        raise KernelError(f"activation: shapes {tuple(x.shape)} and {tuple(out.shape)} differ")
    if bias is not None:
        n, F = x.shape
        call("fl_bias_activation", _check(x, "activation.x", torch.float32), _check(bias, "activation.bias", torch.float32, (F,)),
             _check(out, "activation.out"), dtype_code(out.dtype), n, F, ACTIVATIONS[kind], stream_handle())
        return out
    call("fl_activation", _check(x, "activation.x", torch.float32), _check(out, "activation.out"), dtype_code(out.dtype),
         x.numel(), ACTIVATIONS[kind], stream_handle())
    return out


def moe_tile_rows() -> int:
    from .library import load
    return load().fl_moe_tile_rows()


def moe_max_tiles(n_pairs: int, n_experts: int) -> int:
    """Upper bound of the row tiles of ``n_pairs`` (token, expert) pairs spread over ``n_experts``."""
    return n_pairs // moe_tile_rows() + min(n_pairs, n_experts)


ROUTER_SCORINGS = {"sigmoid": 0, "softmax": 1, "softmax_chosen": 2, "softmax_grouped": 3}     # (the last has a launch function of its own)


def moe_route(logits, col0, n_experts, top, place, src_row, src_scale, pair_w, tiles, scoring="sigmoid", renormalise=False):
    n, ld = logits.shape
    P_ = n * top
    call("fl_moe_route", _check(logits, "moe_route.logits", torch.float32), ld, int(col0), n, int(n_experts), int(top),
         ROUTER_SCORINGS[scoring], int(bool(renormalise)),
         _check(place, "moe_route.place", torch.int32, (P_,)), _check(src_row, "moe_route.src_row", torch.int32, (P_,)),
         _check(src_scale, "moe_route.src_scale", torch.float32, (P_,)), _check(pair_w, "moe_route.pair_w", torch.float32, (P_,)),
         _check(tiles, "moe_route.tiles", torch.int32, (None, 4)), tiles.shape[0], stream_handle())


def gemm_few(x, w, out):
    """``out[m, f] = sum_k x[m, k] w[f, k]`` (float32 ``out``) for a handful of features: one wave per output."""
    M, K = x.shape
    N = w.shape[0]
    call("fl_gemm_few", _check(x, "gemm_few.x", w.dtype, (M, K)), _check(w, "gemm_few.w", None, (N, K)),
         _check(out, "gemm_few.out", torch.float32, (M, N)), dtype_code(x.dtype), M, N, K, stream_handle())
    return out


def moe_gemm(x, w, out, tiles, src_row=None, src_scale=None, matrix_cores=False):
    """``out[p] = (src_scale[p] * x[src_row[p]]) @ w[e].T`` for the sorted places ``p`` of every tile, ``e`` the
    tile's expert; ``w`` ``[E, N, K]``; without ``src_row`` the rows of ``x`` are the places themselves.
    ``matrix_cores``: the bfloat16 kernel on the matrix cores where it takes the sizes."""
    E, N, K = w.shape
    P_ = out.shape[0]
    if matrix_cores and w.dtype == torch.bfloat16:
        from .library import load
        if load().fl_moe_gemm_mfma_takes(N, K):
            call("fl_moe_gemm_mfma", _check(x, "moe_gemm.x", w.dtype, (None, K)),
                 _check(src_row, "moe_gemm.src_row", torch.int32, (P_,)) if src_row is not None else None,
                 _check(src_scale, "moe_gemm.src_scale", torch.float32, (P_,)) if src_scale is not None else None,
                 _check(w, "moe_gemm.w"), _check(out, "moe_gemm.out", torch.float32, (P_, N)),
                 _check(tiles, "moe_gemm.tiles", torch.int32, (None, 4)), tiles.shape[0], P_, N, K, stream_handle())
            return out
    call("fl_moe_gemm", _check(x, "moe_gemm.x", w.dtype, (None, K)), dtype_code(w.dtype),
         _check(src_row, "moe_gemm.src_row", torch.int32, (P_,)) if src_row is not None else None,
         _check(src_scale, "moe_gemm.src_scale", torch.float32, (P_,)) if src_scale is not None else None,
         _check(w, "moe_gemm.w"), _check(out, "moe_gemm.out", torch.float32, (P_, N)),
         _check(tiles, "moe_gemm.tiles", torch.int32, (None, 4)), tiles.shape[0], N, K, stream_handle())
    return out


def moe_combine(y, place, top, delta, shared=None, gate=None, gate_col=0):
    n, W = delta.shape
    call("fl_moe_combine", _check(y, "moe_combine.y", torch.float32, (n * top, W)),
         _check(place, "moe_combine.place", torch.int32, (n * top,)), int(top),
         _check(shared, "moe_combine.shared", torch.float32, (n, W)) if shared is not None else None,
         _check(gate, "moe_combine.gate", torch.float32, (n, None)) if gate is not None else None,
         gate.shape[1] if gate is not None else 0, int(gate_col),
         _check(delta, "moe_combine.delta", torch.float32), n, W, stream_handle())
    return delta


def concat_cast(a, b, out):
    """``out = [a ; b]`` (two float32 ``[n, W]`` side by side) in ``out``'s dtype."""
    n, W = a.shape
    call("fl_concat_cast", _check(a, "concat.a", torch.float32), _check(b, "concat.b", torch.float32, (n, W)),
         _check(out, "concat.out", None, (n, 2 * W)), dtype_code(out.dtype), n, W, stream_handle())
    return out


def add_rowvec(x, v):
    """``x[r] += v`` for every row of the float32 ``x``."""
    n, W = x.shape
    call("fl_add_rowvec", _check(x, "add_rowvec.x", torch.float32), _check(v, "add_rowvec.v", torch.float32, (W,)), n, W,
         stream_handle())
    return x


# ---------------------------------------------------------------- norms without statistics, gated attention, linear recurrences
def dyt(x, alpha, weight, bias, out, delta=None, store_sum=False, rows=None):
    """``out = tanh(alpha * (x (+ delta))) * weight + bias`` (``alpha`` a float32 scalar on the device);
    ``store_sum`` and ``rows`` as for ``rmsnorm``."""
    n, H = x.shape
    px = _check(x, "dyt.x", torch.float32, (n, H))
    pd = _check(delta, "dyt.delta", torch.float32, (n, H)) if delta is not None else None
    pr = _check(rows, "dyt.rows", torch.int32) if rows is not None else None
    n_out = rows.shape[0] if rows is not None else n
    if alpha.numel() != 1:
        raise KernelError(f"dyt.alpha: {alpha.numel()} values, one wanted")
    call("fl_dyt", px, pd, px if store_sum and delta is not None else None, pr, _check(alpha, "dyt.alpha", torch.float32),
         _check(weight, "dyt.weight", torch.float32, (H,)), _check(bias, "dyt.bias", torch.float32, (H,)) if bias is not None else None,
         _check(out, "dyt.out", None, (n_out, H)), dtype_code(out.dtype), n_out, H, stream_handle())
    return out


def embed_scaled(table, tokens, out, scale: float):
    V, H = table.shape
    n = tokens.shape[0]
    call("fl_embed_scaled", _check(table, "embed.table"), dtype_code(table.dtype), _check(tokens, "embed.tokens", torch.int32, (n,)),
         _check(out, "embed.out", torch.float32, (n, H)), n, H, V, float(scale), stream_handle())
    return out


def gated_act(gu, out, kind: str):
    """``out[r, i] = act(gu[r, i]) * gu[r, I + i]`` for float32 ``gu`` ``[n, 2 I]``."""
    n, two_i = gu.shape
    I = two_i // 2
    call("fl_gated_act", _check(gu, "gated_act.gu", torch.float32), _check(out, "gated_act.out", None, (n, I)), dtype_code(out.dtype),
         n, I, ACTIVATIONS[kind], stream_handle())
    return out


def norm_mix(a, weight_a, factor_a, b, weight_b, factor_b, out, eps):
    """``out = factor_a * rmsnorm(a) * weight_a + factor_b * rmsnorm(b) * weight_b`` row by row, all float32."""
    n, H = a.shape
    call("fl_norm_mix", _check(a, "norm_mix.a", torch.float32), _check(weight_a, "norm_mix.weight_a", torch.float32, (H,)), float(factor_a),
         _check(b, "norm_mix.b", torch.float32, (n, H)), _check(weight_b, "norm_mix.weight_b", torch.float32, (H,)), float(factor_b),
         _check(out, "norm_mix.out", torch.float32, (n, H)), n, H, float(eps), stream_handle())
    return out


HEAD_GATES = {None: 0, "sigmoid": 1, "silu": 2}


def heads_gate(x, head_stride, gate, gate_col0, kind, out, n_heads):
    """``out[t, h, j] = x[t, h, j] * g(gate[t, gate_col0 + h * Dv + j])`` for ``j < Dv``; the heads of ``x`` are
    ``head_stride`` wide (padded), those of ``out`` ``Dv``.  ``kind``: ``None``, ``sigmoid`` or ``silu``."""
    n = x.shape[0]
    Dv = out.shape[1] // n_heads
    call("fl_heads_gate", _check(x, "heads_gate.x", out.dtype, (n, n_heads * head_stride)), dtype_code(x.dtype), int(head_stride),
         _check(gate, "heads_gate.gate", torch.float32, (n, None)) if gate is not None else None,
         gate.shape[1] if gate is not None else 0, int(gate_col0), HEAD_GATES[kind if gate is not None else None],
         _check(out, "heads_gate.out", None, (n, n_heads * Dv)), n, int(n_heads), Dv, stream_handle())
    return out


def qkv_prepare(proj, cols, positions, tok_seq, block_table, q_out, cache: PagedLayerCache, n_heads, dim, vdim, rotated_dims,
                interleaved, table, q_gain, k_gain, head_norm, eps, v_first=None, value_mix: int = 0, mix=None, write_cache=True,
                row_scales=None, q_head_gain=None, k_head_gain=None, bias=None):
    """From the float32 rows of a joined projection (q, k, v at the columns ``cols``) to the rotated, normed
    queries in ``q_out`` and the token's keys and values in the cache, heads stored ``cache.head_dim`` wide.
    ``q_gain`` / ``k_gain``: gains of a norm over the whole projection of q and of k (before rotation);
    ``head_norm``: every head divided by its root mean square after rotation, times ``q_head_gain`` / ``k_head_gain``
    (float32 ``[dim]``, one gain per head dim that all heads share) where given; ``bias``: float32, one value per column of
    ``proj``, added to the projection as it is read (the projections' biases); ``value_mix``: 1 keeps the
    values in ``v_first``, 2 blends them with it by the device scalar ``mix``; ``row_scales``: float32 ``[n, 2]`` of
    scratch for the norm over the projection (a step of many tokens forms its sums in a kernel of their own)."""
    n, ld = proj.shape
    nkv, hdp = cache.n_kv_heads, cache.head_dim
    dt = cache.pool.dtype
    half = rotated_dims // 2
    if cols[1] < 0 and write_cache:
        raise KernelError("qkv_prepare: a projection of queries alone (no key columns) writes no cache")
    call("fl_qkv_prepare", _check(proj, "qkv_prepare.proj", torch.float32), ld, *(int(c) for c in cols),
         _check(positions, "qkv_prepare.positions", torch.int32, (n,)), _check(tok_seq, "qkv_prepare.tok_seq", torch.int32, (n,)),
         _check(block_table, "qkv_prepare.block_table", torch.int32, (None, None)), block_table.shape[1],
         _check(q_out, "qkv_prepare.q_out", dt, (n, n_heads * hdp)), _check(cache.pool, "qkv_prepare.cache"), dtype_code(dt),
         n, int(n_heads), nkv, int(dim), int(vdim), hdp, cache.page_size, cache.n_pages, int(rotated_dims), int(bool(interleaved)),
         _check(table, "qkv_prepare.table", torch.float32, (n, half, 2)) if rotated_dims else None,
         _check(q_gain, "qkv_prepare.q_gain", torch.float32, (n_heads * dim,)) if q_gain is not None else None,
         _check(k_gain, "qkv_prepare.k_gain", torch.float32, (nkv * dim,)) if k_gain is not None else None,
         int(bool(head_norm)),
         _check(q_head_gain, "qkv_prepare.q_head_gain", torch.float32, (dim,)) if q_head_gain is not None else None,
         _check(k_head_gain, "qkv_prepare.k_head_gain", torch.float32, (dim,)) if k_head_gain is not None else None, float(eps),
         _check(v_first, "qkv_prepare.v_first", torch.float32, (n, nkv * vdim)) if v_first is not None else None, int(value_mix),
         _check(mix, "qkv_prepare.mix", torch.float32) if mix is not None else None, int(bool(write_cache)),
         _check(row_scales, "qkv_prepare.row_scales", torch.float32, (n, 2)) if row_scales is not None else None,
         _check(bias, "qkv_prepare.bias", torch.float32, (ld,)) if bias is not None else None, stream_handle())
    return q_out


def linear_scan_max_dim() -> int:
    from .library import load
    return load().fl_linear_scan_max_dim()


def conv_max_taps() -> int:
    from .library import load
    return load().fl_conv_max_taps()


def linear_scan(q, k, v, state, seq_q_start, seq_q_len, seq_slots, out, n_heads, n_qk_heads, dim, vdim,
                head_decay=None, token_gates=None, channel_decay: bool = False, key_decay=None):
    """The recurrence S <- g S + k u^T, o = S^T q over the step's tokens, request by request, from and into
    the first ``heads * dim * vdim`` floats of every slot's record in ``state`` ``[slots, floats]``.
    ``q``, ``k`` float32 ``[n, n_qk_heads * dim]`` (views of wider rows are taken with their row stride),
    ``v`` ``[n, n_heads * vdim]``.  ``head_decay`` float32 ``[heads]``: a fixed g per head and u = v;
    ``token_gates`` float32 ``[n, 2 * heads]`` (g, then beta): the delta rule, u = beta (v - S^T k).
    ``channel_decay``: ``k`` holds a forget gate f per token, head and key dim, S <- diag(f) S + (1 - f) v^T.
    ``key_decay`` float32 ``[n, heads * dim]`` beside ``token_gates``: the delta rule with a decay per token, head and
    key dim, S <- diag(g) S before the correction (the decays of ``token_gates`` are then not read)."""
    n = out.shape[0]
    S = seq_q_start.shape[0]
    if state.dim() != 2 or not state.is_contiguous():
        raise KernelError(f"linear_scan.state: shape {tuple(state.shape)}, expected [slots, floats]")

    def rows(t, name, width):
        if t.dtype != torch.float32 or not t.is_cuda or t.dim() != 2 or t.shape != (n, width) or t.stride(1) != 1:
            raise KernelError(f"linear_scan.{name}: {t.dtype} {tuple(t.shape)}, want float32 [{n}, {width}] with unit stride")
        return t.data_ptr(), t.stride(0)
    (pq, ldq), (pk, ldk), (pv, ldv) = rows(q, "q", n_qk_heads * dim), rows(k, "k", n_qk_heads * dim), rows(v, "v", n_heads * vdim)
    if channel_decay:
        if head_decay is not None or token_gates is not None or n_heads != n_qk_heads:
            raise KernelError("linear_scan: forget gates per key dim come alone, one set per head")
        call("fl_linear_scan_channel", pq, ldq, pk, ldk, pv, ldv, _check(state, "linear_scan.state", torch.float32), state.shape[1],
             _check(seq_q_start, "linear_scan.seq_q_start", torch.int32, (S,)), _check(seq_q_len, "linear_scan.seq_q_len", torch.int32, (S,)),
             _check(seq_slots, "linear_scan.seq_slots", torch.int32, (S,)), _check(out, "linear_scan.out", torch.float32, (n, n_heads * vdim)),
             S, int(n_heads), int(dim), int(vdim), stream_handle())
        return out
    if key_decay is not None:
        if token_gates is None or head_decay is not None:
            raise KernelError("linear_scan: decays per key dim under the delta rule come with the gates per token (their write strengths)")
        pg = _check(token_gates, "linear_scan.gates", torch.float32, (n, 2 * n_heads))
        call("fl_linear_scan_delta_channel", pq, ldq, pk, ldk, pv, ldv,
             _check(key_decay, "linear_scan.key_decay", torch.float32, (n, n_heads * dim)), n_heads * dim, pg + 4 * n_heads, 2 * n_heads,
             _check(state, "linear_scan.state", torch.float32), state.shape[1],
             _check(seq_q_start, "linear_scan.seq_q_start", torch.int32, (S,)), _check(seq_q_len, "linear_scan.seq_q_len", torch.int32, (S,)),
             _check(seq_slots, "linear_scan.seq_slots", torch.int32, (S,)), _check(out, "linear_scan.out", torch.float32, (n, n_heads * vdim)),
             S, int(n_heads), int(n_qk_heads), int(dim), int(vdim), stream_handle())
        return out
    if (head_decay is None) == (token_gates is None):
        raise KernelError("linear_scan: a decay per head or gates per token, one of the two")
    pg = _check(token_gates, "linear_scan.gates", torch.float32, (n, 2 * n_heads)) if token_gates is not None else None
    call("fl_linear_scan", pq, ldq, pk, ldk, pv, ldv,
         _check(head_decay, "linear_scan.decay", torch.float32, (n_heads,)) if head_decay is not None else None,
         pg, pg + 4 * n_heads if pg is not None else None, 2 * n_heads if pg is not None else 0,
         _check(state, "linear_scan.state", torch.float32), state.shape[1],
         _check(seq_q_start, "linear_scan.seq_q_start", torch.int32, (S,)), _check(seq_q_len, "linear_scan.seq_q_len", torch.int32, (S,)),
         _check(seq_slots, "linear_scan.seq_slots", torch.int32, (S,)), _check(out, "linear_scan.out", torch.float32, (n, n_heads * vdim)),
         S, int(n_heads), int(n_qk_heads), int(dim), int(vdim), stream_handle())
    return out


def conv_prepare(proj, col0, col_b, col_a, conv_w, a_log, dt_bias, state, conv_at, tok_seq, seq_q_start, seq_q_len, seq_slots,
                 prep, gates, n_qk_heads, n_heads, dim, vdim, taps, q_scale, unit_eps):
    """Short causal convolution + silu over the channels of q, k, v (columns ``col0`` on of the float32 rows
    ``proj``), unit vectors per head of q (times ``q_scale``) and k, and the gates of every (token, head) into
    ``gates`` ``[n, 2 * heads]`` (decay, then write strength).  The inputs of the last ``taps - 1`` tokens of a
    request live at ``conv_at`` floats into its record of ``state`` ``[slots, floats]`` and are moved on."""
    n, ld = proj.shape
    S = seq_q_start.shape[0]
    C = 2 * n_qk_heads * dim + n_heads * vdim
    if state.dim() != 2 or not state.is_contiguous() or state.shape[1] < conv_at + (taps - 1) * C:
        raise KernelError(f"conv_prepare.state: shape {tuple(state.shape)} does not hold {taps - 1} x {C} floats at {conv_at}")
    call("fl_conv_prepare", _check(proj, "conv_prepare.proj", torch.float32), ld, int(col0), int(col_b), int(col_a),
         _check(conv_w, "conv_prepare.conv_w", torch.float32, (C, taps)),
         _check(a_log, "conv_prepare.a_log", torch.float32, (n_heads,)) if a_log is not None else None,       # (None: the decays are formed elsewhere)
         _check(dt_bias, "conv_prepare.dt_bias", torch.float32, (n_heads,)) if a_log is not None else None,
         _check(state, "conv_prepare.state", torch.float32) + 4 * int(conv_at), state.shape[1],
         _check(tok_seq, "conv_prepare.tok_seq", torch.int32, (n,)), _check(seq_q_start, "conv_prepare.seq_q_start", torch.int32, (S,)),
         _check(seq_q_len, "conv_prepare.seq_q_len", torch.int32, (S,)), _check(seq_slots, "conv_prepare.seq_slots", torch.int32, (S,)),
         _check(prep, "conv_prepare.prep", torch.float32, (n, C)), _check(gates, "conv_prepare.gates", torch.float32, (n, 2 * n_heads)),
         n, S, int(n_qk_heads), int(n_heads), int(dim), int(vdim), int(taps), float(q_scale), float(unit_eps), stream_handle())
    return prep


def rotate_scale(proj, col_a, col_b, table, rotated_dims, interleaved, scale_a, scale_b, out_a, out_b, n_heads, dim):
    """Two sets of heads in the float32 rows ``proj`` (at ``col_a`` and ``col_b``) rotated by the step's table
    and multiplied by a factor each, into float32 ``out_a`` and ``out_b`` ``[n, heads * dim]``."""
    n, ld = proj.shape
    call("fl_rotate_scale", _check(proj, "rotate_scale.proj", torch.float32), ld, int(col_a), int(col_b),
         _check(table, "rotate_scale.table", torch.float32, (n, rotated_dims // 2, 2)) if rotated_dims else None,
         int(rotated_dims), int(bool(interleaved)), float(scale_a), float(scale_b),
         _check(out_a, "rotate_scale.out_a", torch.float32, (n, n_heads * dim)),
         _check(out_b, "rotate_scale.out_b", torch.float32, (n, n_heads * dim)), n, int(n_heads), int(dim), stream_handle())


# ---------------------------------------------------------------- layer norm, learned positions, forget gates, mixed heads
def layernorm(x, weight, bias, out, eps, delta=None, store_sum=False, rows=None):
    """``out = layernorm(x (+ delta)) * weight + bias`` (mean and variance over a row); ``store_sum`` and ``rows``
    as for ``rmsnorm``; ``out`` may be ``x`` itself."""
    n, H = x.shape
    px = _check(x, "layernorm.x", torch.float32, (n, H))
    pd = _check(delta, "layernorm.delta", torch.float32, (n, H)) if delta is not None else None
    pr = _check(rows, "layernorm.rows", torch.int32) if rows is not None else None
    n_out = rows.shape[0] if rows is not None else n
    call("fl_layernorm", px, pd, px if store_sum and delta is not None else None, pr,
         _check(weight, "layernorm.weight", torch.float32, (H,)),
         _check(bias, "layernorm.bias", torch.float32, (H,)) if bias is not None else None,
         _check(out, "layernorm.out", None, (n_out, H)), dtype_code(out.dtype), n_out, H, float(eps), stream_handle())
    return out


def layernorm_add(delta, weight, bias, resid, eps, cast=None):
    """``resid += layernorm(delta) * weight + bias``; ``cast`` (optional) receives the new ``resid`` in its dtype."""
    n, H = resid.shape
    call("fl_layernorm_add", _check(delta, "layernorm_add.delta", torch.float32, (n, H)),
         _check(weight, "layernorm_add.weight", torch.float32, (H,)),
         _check(bias, "layernorm_add.bias", torch.float32, (H,)) if bias is not None else None,
         _check(resid, "layernorm_add.resid", torch.float32),
         _check(cast, "layernorm_add.cast", None, (n, H)) if cast is not None else None,
         dtype_code(cast.dtype) if cast is not None else 0, n, H, float(eps), stream_handle())
    return resid


def embed_positions(table, pos_table, tokens, positions, out):
    """``out[t] = table[tokens[t]] + pos_table[positions[t]]`` in float32."""
    V, H = table.shape
    P_ = pos_table.shape[0]
    n = tokens.shape[0]
    call("fl_embed_positions", _check(table, "embed.table"), _check(pos_table, "embed.pos_table", table.dtype, (P_, H)),
         dtype_code(table.dtype), _check(tokens, "embed.tokens", torch.int32, (n,)),
         _check(positions, "embed.positions", torch.int32, (n,)), _check(out, "embed.out", torch.float32, (n, H)),
         n, H, V, P_, stream_handle())
    return out


def cast_rows(x, out):
    """The float32 ``x`` in ``out``'s dtype."""
    if x.shape != out.shape:
        raise KernelError(f"cast_rows: shapes {tuple(x.shape)} and {tuple(out.shape)} differ")
    call("fl_cast_rows", _check(x, "cast_rows.x", torch.float32), _check(out, "cast_rows.out"), dtype_code(out.dtype),
         x.numel(), stream_handle())
    return out


def scale_inplace(x, factor: float):
    call("fl_scale_inplace", _check(x, "scale.x", torch.float32), x.numel(), float(factor), stream_handle())
    return x


def forget_gates(proj, col_q, col_f, bias, lower, q_out, f_out):
    """``q_out = silu(proj[:, col_q:])``, ``f_out = lower + (1 - lower) * sigmoid(proj[:, col_f:] + bias)``, float32
    ``[n, HD]`` each: the read-out vector and the forget gates of a recurrence whose gate is also its key."""
    n, ld = proj.shape
    HD = q_out.shape[1]
    call("fl_forget_gates", _check(proj, "forget_gates.proj", torch.float32), ld, int(col_q), int(col_f),
         _check(bias, "forget_gates.bias", torch.float32, (HD,)) if bias is not None else None,
         _check(lower, "forget_gates.lower", torch.float32, (HD,)) if lower is not None else None,
         _check(q_out, "forget_gates.q", torch.float32, (n, HD)), _check(f_out, "forget_gates.f", torch.float32, (n, HD)),
         n, HD, stream_handle())


def attn_mixed_max_heads(head_dim: int) -> int:
    """How many heads of ``head_dim`` stored values a block of the mixed-heads attention kernel holds."""
    from .library import load
    return load().fl_attn_mixed_max_heads(int(head_dim))


def attn_mixed(q, out, cache: PagedLayerCache, positions, tok_seq, block_table, n_heads, scale, window,
               slopes=None, talk=None, sink=None, part_keys: int = 0, n_parts: int = 1, part_acc=None, part_ml=None,
               keep_first: int = 0, chunk: int = 0):
    """Attention over the paged cache with ``slopes[g] * (i - j)`` taken off the scores, the heads' scores mixed by
    ``talk`` ``[H, H]`` and ``exp(sink[h])`` in the denominator (each optional).  ``part_keys`` > 0: every
    token's keys are dealt out to ``n_parts`` blocks; ``part_acc`` / ``part_ml`` float32 scratch for them.
    The mask: ``window`` newest keys, or (``chunk`` > 0 instead) the keys of the query's own run of ``chunk`` positions
    counted from 0, or all; and always the first ``keep_first`` keys."""
    n = q.shape[0]
    hd = cache.head_dim
    dt = cache.pool.dtype
    f = lambda t, name, shape: _check(t, "attn_mixed." + name, torch.float32, shape) if t is not None else None
    if part_keys:
        if part_acc is None or part_ml is None or part_acc.numel() < n * n_parts * n_heads * hd or part_ml.numel() < n * n_parts * n_heads * 2:
            raise KernelError("attn_mixed: the parts' scratch is missing or too small")
    call("fl_attn_mixed", _check(q, "attn_mixed.q", dt, (n, n_heads * hd)), _check(out, "attn_mixed.out", dt, (n, n_heads * hd)),
         _check(cache.pool, "attn_mixed.cache"), dtype_code(dt), _check(positions, "attn_mixed.positions", torch.int32, (n,)),
         _check(tok_seq, "attn_mixed.tok_seq", torch.int32, (n,)),
         _check(block_table, "attn_mixed.block_table", torch.int32, (None, None)), block_table.shape[1],
         n, int(n_heads), cache.n_kv_heads, hd, cache.page_size, cache.n_pages, float(scale), int(window), int(keep_first), int(chunk),
         f(slopes, "slopes", (n_heads,)), f(talk, "talk", (n_heads, n_heads)), f(sink, "sink", (n_heads,)),
         int(part_keys), int(n_parts), f(part_acc, "part_acc", None), f(part_ml, "part_ml", None), stream_handle())
    return out


def attn_mixed_tiled_fits(n_heads: int, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core form of the mixed-heads attention takes these sizes (bfloat16 caches only)."""
    from .library import load
    return bool(load().fl_attn_mixed_tiled_fits(int(n_heads), int(head_dim), int(page_size)))


def attn_mixed_tiled(q, out, cache: PagedLayerCache, positions, block_table, seq_q_start, seq_q_len, n_tiles, n_heads, scale, window,
                     slopes=None, talk=None, sink=None, part_keys: int = 0, n_parts: int = 1, part_acc=None, part_ml=None,
                     keep_first: int = 0, chunk: int = 0):
    """``attn_mixed`` on the matrix cores: blocks take tiles of 16 rows of one request; ``n_tiles`` is the sum over
    the requests of ceil(rows / 16), ``seq_q_start`` / ``seq_q_len`` the first row and the rows of every request."""
    n = q.shape[0]
    hd = cache.head_dim
    dt = cache.pool.dtype
    if dt != torch.bfloat16:
        raise KernelError("attn_mixed_tiled: bfloat16 caches only")
    S = seq_q_start.shape[0]
    f = lambda t, name, shape: _check(t, "attn_mixed_tiled." + name, torch.float32, shape) if t is not None else None
    if part_keys:
        if part_acc is None or part_ml is None or part_acc.numel() < n * n_parts * n_heads * hd or part_ml.numel() < n * n_parts * n_heads * 2:
            raise KernelError("attn_mixed_tiled: the parts' scratch is missing or too small")
    call("fl_attn_mixed_tiled", _check(q, "attn_mixed_tiled.q", dt, (n, n_heads * hd)), _check(out, "attn_mixed_tiled.out", dt, (n, n_heads * hd)),
         _check(cache.pool, "attn_mixed_tiled.cache"), _check(positions, "attn_mixed_tiled.positions", torch.int32, (n,)),
         _check(block_table, "attn_mixed_tiled.block_table", torch.int32, (None, None)), block_table.shape[1],
         _check(seq_q_start, "attn_mixed_tiled.seq_q_start", torch.int32, (S,)), _check(seq_q_len, "attn_mixed_tiled.seq_q_len", torch.int32, (S,)),
         S, int(n_tiles), n, int(n_heads), cache.n_kv_heads, hd, cache.page_size, cache.n_pages, float(scale), int(window),
         int(keep_first), int(chunk), f(slopes, "slopes", (n_heads,)), f(talk, "talk", (n_heads, n_heads)), f(sink, "sink", (n_heads,)),
         int(part_keys), int(n_parts), f(part_acc, "part_acc", None), f(part_ml, "part_ml", None), stream_handle())
    return out


# ---------------------------------------------------------------- hyper-connections, decays per key dim, routers with groups
def channel_decay(a, col, a_log, dt_bias, out, n_heads, dim):
    """``out[t, h * dim + d] = exp(-exp(a_log[h]) * softplus(a[t, col + h * dim + d] + dt_bias[h * dim + d]))``."""
    n, ld = a.shape
    call("fl_channel_decay", _check(a, "channel_decay.a", torch.float32), ld, int(col),
         _check(a_log, "channel_decay.a_log", torch.float32, (n_heads,)), _check(dt_bias, "channel_decay.dt_bias", torch.float32, (n_heads * dim,)),
         _check(out, "channel_decay.out", torch.float32, (n, n_heads * dim)), n, int(n_heads), int(dim), stream_handle())
    return out


def lowrank_expand(x, col, w, wt, out):
    """``out[t] = w @ x[t, col : col + rank]``: the second factor of a projection of low rank; ``x`` float32 rows (the
    first factor's products, not rounded), ``w`` the factor ``[features, rank]`` as it is stored and ``wt`` the same
    transposed (a step of few tokens reads the one, a larger step the other: the same sums in the same order), ``out`` float32."""
    n, ld = x.shape
    N, R = w.shape
    if wt.shape != (R, N) or wt.dtype != w.dtype:
        raise KernelError(f"lowrank_expand: a factor {tuple(w.shape)} with a transposed copy {tuple(wt.shape)}")
    call("fl_lowrank_expand", _check(x, "lowrank_expand.x", torch.float32), ld, int(col), _check(w, "lowrank_expand.w"), _check(wt, "lowrank_expand.wt"), dtype_code(w.dtype),
         _check(out, "lowrank_expand.out", torch.float32, (n, N)), n, N, R, stream_handle())
    return out


def moe_route_grouped(logits, col0, n_outputs, n_identity, top, correction, n_groups, keep_groups, scale, place, src_row, src_scale,
                      pair_w, tiles):
    """``moe_route`` for a router that scores by a softmax over all its ``n_outputs`` outputs (the last ``n_identity`` of
    them identity experts), chooses by score + ``correction`` inside the ``keep_groups`` best of ``n_groups`` groups of
    neighbours, and weights the chosen by their scores over their sum, times ``scale``."""
    n, ld = logits.shape
    P_ = n * top
    call("fl_moe_route_grouped", _check(logits, "moe_route.logits", torch.float32), ld, int(col0), n, int(n_outputs), int(n_identity), int(top),
         _check(correction, "moe_route.correction", torch.float32, (n_outputs,)) if correction is not None else None,
         int(n_groups), int(keep_groups), float(scale),
         _check(place, "moe_route.place", torch.int32, (P_,)), _check(src_row, "moe_route.src_row", torch.int32, (P_,)),
         _check(src_scale, "moe_route.src_scale", torch.float32, (P_,)), _check(pair_w, "moe_route.pair_w", torch.float32, (P_,)),
         _check(tiles, "moe_route.tiles", torch.int32, (None, 4)), tiles.shape[0], stream_handle())


def moe_identity(x, src_row, src_scale, y, tiles):
    """``y[p] = src_scale[p] * x[src_row[p]]`` for the sorted places of the identity experts' tiles."""
    P_, W = y.shape
    call("fl_moe_identity", _check(x, "moe_identity.x", None, (None, W)), dtype_code(x.dtype),
         _check(src_row, "moe_identity.src_row", torch.int32, (P_,)), _check(src_scale, "moe_identity.src_scale", torch.float32, (P_,)),
         _check(y, "moe_identity.y", torch.float32), _check(tiles, "moe_identity.tiles", torch.int32, (None, 4)), tiles.shape[0], W,
         stream_handle())
    return y


HYPER_MAX_STREAMS = 16     # copies of a residual stream that the kernels of hyper-connections take


def hyper_spread(x, xs, n_streams):
    """``xs[t, s] = x[t]`` for every copy ``s``: the copies of a stream as the embedding leaves it."""
    n, W = x.shape
    call("fl_hyper_spread", _check(x, "hyper_spread.x", torch.float32), _check(xs, "hyper_spread.xs", torch.float32, (n, n_streams * W)),
         n, int(n_streams), W, stream_handle())
    return xs


def hyper_step(xs, n_streams, y=None, mix=None, out_w=None, in_w=None, u_out=None, gain=None, eps=0.0, normed=None, rows=None,
               y_bias=None):
    """One pass over the copies ``xs`` float32 ``[n, S * W]`` of a stream.  With ``y`` (float32 ``[n, W]``, a sublayer's
    output, plus ``y_bias`` float32 ``[W]`` in every row where given): x_t <- sum_s mix[s, t] x_s + out_w[t] y.  With ``in_w``: u = sum_s in_w[s] x_s of the new copies into ``u_out``
    and, with ``gain``, ``normed = u / sqrt(mean(u^2) + eps) * gain``.  ``rows`` (int32) picks the tokens that are read."""
    n, SW = xs.shape
    S = int(n_streams)
    W = SW // S
    f = lambda t, name, shape: _check(t, "hyper_step." + name, torch.float32, shape) if t is not None else None
    n_rows = rows.shape[0] if rows is not None else n
    call("fl_hyper_step", _check(xs, "hyper_step.xs", torch.float32), n, S, W, f(y, "y", (n, W)), f(y_bias, "y_bias", (W,)), f(mix, "mix", (S, S)),
         f(out_w, "out", (S,)), f(in_w, "in", (S,)), _check(rows, "hyper_step.rows", torch.int32) if rows is not None else None, n_rows,
         f(u_out, "u", (n_rows, W)), f(gain, "gain", (W,)), float(eps),
         _check(normed, "hyper_step.normed", None, (n_rows, W)) if normed is not None else None,
         dtype_code(normed.dtype) if normed is not None else 0, stream_handle())


def scaled_sum(a, factor_a, b, factor_b, out):
    """``out = factor_a * a + factor_b * b`` (float32, equal shapes)."""
    if a.shape != b.shape or a.shape != out.shape:
        raise KernelError(f"scaled_sum: shapes {tuple(a.shape)}, {tuple(b.shape)}, {tuple(out.shape)} differ")
    call("fl_scaled_sum", _check(a, "scaled_sum.a", torch.float32), float(factor_a), _check(b, "scaled_sum.b", torch.float32), float(factor_b),
         _check(out, "scaled_sum.out", torch.float32), a.numel(), stream_handle())
    return out


def softcap_inplace(x, cap: float):
    """``x <- cap * tanh(x / cap)`` (float32)."""
    call("fl_softcap_inplace", _check(x, "softcap.x", torch.float32), x.numel(), float(cap), stream_handle())
    return x
