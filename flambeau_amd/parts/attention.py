"""Grouped-query attention over the paged cache.

x -> Q, K, V (one joined matrix product) -> position encoding on Q and K -> K, V stored at
the tokens' positions -> softmax(Q K^T / sqrt(hd)) V over the keys
[max(0, p - window + 1), p] of the same request -> output projection.
(crates/forward/src/core/composites/standard_attn.rs:198-286 projections, :356-397
rotation, :485-500 paged store, :509-533 attention, :1289-1301 output projection; head map
kv_head = q_head / (n_heads / n_kv_heads), crates/kernels-hip/src/kernels/attention_prefill_f16.cu:50-51.)

This step's keys are stored before attention runs, so every query reads all its keys from the
cache and the same code serves whole prompts, portions and single decoded tokens.
"""
from __future__ import annotations

import math

import torch

from ..config.base import ConfigError
from ..kernels import ops
from ..kernels import paged_attention  # noqa: F401  (registers this mixer's kernel set)
from ..kernels import mixed_attention  # noqa: F401  (the kernel set of attention whose heads' scores are mixed)
from .base import MIXERS, POSITION_ENCODINGS, BiasedProduct, Mixer, PagedKVSpec, PartSpec, Product, TensorSpec


@MIXERS.register("paged_gqa_attention")
class PagedGQAAttention(Mixer):
    graph_safe = True
    lazy_input = True
    replayable = True

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: PartSpec, window: int = 0, scale: float | None = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key/value heads")
        if head_dim > ops.attention_max_head_dim():
            # refused when the model is built, not at its first step
            raise ConfigError(f"paged_gqa_attention: 'head_dim' {head_dim} is beyond what the attention kernels take "
                              f"(head sizes up to {ops.attention_max_head_dim()})")
        self.hidden_size = hidden_size
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = POSITION_ENCODINGS.create(position)

    def cache_spec(self):
        return PagedKVSpec(self.n_kv_heads, self.head_dim, self.window)

    def subparts(self):
        return [self.position]

    def signature_group(self):
        return ("paged_gqa_attention", self.n_heads, self.n_kv_heads, self.head_dim, self.window)

    def step_signature(self, batch):
        """Into how many parts the kernels split the keys: all that this mixer decides from the
        contexts' lengths."""
        return self.kernels.signature(batch, self.n_heads, self.n_kv_heads, self.head_dim, self.window)

    def tensors(self):
        H, qw, kvw = self.hidden_size, self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
        return {"q.weight": TensorSpec((qw, H)), "k.weight": TensorSpec((kvw, H)),
                "v.weight": TensorSpec((kvw, H)), "o.weight": TensorSpec((H, qw))}

    @classmethod
    def step_metadata_for(cls, batch, mixers):
        """The work lists the attention kernels of the mixers' runtime want for the batch."""
        return mixers[0].kernels.metadata(batch, mixers) if mixers else {}

    def bind(self, weights, rt):
        self.rt = rt
        self.kernels = rt.kernels("paged_attention")
        w_qkv = torch.cat([weights["q.weight"], weights["k.weight"], weights["v.weight"]], dim=0)
        # Where the runtime's kernels want it, the rows of a rotated projection are put in an order in which the
        # product's own kernel can rotate (8 dims, their 8 partners, ...); the rotation kernel reads
        # that order too.
        rotary = self.position.rotary_parameters()
        order = self.kernels.row_order(self.n_heads, self.n_kv_heads, self.head_dim, rotary[0]) if rotary is not None else None
        self.paired = order is not None
        if self.paired:
            w_qkv = w_qkv[order.to(w_qkv.device)]
        self.w_qkv = rt.prepare_weight(w_qkv.contiguous())
        self.w_o = rt.prepare_weight(weights["o.weight"])
        self.position.bind({}, rt)

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        nh, nkv, hd = self.n_heads, self.n_kv_heads, self.head_dim
        table = step.block_tables[cache.group]
        rotary = self.position.rotary_parameters()
        angles = self.position.rotary_table(rt, step) if rotary is not None and rotary[0] else None
        q = rt.buffer("attn_q", n, nh * hd)
        fused = False
        if self.paired and angles is not None:
            fused = self.kernels.project_rotate_store(x, self.w_qkv, step, table, angles, q, cache.kv, nh, rotary[0], cache.writes)
        if not fused:
            qkv = rt.buffer("attn_qkv", n, (nh + 2 * nkv) * hd, torch.float32)
            rt.gemm(x, self.w_qkv, qkv)
            if rotary is None:
                self.position.apply(qkv, step.positions, nh, nkv, hd)
                rotary = (0, 1.0)
            ops.rope_kv_write(qkv, step.positions, step.tok_seq, table, q, cache.kv, nh, rotary[0], rotary[1],
                              write_cache=cache.writes, table=angles, paired=self.paired)
        out = rt.buffer("attn_out", n, nh * hd)
        self.kernels.attention(q, out, cache.kv, step, table, nh, self.scale, self.window)
        return Product(out, self.w_o)


@MIXERS.register("normed_gqa_attention")
class NormedGQAAttention(PagedGQAAttention):
    """Grouped-query attention over the paged cache with the extras of newer designs, each a parameter:

    * ``value_dim``: values of another size than queries and keys.  The cache keeps heads
      ``max(head_dim, value_dim)`` wide (rounded up to 8), keys and values padded with zeros, so that the
      attention kernels of one head size serve both;
    * ``qk_norm``: ``"projection"``: q (and k) divided by the root mean square over ALL its heads at once,
      times a gain per value, before rotation; ``"head"``: every head of q and k divided by its own root
      mean square after rotation, no gain; ``"head_gain"``: the same with a gain per head dim that all heads of q
      (of k) share; ``None``;
    * ``position``: any encoding that offers a table of cosines and sines and a ``layout`` (``half`` or
      ``interleaved``), or ``none``;
    * ``softcap``: score <- softcap * tanh(score / softcap) before the softmax;
    * ``value_mix``: ``"source"``: this layer's values are kept for later layers of the step;
      ``"blend"``: v <- (1 - lambda) v + lambda v_source with a learned lambda, and the blend is what
      the cache holds.  Both read and write ``StepState.scratch[value_mix_key]``;
    * ``gate``: the heads' outputs times ``sigmoid`` (or ``silu``) of a projection of the mixer's input,
      value by value, before the output projection.

    One joined product gives q, k, v and the gate's logits in 32-bit; norms, rotation and the blend are
    32-bit; this step's keys are stored before attention runs."""
    graph_safe = True
    lazy_input = True        # its input goes to the joined projection only
    replayable = True

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, position: PartSpec,
                 value_dim: int | None = None, window: int = 0, scale: float | None = None, qk_norm: str | None = None,
                 eps: float = 1e-6, softcap: float | None = None, value_mix: str | None = None,
                 value_mix_key: str = "value_mix", gate: str | None = None):
        value_dim = head_dim if value_dim is None else value_dim
        self.value_dim = value_dim
        self.stored_dim = -(-max(head_dim, value_dim) // 8) * 8
        if qk_norm not in (None, "projection", "head", "head_gain"):
            raise ValueError(f"normed_gqa_attention: qk_norm must be 'projection', 'head', 'head_gain' or None, got {qk_norm!r}")
        if value_mix not in (None, "source", "blend"):
            raise ValueError(f"normed_gqa_attention: value_mix must be 'source', 'blend' or None, got {value_mix!r}")
        if gate not in ops.HEAD_GATES:
            raise ValueError(f"normed_gqa_attention: gate must be 'sigmoid', 'silu' or None, got {gate!r}")
        super().__init__(hidden_size, n_heads, n_kv_heads, self.stored_dim, position, window, scale)
        self.head_dim = head_dim                      # (the base class checked the stored size against the kernels)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.qk_norm, self.eps = qk_norm, float(eps)
        self.softcap = float(softcap or 0.0)
        self.value_mix, self.value_mix_key, self.gate = value_mix, value_mix_key, gate

    def cache_spec(self):
        return PagedKVSpec(self.n_kv_heads, self.stored_dim, self.window)

    def signature_group(self):
        return ("normed_gqa_attention", self.n_heads, self.n_kv_heads, self.stored_dim, self.window)

    def step_signature(self, batch):
        return self.kernels.signature(batch, self.n_heads, self.n_kv_heads, self.stored_dim, self.window)

    def tensors(self):
        W, H, G, D, Dv = self.hidden_size, self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim
        t = {"q.weight": TensorSpec((H * D, W)), "k.weight": TensorSpec((G * D, W)), "v.weight": TensorSpec((G * Dv, W)),
             "o.weight": TensorSpec((W, H * Dv))}
        if self.qk_norm == "projection":
            t["q_norm.weight"] = TensorSpec((H * D,), "vector32")
            t["k_norm.weight"] = TensorSpec((G * D,), "vector32")
        elif self.qk_norm == "head_gain":
            t["q_norm.weight"] = TensorSpec((D,), "vector32")
            t["k_norm.weight"] = TensorSpec((D,), "vector32")
        if self.value_mix is not None:
            # (the layer whose values are the source has the scalar too, and does not use it)
            t["value_mix.weight"] = TensorSpec((), "vector32", init=lambda g, shape, device: torch.rand(shape, generator=g, device=device))
        if self.gate is not None:
            t["g.weight"] = TensorSpec((H * Dv, W))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        self.kernels = rt.kernels("paged_attention")
        H, G, D, Dv = self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim
        joined = [weights["q.weight"], weights["k.weight"], weights["v.weight"]] + ([weights["g.weight"]] if self.gate else [])
        self.w_in = rt.prepare_weight(torch.cat(joined, dim=0).contiguous())
        self.cols = (0, H * D, H * D + G * D)
        self.gate_col = H * D + G * D + G * Dv
        self._bind_gains(weights)
        self.mix = weights["value_mix.weight"].reshape(1) if self.value_mix == "blend" else None
        self.w_o = rt.prepare_weight(weights["o.weight"])
        self.position.bind({}, rt)
        self.rotated_dims = int(getattr(self.position, "rotated_dims", 0) or 0)      # (the encoding 'none' has none)
        self.interleaved = getattr(self.position, "layout", "half") == "interleaved"
        if self.rotated_dims and not hasattr(self.position, "rotary_table"):
            raise ValueError("normed_gqa_attention: the position encoding offers no table of cosines and sines")

    def _bind_gains(self, weights):
        """The gains of the norm over the projection (one per value) or of the heads' own norm (one per head dim)."""
        per_dim = self.qk_norm == "head_gain"
        self.q_gain = None if per_dim else weights.get("q_norm.weight")
        self.k_gain = None if per_dim else weights.get("k_norm.weight")
        self.q_head_gain = weights.get("q_norm.weight") if per_dim else None
        self.k_head_gain = weights.get("k_norm.weight") if per_dim else None

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, G, D, Dv, P = self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim, self.stored_dim
        table = step.block_tables[cache.group]
        proj = rt.buffer("nattn_proj", n, self.w_in.rows, torch.float32)
        rt.gemm(x, self.w_in, proj)
        angles = self.position.rotary_table(rt, step) if self.rotated_dims else None
        v_first, mode = None, 0
        if self.value_mix == "source":
            v_first = step.scratch[self.value_mix_key] = rt.buffer("nattn_" + self.value_mix_key, n, G * Dv, torch.float32)
            mode = 1
        elif self.value_mix == "blend":
            v_first = step.scratch.get(self.value_mix_key)
            if v_first is None or v_first.shape != (n, G * Dv):
                raise RuntimeError("normed_gqa_attention: no layer before this one has left values of this shape to blend with")
            mode = 2
        q = rt.buffer("nattn_q", n, H * P)
        ops.qkv_prepare(proj, self.cols, step.positions, step.tok_seq, table, q, cache.kv, H, D, Dv, self.rotated_dims,
                        self.interleaved, angles, self.q_gain, self.k_gain, self.qk_norm in ("head", "head_gain"), self.eps,
                        v_first=v_first, value_mix=mode, mix=self.mix, write_cache=cache.writes,
                        row_scales=rt.buffer("nattn_row_scales", n, 2, torch.float32) if self.qk_norm == "projection" else None,
                        q_head_gain=self.q_head_gain, k_head_gain=self.k_head_gain)
        out = rt.buffer("nattn_out", n, H * P)
        self.kernels.attention(q, out, cache.kv, step, table, H, self.scale, self.window, softcap=self.softcap)
        if self.gate is not None or P != Dv:
            gated = rt.buffer("nattn_gated", n, H * Dv)
            ops.heads_gate(out, P, proj if self.gate is not None else None, self.gate_col, self.gate, gated, H)
            out = gated
        return Product(out, self.w_o)


@MIXERS.register("mixed_heads_attention")
class MixedHeadsAttention(NormedGQAAttention):
    """Grouped-query attention over the paged cache whose scores pass three more steps before the softmax
    weights exist, each a parameter:

    * ``slope_exponent`` e: a distance bias, slope_g * (i - j) is taken off the score of query head g,
      slope_g = 2^(-e (g + 1) / heads) (``None``: no bias);
    * ``head_mix``: the heads' scores are mixed by a learned matrix, score_h <- sum_g T[h, g] score_g, after scale
      and bias and before the window's mask and the softmax;
    * ``sink``: a learned number per head whose exponential joins the softmax's denominator once; it has no key
      and no value;
    * the mask: ``window`` newest keys (the base class's), with ``keep_first`` the first tokens of a sequence stay
      visible to every later query beside the window (at their true positions); ``chunk`` > 0 instead of a window: a
      query sees the earlier keys of its own run of ``chunk`` positions, counted from position 0 of the sequence;
    * ``bias``: the projections of q, k and v have biases; ``out_bias``: the output projection has one;
    * ``values="keys"``: there is no value projection: what the key projection returns for a token (bias included, ahead of
      the keys' norm) is also that token's value; key and value size are then equal.

    ``own_kv=False``: the layer has no key and value projections (nor their norm); its run-order entry reads the
    cache of an earlier entry with equal head counts and sizes.  ``cache_window``: how many of the newest keys the
    cache keeps (0: all); by default the mixer's own ``window``, more where another layer with a wider window
    reads this one's cache.  Norm over the projection, value size and window are the base class's."""
    graph_safe = True
    lazy_input = True
    replayable = True

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int | None = None,
                 window: int = 0, scale: float | None = None, qk_norm: str | None = None, eps: float = 1e-6,
                 slope_exponent: float | None = None, head_mix: bool = False, sink: bool = False, own_kv: bool = True,
                 cache_window: int | None = None, keep_first: int = 0, chunk: int = 0, bias: bool = False, out_bias: bool = False,
                 values: str = "projection"):
        if values not in ("projection", "keys"):
            raise ValueError(f"mixed_heads_attention: values must be 'projection' or 'keys', got {values!r}")
        if values == "keys" and value_dim not in (None, head_dim):
            raise ConfigError(f"mixed_heads_attention: values that are the keys have the keys' size {head_dim}, not {value_dim}")
        if chunk and window:
            raise ConfigError("mixed_heads_attention: a window or chunks, not both")
        if chunk < 0 or keep_first < 0 or (chunk and keep_first):
            raise ConfigError(f"mixed_heads_attention: chunks of {chunk} positions with {keep_first} kept first tokens")
        self.keep_first, self.chunk = int(keep_first), int(chunk)
        self.has_bias, self.has_out_bias, self.values = bool(bias), bool(out_bias), values
        super().__init__(hidden_size, n_heads, n_kv_heads, head_dim, PartSpec("none", {}), value_dim=value_dim, window=window,
                         scale=scale, qk_norm=qk_norm, eps=eps)
        self.slope_exponent = float(slope_exponent) if slope_exponent is not None else None
        self.head_mix, self.sink, self.own_kv = bool(head_mix), bool(sink), bool(own_kv)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        self.cache_chunk = self.chunk if cache_window is None else 0         # (a cache that others read keeps what they ask for)
        if self.cache_window and ((not self.window and not self.chunk) or self.window > self.cache_window or self.chunk > self.cache_window):
            raise ConfigError(f"mixed_heads_attention: a window of {self.window or 'all'} keys over a cache that keeps {self.cache_window}")
        most = ops.attn_mixed_max_heads(self.stored_dim)
        if n_heads > most:
            raise ConfigError(f"mixed_heads_attention: {n_heads} heads of {self.stored_dim} stored values are more than the "
                              f"kernel holds at once ({most})")

    def cache_spec(self):
        return PagedKVSpec(self.n_kv_heads, self.stored_dim, self.cache_window, self.keep_first if self.cache_window else 0, self.cache_chunk)

    def signature_group(self):
        return ("mixed_heads_attention", self.window or self.chunk)

    def step_signature(self, batch):
        return self.kernels.signature(batch, self.window or self.chunk)       # (how far back a row's own run of keys can reach)

    @classmethod
    def step_metadata_for(cls, batch, mixers):
        return {}

    def tensors(self):
        H = self.n_heads
        t = super().tensors()
        if not self.own_kv:
            for name in ("k.weight", "v.weight", "k_norm.weight"):
                t.pop(name, None)
        if self.values == "keys":
            t.pop("v.weight", None)
        if self.has_bias:
            for name in ("q", "k", "v"):
                if name + ".weight" in t:
                    t[name + ".bias"] = TensorSpec((t[name + ".weight"].shape[0],), "vector32", init="normal")
        if self.has_out_bias:
            t["o.bias"] = TensorSpec((self.hidden_size,), "vector32", init="normal")
        if self.head_mix:
            eye = lambda g, shape, device: torch.eye(shape[0], device=device) + 0.3 * torch.randn(shape, generator=g, device=device)
            t["talk"] = TensorSpec((H, H), "vector32", init=eye)
        if self.sink:
            t["sink"] = TensorSpec((H,), "vector32", init="normal")
        return t

    def bind(self, weights, rt):
        self.rt = rt
        self.kernels = rt.kernels("mixed_heads_attention")
        H, G, D, Dv = self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim
        names = ["q"] + ((["k"] if self.values == "keys" else ["k", "v"]) if self.own_kv else [])
        self.w_in = rt.prepare_weight(torch.cat([weights[k + ".weight"] for k in names], dim=0).contiguous())
        self.b_in = torch.cat([weights[k + ".bias"] for k in names]).contiguous() if self.has_bias else None
        # (values that are the keys are read from the keys' columns of the projection, as it leaves the product and its bias)
        self.cols = (0, H * D, H * D if self.values == "keys" else H * D + G * D) if self.own_kv else (0, -1, -1)
        self._bind_gains(weights)
        self.w_o = rt.prepare_weight(weights["o.weight"])
        self.b_o = weights.get("o.bias")
        self.talk, self.sinks = weights.get("talk"), weights.get("sink")
        self.slopes = None
        if self.slope_exponent is not None:
            self.slopes = torch.tensor([2.0 ** (-self.slope_exponent * (g + 1) / H) for g in range(H)], dtype=torch.float32, device=rt.device)
        self.position.bind({}, rt)

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, D, Dv, P = self.n_heads, self.head_dim, self.value_dim, self.stored_dim
        if cache.writes != self.own_kv:
            raise RuntimeError("mixed_heads_attention: a layer with projections of its own writes its cache, one without reads another's")
        table = step.block_tables[cache.group]
        proj = rt.buffer("amix_proj", n, self.w_in.rows, torch.float32)
        rt.gemm(x, self.w_in, proj)
        q = rt.buffer("amix_q", n, H * P)
        ops.qkv_prepare(proj, self.cols, step.positions, step.tok_seq, table, q, cache.kv, H, D, Dv, 0, False, None,
                        self.q_gain, self.k_gain, self.qk_norm in ("head", "head_gain"), self.eps, write_cache=cache.writes,
                        row_scales=rt.buffer("amix_row_scales", n, 2, torch.float32) if self.qk_norm == "projection" else None,
                        q_head_gain=self.q_head_gain, k_head_gain=self.k_head_gain, bias=self.b_in)      # (the biases are added as the projection is read)
        out = rt.buffer("amix_out", n, H * P)
        self.kernels.attention(q, out, cache.kv, step, table, H, self.scale, self.window, self.slopes, self.talk, self.sinks,
                               keep_first=self.keep_first, chunk=self.chunk)
        if P != Dv:
            packed = rt.buffer("amix_packed", n, H * Dv)
            ops.heads_gate(out, P, None, 0, None, packed, H)
            out = packed
        return Product(out, self.w_o) if self.b_o is None else BiasedProduct(out, self.w_o, self.b_o)
