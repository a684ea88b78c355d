"""Mixers that keep a matrix per head instead of keys and values: retention and the gated delta rule.

Both walk S [dim, vdim] per head through the tokens, S <- g S + k u^T, o = S^T q, in 32-bit, with the
state in the request's slot (``StateSpec``), so that a prompt may be cut anywhere.

Retention: g is a constant per head, u = v; q and k are rotated by position, k is multiplied by
dim^(-1/2) afterwards; there is no softmax and no denominator.  Every head's o is divided by its root
mean square, multiplied by silu of a projection of the mixer's input, and projected.

Gated delta rule: q, k and v pass a short causal convolution over time (per channel, silu behind it;
its last taps - 1 inputs are state too); q and k become unit vectors per head, q times dim^(-1/2);
per (token, head) a decay g = exp(-exp(A_log) softplus(W_a h + dt_bias)) and a write strength
beta = sigmoid(W_b h); u = beta (v - S^T k) with the decayed S: the memory is corrected towards v at
the key, not just added to.  Query/key head of head h: h // (heads / qk_heads).  Every head's o is
divided by its root mean square, times a gain shared by the heads, times silu of a projection.
Options: a decay per head AND key dim (``decay="key_dim"``: A_log per head, W_a and dt_bias heads x dim wide,
S <- diag(g) S), the decay's and the output gate's projections as products of two matrices of low rank
(``decay_rank``, ``gate_rank``), and a sigmoid in place of the silu (``gate``).

HGRN2: the forget gate is a vector per head (one value per key dim) and also decides what is written:
S <- diag(f) S + (1 - f) v^T, o = S^T q, with f = l + (1 - l) sigmoid(W_f h + b_f) above a learned lower bound
l, q = silu(W_q h), no key of its own and no other scale.  Every head's o is divided by its root mean square
and multiplied by a gain shared by the heads.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import MIXERS, POSITION_ENCODINGS, Mixer, PartSpec, Product, StateSpec, TensorSpec


@MIXERS.register("retention")
class Retention(Mixer):
    graph_safe = False          # a step run twice advances the state twice
    replayable = True
    lazy_input = True           # its input goes to the joined projection only

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, value_dim: int, decay, position: PartSpec, eps: float,
                 key_scale: float | None = None, gate: str | None = "silu"):
        if head_dim > ops.linear_scan_max_dim():
            raise ConfigError(f"retention: 'dim' {head_dim} is beyond what the kernel takes ({ops.linear_scan_max_dim()})")
        if len(decay) != n_heads:
            raise ConfigError(f"retention: {len(decay)} decays for {n_heads} heads")
        self.hidden_size, self.n_heads, self.head_dim, self.value_dim = hidden_size, n_heads, head_dim, value_dim
        self.decay = tuple(float(d) for d in decay)
        self.eps = float(eps)
        self.key_scale = float(key_scale) if key_scale is not None else head_dim ** -0.5
        self.gate = gate
        self.position = POSITION_ENCODINGS.create(position)

    def cache_spec(self):
        return StateSpec((self.n_heads * self.head_dim * self.value_dim,), torch.float32)

    def subparts(self):
        return [self.position]

    def signature_group(self):
        return ("retention",)

    def step_signature(self, batch):
        return ()

    def tensors(self):
        W, H, D, Dv = self.hidden_size, self.n_heads, self.head_dim, self.value_dim
        t = {"q.weight": TensorSpec((H * D, W)), "k.weight": TensorSpec((H * D, W)), "v.weight": TensorSpec((H * Dv, W)),
             "o.weight": TensorSpec((W, H * Dv))}
        if self.gate is not None:
            t["g.weight"] = TensorSpec((H * Dv, W))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        H, D, Dv = self.n_heads, self.head_dim, self.value_dim
        joined = [weights["q.weight"], weights["k.weight"], weights["v.weight"]] + ([weights["g.weight"]] if self.gate else [])
        self.w_in = rt.prepare_weight(torch.cat(joined, dim=0).contiguous())
        self.col_k, self.col_v, self.col_g = H * D, 2 * H * D, 2 * H * D + H * Dv
        self.decay_dev = torch.tensor(self.decay, dtype=torch.float32, device=rt.device)
        self.w_o = rt.prepare_weight(weights["o.weight"])
        self.position.bind({}, rt)
        self.rotated_dims = int(getattr(self.position, "rotated_dims", 0) or 0)
        self.interleaved = getattr(self.position, "layout", "half") == "interleaved"

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, D, Dv = self.n_heads, self.head_dim, self.value_dim
        proj = rt.buffer("ret_proj", n, self.w_in.rows, torch.float32)
        rt.gemm(x, self.w_in, proj)
        angles = self.position.rotary_table(rt, step) if self.rotated_dims else None
        q = rt.buffer("ret_q", n, H * D, torch.float32)
        k = rt.buffer("ret_k", n, H * D, torch.float32)
        ops.rotate_scale(proj, 0, self.col_k, angles, self.rotated_dims, self.interleaved, 1.0, self.key_scale, q, k, H, D)
        hidden = rt.buffer("ret_hidden", n, H * Dv, torch.float32)
        ops.linear_scan(q, k, proj[:, self.col_v:self.col_v + H * Dv], cache.state, step.seq_q_start, step.seq_q_len,
                        step.seq_slots, hidden, H, H, D, Dv, head_decay=self.decay_dev)
        out = rt.buffer("ret_out", n, H * Dv)
        ops.headnorm_gate(hidden, None, proj if self.gate else None, self.col_g, out, H, self.eps, gate_kind=self.gate or "sigmoid")
        return Product(out, self.w_o)


@MIXERS.register("gated_delta")
class GatedDelta(Mixer):
    graph_safe = False
    replayable = True
    lazy_input = True

    def __init__(self, hidden_size: int, n_heads: int, n_qk_heads: int, head_dim: int, value_dim: int, conv_taps: int, eps: float,
                 unit_eps: float = 1e-6, query_scale: float | None = None, decay: str = "head", decay_rank: int | None = None,
                 gate_rank: int | None = None, gate: str = "silu"):
        if decay not in ("head", "key_dim"):
            raise ValueError(f"gated_delta: decay must be 'head' or 'key_dim', got {decay!r}")
        if gate not in ("silu", "sigmoid"):
            raise ValueError(f"gated_delta: gate must be 'silu' or 'sigmoid', got {gate!r}")
        if decay_rank is not None and decay != "key_dim":
            raise ConfigError("gated_delta: a decay projection of low rank comes with a decay per key dim")
        if any(r is not None and r < 1 for r in (decay_rank, gate_rank)):
            raise ConfigError(f"gated_delta: ranks {decay_rank} and {gate_rank} of the decay's and the gate's projections")
        self.decay, self.decay_rank, self.gate_rank, self.gate = decay, decay_rank, gate_rank, gate
        if head_dim > ops.linear_scan_max_dim():
            raise ConfigError(f"gated_delta: 'dim' {head_dim} is beyond what the kernel takes ({ops.linear_scan_max_dim()})")
        if not 1 <= conv_taps <= ops.conv_max_taps():
            raise ConfigError(f"gated_delta: 'conv' {conv_taps} taps, the kernel takes 1 to {ops.conv_max_taps()}")
        if n_heads % n_qk_heads:
            raise ConfigError(f"gated_delta: {n_heads} heads are not a multiple of {n_qk_heads} query/key heads")
        if n_heads > 256:
            raise ConfigError(f"gated_delta: {n_heads} heads, the kernel takes 256")
        self.hidden_size, self.n_heads, self.n_qk_heads = hidden_size, n_heads, n_qk_heads
        self.head_dim, self.value_dim, self.conv_taps = head_dim, value_dim, conv_taps
        self.eps, self.unit_eps = float(eps), float(unit_eps)
        self.query_scale = float(query_scale) if query_scale is not None else head_dim ** -0.5
        self.channels = 2 * n_qk_heads * head_dim + n_heads * value_dim
        self.conv_at = n_heads * head_dim * value_dim            # where the kept inputs start in a slot's record

    def cache_spec(self):
        return StateSpec((self.conv_at + (self.conv_taps - 1) * self.channels,), torch.float32)

    def signature_group(self):
        return ("gated_delta",)

    def step_signature(self, batch):
        return ()

    def tensors(self):
        W, H, G, D, Dv, K = self.hidden_size, self.n_heads, self.n_qk_heads, self.head_dim, self.value_dim, self.conv_taps
        uniform = lambda lo, hi: (lambda g, shape, device: lo + (hi - lo) * torch.rand(shape, generator=g, device=device))
        A = H * D if self.decay == "key_dim" else H          # decays per token
        t = {"q.weight": TensorSpec((G * D, W)), "k.weight": TensorSpec((G * D, W)), "v.weight": TensorSpec((H * Dv, W)),
             "q_conv.weight": TensorSpec((G * D, K), "vector32", init=uniform(-0.5, 0.5)),
             "k_conv.weight": TensorSpec((G * D, K), "vector32", init=uniform(-0.5, 0.5)),
             "v_conv.weight": TensorSpec((H * Dv, K), "vector32", init=uniform(-0.5, 0.5)),
             "b.weight": TensorSpec((H, W)),
             "A_log": TensorSpec((H,), "vector32", init=uniform(-3.0, 0.5)),
             "dt_bias": TensorSpec((A,), "vector32", init=uniform(-2.0, 1.0)),
             "norm.weight": TensorSpec((Dv,), "vector32"), "o.weight": TensorSpec((W, H * Dv))}
        if self.decay_rank is not None:
            t.update({"a1.weight": TensorSpec((self.decay_rank, W)), "a2.weight": TensorSpec((A, self.decay_rank))})
        else:
            t["a.weight"] = TensorSpec((A, W))
        if self.gate_rank is not None:
            t.update({"g1.weight": TensorSpec((self.gate_rank, W)), "g2.weight": TensorSpec((H * Dv, self.gate_rank))})
        else:
            t["g.weight"] = TensorSpec((H * Dv, W))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        H, G, D, Dv = self.n_heads, self.n_qk_heads, self.head_dim, self.value_dim
        a_name, g_name = ("a1" if self.decay_rank is not None else "a"), ("g1" if self.gate_rank is not None else "g")
        self.w_in = rt.prepare_weight(torch.cat([weights[k + ".weight"] for k in ("q", "k", "v", "b", a_name, g_name)], dim=0).contiguous())
        self.col_b = self.channels
        self.col_a = self.col_b + H
        self.col_g = self.col_a + weights[a_name + ".weight"].shape[0]
        # (second factors, as they are stored and transposed: a step of few tokens reads a feature's own row, a larger one
        # neighbouring features side by side)
        self.w_a2, self.w_g2 = ((weights[k].contiguous(), weights[k].t().contiguous()) if k in weights else None for k in ("a2.weight", "g2.weight"))
        self.conv_w = torch.cat([weights[k + "_conv.weight"] for k in ("q", "k", "v")], dim=0).contiguous()
        self.a_log, self.dt_bias = weights["A_log"], weights["dt_bias"]
        self.norm = weights["norm.weight"].repeat(H).contiguous()          # one gain for every head, laid out heads x vdim
        self.w_o = rt.prepare_weight(weights["o.weight"])

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, G, D, Dv = self.n_heads, self.n_qk_heads, self.head_dim, self.value_dim
        proj = rt.buffer("gd_proj", n, self.w_in.rows, torch.float32)
        rt.gemm(x, self.w_in, proj)
        prep = rt.buffer("gd_prep", n, self.channels, torch.float32)
        gates = rt.buffer("gd_gates", n, 2 * H, torch.float32)
        per_dim = self.decay == "key_dim"
        ops.conv_prepare(proj, 0, self.col_b, self.col_a, self.conv_w, None if per_dim else self.a_log, self.dt_bias, cache.state,
                         self.conv_at, step.tok_seq, step.seq_q_start, step.seq_q_len, step.seq_slots, prep, gates, G, H, D, Dv,
                         self.conv_taps, self.query_scale, self.unit_eps)
        key_decay = None
        if per_dim:
            # the decays per head and key dim: exp(-exp(A_log) softplus(a + dt_bias)), a straight from the joined
            # projection or through the second factor of a projection of low rank (its first factor's products in 32-bit)
            a, col = proj, self.col_a
            if self.w_a2 is not None:
                a, col = ops.lowrank_expand(proj, self.col_a, *self.w_a2, rt.buffer("gd_decay_in", n, H * D, torch.float32)), 0
            key_decay = ops.channel_decay(a, col, self.a_log, self.dt_bias, rt.buffer("gd_decay", n, H * D, torch.float32), H, D)
        hidden = rt.buffer("gd_hidden", n, H * Dv, torch.float32)
        ops.linear_scan(prep[:, :G * D], prep[:, G * D:2 * G * D], prep[:, 2 * G * D:], cache.state, step.seq_q_start,
                        step.seq_q_len, step.seq_slots, hidden, H, G, D, Dv, token_gates=gates, key_decay=key_decay)
        gate_rows, gate_col = proj, self.col_g
        if self.w_g2 is not None:
            gate_rows, gate_col = ops.lowrank_expand(proj, self.col_g, *self.w_g2, rt.buffer("gd_gate_in", n, H * Dv, torch.float32)), 0
        out = rt.buffer("gd_out", n, H * Dv)
        ops.headnorm_gate(hidden, self.norm, gate_rows, gate_col, out, H, self.eps, gate_kind=self.gate)
        return Product(out, self.w_o)


@MIXERS.register("hgrn2")
class Hgrn2(Mixer):
    graph_safe = False          # a step run twice advances the state twice
    replayable = True
    lazy_input = True           # its input goes to the joined projection only

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, value_dim: int, eps: float, lower_bound: bool = True,
                 gate_bias: bool = True):
        if head_dim > ops.linear_scan_max_dim():
            raise ConfigError(f"hgrn2: 'dim' {head_dim} is beyond what the kernel takes ({ops.linear_scan_max_dim()})")
        self.hidden_size, self.n_heads, self.head_dim, self.value_dim = hidden_size, n_heads, head_dim, value_dim
        self.eps = float(eps)
        self.lower_bound, self.gate_bias = bool(lower_bound), bool(gate_bias)

    def cache_spec(self):
        return StateSpec((self.n_heads * self.head_dim * self.value_dim,), torch.float32)

    def signature_group(self):
        return ("hgrn2",)

    def step_signature(self, batch):
        return ()

    def tensors(self):
        W, H, D, Dv = self.hidden_size, self.n_heads, self.head_dim, self.value_dim
        t = {"q.weight": TensorSpec((H * D, W)), "f.weight": TensorSpec((H * D, W)), "v.weight": TensorSpec((H * Dv, W)),
             "norm.weight": TensorSpec((Dv,), "vector32"), "o.weight": TensorSpec((W, H * Dv))}
        if self.gate_bias:
            t["f.bias"] = TensorSpec((H * D,), "vector32", init="normal")
        if self.lower_bound:
            t["lower"] = TensorSpec((H * D,), "vector32", init=lambda g, shape, device: torch.rand(shape, generator=g, device=device))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        H, D, Dv = self.n_heads, self.head_dim, self.value_dim
        self.w_in = rt.prepare_weight(torch.cat([weights["q.weight"], weights["f.weight"], weights["v.weight"]], dim=0).contiguous())
        self.col_f, self.col_v = H * D, 2 * H * D
        self.f_bias, self.lower = weights.get("f.bias"), weights.get("lower")
        self.norm = weights["norm.weight"].repeat(H).contiguous()          # one gain for every head, laid out heads x vdim
        self.w_o = rt.prepare_weight(weights["o.weight"])

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        H, D, Dv = self.n_heads, self.head_dim, self.value_dim
        proj = rt.buffer("hgrn_proj", n, self.w_in.rows, torch.float32)
        rt.gemm(x, self.w_in, proj)
        q = rt.buffer("hgrn_q", n, H * D, torch.float32)
        f = rt.buffer("hgrn_f", n, H * D, torch.float32)
        ops.forget_gates(proj, 0, self.col_f, self.f_bias, self.lower, q, f)
        hidden = rt.buffer("hgrn_hidden", n, H * Dv, torch.float32)
        ops.linear_scan(q, f, proj[:, self.col_v:self.col_v + H * Dv], cache.state, step.seq_q_start, step.seq_q_len,
                        step.seq_slots, hidden, H, H, D, Dv, channel_decay=True)
        out = rt.buffer("hgrn_out", n, H * Dv)
        ops.headnorm_gate(hidden, self.norm, None, 0, out, H, self.eps)
        return Product(out, self.w_o)
