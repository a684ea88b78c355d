"""A feed-forward of routed experts, and the ungated feed-forward with an activation of choice.

Routed: router logits z = W_r h in 32-bit, scores s = sigmoid(z) (or a softmax), the ``top`` largest
are chosen, their scores are the weights (divided by their sum only if ``renormalise``).  An expert
is gated, W_down (silu(W_gate u) * (W_up u)), and its weight multiplies its INPUT, u = w h
(``weight_on="input"``), or its output.  A shared expert of the same form may run for every token and
is added, multiplied by sigmoid(w_sg . h), one number per token.

The choice never leaves the device: a kernel sorts the (token, expert) pairs by expert and cuts them
into row tiles, the two products of all experts run as one launch each over those tiles, and a last
kernel adds each token's experts in rising order of rank.  The router's product is a kernel of its own
(one wave per score: exact products, float sums in a fixed order), whatever the runtime's other products
are; the experts' products run on the matrix cores in bfloat16 and as plain products in 32-bit.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, Product, TensorSpec


@FEED_FORWARDS.register("mlp")
class Mlp(FeedForward):
    """d = W_down act(W_up h (+ b_up)) (+ b_down); ``activation``: ``gelu`` (error function), ``gelu_tanh``, ``silu``
    or ``relu2`` (the square of relu); ``bias``: both products have one."""
    replayable = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu", bias: bool = False):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"mlp: unknown activation '{activation}'; known: {sorted(ops.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation = hidden_size, intermediate_size, activation
        self.has_bias = bool(bias)

    def tensors(self):
        W, F = self.hidden_size, self.intermediate_size
        t = {"up.weight": TensorSpec((F, W)), "down.weight": TensorSpec((W, F))}
        if self.has_bias:
            t.update({"up.bias": TensorSpec((F,), "vector32", init="normal"), "down.bias": TensorSpec((W,), "vector32", init="normal")})
        return t

    def bind(self, weights, rt):
        self.rt = rt
        self.w_up = rt.prepare_weight(weights["up.weight"])
        self.w_down = rt.prepare_weight(weights["down.weight"])
        self.b_up, self.b_down = weights.get("up.bias"), weights.get("down.bias")

    def forward(self, x, step):
        rt, n, F = self.rt, x.shape[0], self.intermediate_size
        pre = rt.buffer("mlp_pre", n, F, torch.float32)
        rt.gemm(x, self.w_up, pre)
        act = rt.buffer("mlp_act", n, F)
        ops.activation(pre, act, self.activation, bias=self.b_up)
        if self.b_down is None:
            return Product(act, self.w_down)
        delta = rt.buffer("mlp_delta", n, self.hidden_size, torch.float32)
        rt.gemm(act, self.w_down, delta)
        return ops.add_rowvec(delta, self.b_down)


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    replayable = True

    def __init__(self, hidden_size: int, n_experts: int, top: int, expert_size: int, shared_size: int | None = None,
                 scoring: str = "sigmoid", renormalise: bool = False, weight_on: str = "input", shared_gate: bool = True,
                 gated: bool = True, activation: str = "silu", router_bias: bool = False, correction: bool = False,
                 n_groups: int = 1, keep_groups: int = 1, n_identity: int = 0, weight_scale: float = 1.0):
        """``scoring``: ``sigmoid``, ``softmax`` (over all experts), ``softmax_chosen`` (over the chosen logits only) or
        ``softmax_grouped``; ``gated=False``: an expert is W_down act(W_up u) with ``activation`` (no gate matrix);
        ``router_bias``: the router's logits have a bias.

        ``softmax_grouped``: scores s = softmax over ALL the router's outputs; the choice goes by s + a learned
        ``correction`` per output (if ``correction``), the weights by s alone; the outputs form ``n_groups`` equal groups of
        neighbours, a group's score is its largest choice score, and only outputs of the ``keep_groups`` best groups can
        be chosen; the weights are the chosen scores over their sum (+ 1e-20) times ``weight_scale``.  The last
        ``n_identity`` outputs of the router are identity experts: they have no matrices and return their input (times
        the weight); the router then has ``n_experts + n_identity`` outputs, and groups are formed over all of them."""
        grouped = scoring == "softmax_grouped"
        if not grouped and (correction or n_groups != 1 or keep_groups != 1 or n_identity or weight_scale != 1.0):
            raise ValueError("routed_experts: correction, groups, identity experts and a weight scale come with scoring 'softmax_grouped'")
        n_outputs = n_experts + int(n_identity)
        if grouped and (n_groups < 1 or n_outputs % n_groups or not 1 <= keep_groups <= n_groups or keep_groups * (n_outputs // n_groups) < top):
            raise ValueError(f"routed_experts: {keep_groups} of {n_groups} groups over {n_outputs} router outputs cannot give {top} choices")
        if grouped and (weight_on != "output" or router_bias):
            raise ValueError("routed_experts: scoring 'softmax_grouped' weights the experts' outputs and has no router bias")
        self.grouped, self.correction, self.n_groups, self.keep_groups = grouped, bool(correction), int(n_groups), int(keep_groups)
        self.n_identity, self.n_outputs, self.weight_scale = int(n_identity), n_outputs, float(weight_scale)
        if weight_on not in ("input", "output"):
            raise ValueError(f"routed_experts: weight_on must be 'input' or 'output', got {weight_on!r}")
        if scoring not in ops.ROUTER_SCORINGS:
            raise ValueError(f"routed_experts: scoring must be one of {sorted(ops.ROUTER_SCORINGS)}, got {scoring!r}")
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"routed_experts: unknown activation '{activation}'; known: {sorted(ops.ACTIVATIONS)}")
        if gated and activation != "silu":
            raise ValueError("routed_experts: gated experts take the silu gate")
        self.gated, self.activation, self.router_bias = bool(gated), activation, bool(router_bias)
        self.hidden_size, self.n_experts, self.top = hidden_size, n_experts, top
        self.expert_size, self.shared_size = expert_size, shared_size
        self.scoring, self.renormalise, self.weight_on = scoring, bool(renormalise), weight_on
        self.shared_gate = bool(shared_gate) and shared_size is not None

    def tensors(self):
        W, F = self.hidden_size, self.expert_size
        t = {"router.weight": TensorSpec((self.n_outputs, W))}
        if self.correction:
            t["correction"] = TensorSpec((self.n_outputs,), "vector32", init="normal")
        if self.router_bias:
            t["router.bias"] = TensorSpec((self.n_experts,), "vector32", init="normal")
        for e in range(self.n_experts):
            if self.gated:
                t[f"e{e}.gate.weight"] = TensorSpec((F, W))
            t[f"e{e}.up.weight"] = TensorSpec((F, W))
            t[f"e{e}.down.weight"] = TensorSpec((W, F))
        if self.shared_size is not None:
            Fs = self.shared_size
            t.update({"shared.gate.weight": TensorSpec((Fs, W)), "shared.up.weight": TensorSpec((Fs, W)),
                      "shared.down.weight": TensorSpec((W, Fs))})
            if self.shared_gate:
                t["shared.sg.weight"] = TensorSpec((1, W))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        E = self.n_experts
        # the router's rows and, behind them, the shared expert's gate: one plain product gives all logits
        rows = [weights["router.weight"]] + ([weights["shared.sg.weight"]] if self.shared_gate else [])
        self.w_logits = torch.cat(rows, dim=0).contiguous()
        first = (lambda e: torch.cat([weights[f"e{e}.gate.weight"], weights[f"e{e}.up.weight"]], dim=0)) if self.gated else (lambda e: weights[f"e{e}.up.weight"])
        self.w_gate_up = torch.stack([first(e) for e in range(E)]).contiguous()       # (ungated experts: the up matrices alone)
        self.b_logits = None
        if self.router_bias:
            extra = self.w_logits.shape[0] - E
            self.b_logits = torch.cat([weights["router.bias"], torch.zeros(extra, dtype=torch.float32, device=weights["router.bias"].device)]).contiguous()
        self.w_down = torch.stack([weights[f"e{e}.down.weight"] for e in range(E)]).contiguous()
        self.correction_w = weights.get("correction")
        if self.shared_size is not None:
            self.ws_gate_up = rt.prepare_gate_up(weights["shared.gate.weight"], weights["shared.up.weight"])
            self.ws_down = rt.prepare_weight(weights["shared.down.weight"])

    def forward(self, x, step):
        rt, n = self.rt, x.shape[0]
        W, E, top, F = self.hidden_size, self.n_experts, self.top, self.expert_size
        pairs = n * top
        most = rt.max_batch_tokens * top
        logits = rt.buffer("moe_logits", n, self.w_logits.shape[0], torch.float32)
        ops.gemm_few(x, self.w_logits, logits)
        if self.b_logits is not None:
            ops.add_rowvec(logits, self.b_logits)
        ints = lambda name, rows, cols, cap: rt.buffer(name, rows, cols, torch.int32, max_rows=cap)
        place = ints("moe_place", pairs, 1, most).view(-1)
        src_row = ints("moe_src_row", pairs, 1, most).view(-1)
        src_scale = rt.buffer("moe_src_scale", pairs, 1, torch.float32, max_rows=most).view(-1)
        pair_w = rt.buffer("moe_pair_w", pairs, 1, torch.float32, max_rows=most).view(-1)
        n_tiles = ops.moe_max_tiles(pairs, self.n_outputs)
        tiles = ints("moe_tiles", n_tiles, 4, ops.moe_max_tiles(most, self.n_outputs))
        if self.grouped:
            ops.moe_route_grouped(logits, 0, self.n_outputs, self.n_identity, top, self.correction_w, self.n_groups, self.keep_groups,
                                  self.weight_scale, place, src_row, src_scale, pair_w, tiles)
        else:
            ops.moe_route(logits, 0, E, top, place, src_row, src_scale, pair_w, tiles, self.scoring, self.renormalise)
        on_input = self.weight_on == "input"
        gate_up = rt.buffer("moe_gate_up", pairs, (2 if self.gated else 1) * F, torch.float32, max_rows=most)
        ops.moe_gemm(x, self.w_gate_up, gate_up, tiles, src_row, src_scale if on_input else None, matrix_cores=rt.tuned)
        act = rt.buffer("moe_act", pairs, F, max_rows=most)
        if self.gated:
            ops.silu_mul(gate_up, act)
        else:
            ops.activation(gate_up, act, self.activation)
        y = rt.buffer("moe_y", pairs, W, torch.float32, max_rows=most)
        ops.moe_gemm(act, self.w_down, y, tiles, None, None if on_input else src_scale, matrix_cores=rt.tuned)
        if self.n_identity:
            ops.moe_identity(x, src_row, src_scale, y, tiles)          # (the rows of identity experts: weight * input)
        shared = None
        if self.shared_size is not None:
            sact = rt.buffer("moe_shared_act", n, self.shared_size)
            rt.gemm_swiglu(x, self.ws_gate_up, sact)
            shared = rt.buffer("moe_shared", n, W, torch.float32)
            rt.gemm(sact, self.ws_down, shared)
        delta = rt.buffer("moe_delta", n, W, torch.float32)
        ops.moe_combine(y, place, top, delta, shared=shared, gate=logits if self.shared_gate else None, gate_col=self.n_outputs)
        return delta
