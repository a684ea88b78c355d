"""Two mixers side by side: both read the same normed input, each output is normed over the model width
(root mean square, eps inside the root, a plain gain of its own) and the results are added with a factor
each (a half each: their mean); with ``normed=False`` the outputs are added as they are, each with its factor.
The members are any registered mixers; one of them may keep pages, the others records per slot, which the
joined cache lays side by side."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import MIXERS, JoinedCacheSpec, LayerCache, Mixer, PartSpec, Product, StateSpec, TensorSpec


@MIXERS.register("side_by_side")
class SideBySide(Mixer):
    replayable = True
    graph_safe = True           # as far as it goes itself: its members are asked one by one (``mixers``)

    @property
    def lazy_input(self):
        return all(m.lazy_input for m in self._members.values())

    def __init__(self, hidden_size: int, left: PartSpec, right: PartSpec, eps: float = 0.0, factors=(0.5, 0.5), normed: bool = True):
        self.hidden_size, self.eps, self.normed = hidden_size, float(eps), bool(normed)
        self.factors = (float(factors[0]), float(factors[1]))
        self.left, self.right = MIXERS.create(left), MIXERS.create(right)
        self._members = {"left": self.left, "right": self.right}
        specs = [m.cache_spec() for m in self._members.values()]
        paged = [s for s in specs if s is not None and s.page_group() is not None]
        if len(paged) > 1:
            raise ValueError("side_by_side: at most one member may keep pages")
        states = tuple(s if isinstance(s, StateSpec) else None for s in specs)
        if any(s is not None and s.page_group() is None and not isinstance(s, StateSpec) for s in specs):
            raise ValueError("side_by_side: a member's cache is neither paged nor a record per slot")
        if sum(s is not None for s in states) > 1:
            raise ValueError("side_by_side: at most one member may keep a record per slot")
        self._spec = JoinedCacheSpec(paged[0] if paged else None, states) if any(s is not None for s in specs) else None


    def cache_spec(self):
        return self._spec

    def subparts(self):
        return list(self._members.values())

    def mixers(self):
        """The members: what keeps work lists and signatures per kind of mixer looks inside."""
        return list(self._members.values())

    def signature_group(self):
        return ("side_by_side", self.left.signature_group(), self.right.signature_group())

    def step_signature(self, batch):
        return (self.left.step_signature(batch), self.right.step_signature(batch))

    def tensors(self):
        t = {f"{p}.{name}": spec for p, m in self._members.items() for name, spec in m.tensors().items()}
        if self.normed:
            t["left_out.weight"] = TensorSpec((self.hidden_size,), "vector32")
            t["right_out.weight"] = TensorSpec((self.hidden_size,), "vector32")
        return t

    def bind(self, weights, rt):
        self.rt = rt
        for p, m in self._members.items():
            m.bind({k[len(p) + 1:]: v for k, v in weights.items() if k.startswith(p + ".")}, rt)
        self.gain_left, self.gain_right = weights.get("left_out.weight"), weights.get("right_out.weight")

    def _member_cache(self, cache: LayerCache, index: int):
        """What a member sees: the pages as they are, and its own stretch of the slot's record."""
        spec = self._spec
        own = spec.states[index] if spec is not None else None
        state = None
        if own is not None and cache.state is not None:
            offsets, _ = spec.state_offsets()
            n = 1
            for d in own.shape:
                n *= d
            assert offsets[index] == 0 and cache.state.shape[1] == n      # one record per slot, checked when built
            state = cache.state.view(cache.state.shape[0], *own.shape)
        return LayerCache(kv=cache.kv, group=cache.group, state=state, writes=cache.writes)

    def forward(self, x, step, cache):
        rt, n, W = self.rt, x.shape[0], self.hidden_size
        outs = []
        for index, (name, m) in enumerate(self._members.items()):
            d = m.forward(x, step, self._member_cache(cache, index))
            if isinstance(d, Product):
                d = d.compute(rt, out=rt.buffer("sbs_" + name, n, W, torch.float32))
            outs.append(d)
        delta = rt.buffer("sbs_delta", n, W, torch.float32)
        if self.normed:
            ops.norm_mix(outs[0], self.gain_left, self.factors[0], outs[1], self.gain_right, self.factors[1], delta, self.eps)
        else:
            ops.scaled_sum(outs[0], self.factors[0], outs[1], self.factors[1], delta)
        return delta
