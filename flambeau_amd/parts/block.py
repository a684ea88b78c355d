"""Arrangements of parts in a layer, and the residual stream they advance.

Pre-norm decoder layer: x += Mixer(Norm1(x)); x += FeedForward(Norm2(x))
(crates/forward/README.md:28-40; crates/models/qwen35-v2/src/model.rs:19-50).  The residual
stream is kept in 32-bit.  A delta is not added at once: it stays pending until the next norm,
which adds it, stores the sum and norms it in one kernel
(crates/kernels-hip/src/kernels/rmsnorm_f16_add_residual.cu)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, BiasedProduct, Block, PartSpec, Product, TensorSpec
from .norm import RMSNorm


class ResidualStream:
    def __init__(self, resid, rt):
        self.resid = resid          # float32 [n, hidden]
        self.rt = rt
        self.pending = None         # float32 [n, hidden] not yet added, or a Product not yet computed
        self.cast = None            # the stream in the compute dtype, where a kernel left it beside the float one

    def push(self, delta):
        """``delta``: what a part returned, a tensor or a ``Product``."""
        self.flush()
        self.pending = delta

    def _pending_tensor(self):
        if isinstance(self.pending, Product):
            self.pending = self.pending.compute(self.rt)
        return self.pending

    def flush(self):
        if self._pending_tensor() is not None:
            ops.add_inplace(self.resid, self.pending)
            self.pending = None
            self.cast = None
        return self.resid

    def values(self, name="stream_values"):
        """The stream itself (no norm) as a sublayer's input: in the compute dtype, pending sums added."""
        resid = self.flush()
        if resid.dtype == self.rt.dtype:
            return resid
        if self.cast is None:
            self.cast = ops.cast_rows(resid, self.rt.buffer(name, resid.shape[0], resid.shape[1]))
        return self.cast

    def add_normed(self, norm, delta, name="stream_values"):
        """``stream += norm(delta)``: the norm stands behind the sublayer.  ``delta``: what a part returned, a
        tensor or a ``Product``.  The kernel leaves the new stream in the compute dtype too, for the sublayer
        that reads it next."""
        resid = self.flush()
        if isinstance(delta, Product):
            delta = delta.compute(self.rt)
        cast = None if resid.dtype == self.rt.dtype else self.rt.buffer(name, resid.shape[0], resid.shape[1])
        norm.add_to(resid, delta, cast=cast)
        self.cast = cast

    def normed(self, norm, rows=None, name="normed", lazy=False):
        """The normed stream in the compute dtype, the pending delta added on the way.  With
        ``lazy`` the caller takes what ``Norm.after_product`` returns as well as a tensor."""
        n, H = self.resid.shape
        if lazy and rows is None and type(self.pending) is Product:          # (a product with a bias is computed first)
            fused = norm.after_product(self.rt, self.resid, self.pending)
            if fused is not None:
                self.pending = None
                return fused
        self._pending_tensor()
        if rows is not None:
            out = self.rt.buffer(name + "_rows", rows.shape[0], H)
            norm.forward(self.resid, out, delta=self.pending, rows=rows)
            return out
        out = self.rt.buffer(name, n, H)
        norm.forward(self.resid, out, delta=self.pending, store_sum=True)
        self.pending = None
        return out


class HyperStream(ResidualStream):
    """A residual stream kept in ``n_streams`` copies (hyper-connections).  All copies start as the embedding's
    output.  A sublayer reads a weighted sum of the copies, u = sum_s in[s] x_s, and its output y changes all copies
    at once, x_t <- sum_s mix[s, t] x_s + out[t] y.  What the model's last norm (or anything else that asks for the
    one stream: ``flush``, ``normed``) reads is the sum of the copies, which is then formed in ``resid``.

    A sublayer's output is not written at once: it waits until the next read, and one kernel then writes the new
    copies, forms the next sublayer's input and, where the norm is a root-mean-square norm, norms it."""

    def __init__(self, resid, rt, n_streams: int, ones):
        super().__init__(resid, rt)
        self.n_streams = int(n_streams)
        n, W = resid.shape
        self.copies = ops.hyper_spread(resid, rt.buffer("hyper_copies", n, self.n_streams * W, torch.float32), self.n_streams)
        self.ones = ones                  # float32 [n_streams] of ones, on the device
        self.waiting = None               # (y, mix, out): a sublayer's output that the copies have not taken yet
        self.summed = False               # resid holds the sum of the copies as they are now

    def sublayer_input(self, in_w, norm, name="normed"):
        """norm(sum_s in_w[s] x_s) in the compute dtype; the waiting output of the sublayer before is written on the way."""
        n, W = self.resid.shape
        y, mix, out_w, y_bias = self.waiting if self.waiting is not None else (None, None, None, None)
        u = self.rt.buffer("hyper_u", n, W, torch.float32)
        out = self.rt.buffer(name, n, W)
        if isinstance(norm, RMSNorm):
            ops.hyper_step(self.copies, self.n_streams, y=y, y_bias=y_bias, mix=mix, out_w=out_w, in_w=in_w, u_out=u, gain=norm.weight,
                           eps=norm.eps, normed=out)
        else:
            ops.hyper_step(self.copies, self.n_streams, y=y, y_bias=y_bias, mix=mix, out_w=out_w, in_w=in_w, u_out=u)
            norm.forward(u, out)
        if y is not None:
            self.summed = False
        self.waiting = None
        return out

    def sublayer_output(self, delta, mix, out_w):
        """``delta``: what a part returned, a tensor or a ``Product``."""
        if self.waiting is not None:
            self._write()
        bias = None
        if isinstance(delta, BiasedProduct):             # (its bias rides in the kernel that writes the copies)
            delta, bias = delta.product(self.rt), delta.bias
        elif isinstance(delta, Product):
            delta = delta.compute(self.rt)
        self.waiting = (delta, mix, out_w, bias)

    def _write(self):
        y, mix, out_w, y_bias = self.waiting
        ops.hyper_step(self.copies, self.n_streams, y=y, y_bias=y_bias, mix=mix, out_w=out_w)
        self.waiting, self.summed = None, False

    def flush(self):
        """The one stream: the sum of the copies, in ``resid``."""
        if self.pending is not None:
            raise RuntimeError("a residual stream in several copies takes a sublayer's output with its numbers (sublayer_output), not a plain sum")
        if self.waiting is not None or not self.summed:
            y, mix, out_w, y_bias = self.waiting if self.waiting is not None else (None, None, None, None)
            ops.hyper_step(self.copies, self.n_streams, y=y, y_bias=y_bias, mix=mix, out_w=out_w, in_w=self.ones, u_out=self.resid)
            self.waiting, self.summed, self.cast = None, True, None
        return self.resid

    def push(self, delta):
        raise RuntimeError("a residual stream in several copies takes a sublayer's output with its numbers (sublayer_output)")

    def add_normed(self, norm, delta, name="stream_values"):
        raise RuntimeError("a residual stream in several copies takes a sublayer's output with its numbers (sublayer_output)")

    def normed(self, norm, rows=None, name="normed", lazy=False):
        self.flush()
        return super().normed(norm, rows=rows, name=name, lazy=False)


@BLOCKS.register("hyper_prenorm")
class HyperConnectionBlock(Block):
    """The pre-norm layer over a stream in ``n_streams`` copies (``HyperStream``): for the mixer and then the
    feed-forward, u = sum_s in[s] x_s; y = sublayer(norm(u)); x_t <- sum_s mix[s, t] x_s + out[t] y, with learned
    ``in`` [S], ``out`` [S] and ``mix`` [S, S] (indexed [from, to]) per sublayer.  ``feed_forward`` may be ``None``."""
    replayable = True

    def __init__(self, mixer: PartSpec, feed_forward: PartSpec | None, norm: PartSpec, n_streams: int):
        if n_streams < 1 or n_streams > ops.HYPER_MAX_STREAMS:
            raise ValueError(f"hyper_prenorm: {n_streams} copies of the stream, the kernel takes 1 to {ops.HYPER_MAX_STREAMS}")
        self.n_streams = int(n_streams)
        self.mixer_norm = NORMS.create(norm)
        self.mixer = MIXERS.create(mixer)
        self._parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        self.ffn = None
        if feed_forward is not None:
            self.ffn_norm = NORMS.create(norm)
            self.ffn = FEED_FORWARDS.create(feed_forward)
            self._parts.update({"ffn_norm": self.ffn_norm, "ffn": self.ffn})

    def cache_spec(self):
        return self.mixer.cache_spec()

    def mixers(self):
        return [self.mixer]

    def subparts(self):
        return list(self._parts.values())

    def tensors(self):
        S = self.n_streams
        t = {f"{p}.{name}": spec for p, part in self._parts.items() for name, spec in part.tensors().items()}
        noisy = lambda centre: (lambda g, shape, device: centre(shape, device) + 0.1 * torch.randn(shape, generator=g, device=device))
        for sub in ("hc_mixer", "hc_ffn") if self.ffn is not None else ("hc_mixer",):
            t[f"{sub}.in"] = TensorSpec((S,), "vector32", init=noisy(lambda shape, device: torch.full(shape, 1.0 / S, device=device)))
            t[f"{sub}.out"] = TensorSpec((S,), "vector32", init=noisy(lambda shape, device: torch.ones(shape, device=device)))
            t[f"{sub}.mix"] = TensorSpec((S, S), "vector32", init=noisy(lambda shape, device: torch.eye(shape[0], device=device)))
        return t

    def bind(self, weights, rt):
        self.rt = rt
        for p, part in self._parts.items():
            part.bind({k[len(p) + 1:]: v for k, v in weights.items() if k.startswith(p + ".")}, rt)
        self.hc = {sub: tuple(weights[f"{sub}.{k}"] for k in ("in", "mix", "out")) for sub in ("hc_mixer", "hc_ffn") if f"{sub}.in" in weights}

    def forward(self, stream, step, cache):
        if not isinstance(stream, HyperStream) or stream.n_streams != self.n_streams:
            raise RuntimeError(f"hyper_prenorm: the model's residual stream is not kept in {self.n_streams} copies (ModelSpec.residual_streams)")
        w_in, mix, w_out = self.hc["hc_mixer"]
        stream.sublayer_output(self.mixer.forward(stream.sublayer_input(w_in, self.mixer_norm), step, cache), mix, w_out)
        if self.ffn is not None:
            w_in, mix, w_out = self.hc["hc_ffn"]
            stream.sublayer_output(self.ffn.forward(stream.sublayer_input(w_in, self.ffn_norm), step), mix, w_out)


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    replayable = True

    def __init__(self, mixer: PartSpec, feed_forward: PartSpec | None, norm: PartSpec):
        """``feed_forward`` may be ``None``: a layer of a mixer alone, x += Mixer(Norm1(x)), with no second norm."""
        self.mixer_norm = NORMS.create(norm)
        self.mixer = MIXERS.create(mixer)
        self._parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        self.ffn = None
        if feed_forward is not None:
            self.ffn_norm = NORMS.create(norm)
            self.ffn = FEED_FORWARDS.create(feed_forward)
            self._parts.update({"ffn_norm": self.ffn_norm, "ffn": self.ffn})

    def cache_spec(self):
        return self.mixer.cache_spec()

    def mixers(self):
        return [self.mixer]

    def subparts(self):
        return list(self._parts.values())

    def tensors(self):
        return {f"{p}.{name}": spec for p, part in self._parts.items() for name, spec in part.tensors().items()}

    def bind(self, weights, rt):
        self.rt = rt
        for p, part in self._parts.items():
            part.bind({k[len(p) + 1:]: v for k, v in weights.items() if k.startswith(p + ".")}, rt)

    def forward(self, stream, step, cache):
        stream.push(self.mixer.forward(stream.normed(self.mixer_norm, lazy=self.mixer.lazy_input), step, cache))
        if self.ffn is not None:
            stream.push(self.ffn.forward(stream.normed(self.ffn_norm, lazy=self.ffn.lazy_input), step))


@BLOCKS.register("outnorm")
class OutputNormBlock(PreNormBlock):
    """Norm on the sublayer's output only: x += Norm1(Mixer(x)); x += Norm2(FeedForward(x)).  The sublayers read
    the stream itself.  ``feed_forward`` may be ``None`` (then there is no second norm).  The norm must offer
    ``add_to``."""
    replayable = True

    def forward(self, stream, step, cache):
        stream.add_normed(self.mixer_norm, self.mixer.forward(stream.values(), step, cache))
        if self.ffn is not None:
            stream.add_normed(self.ffn_norm, self.ffn.forward(stream.values(), step))


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """One norm whose output both sublayers read: with h = Norm(x), x += Mixer(h) + FeedForward(h).
    ``feed_forward`` may be ``None`` (a layer of a mixer alone)."""
    replayable = True

    def __init__(self, mixer: PartSpec, feed_forward: PartSpec | None, norm: PartSpec):
        self.norm = NORMS.create(norm)
        self.mixer = MIXERS.create(mixer)
        self.ffn = FEED_FORWARDS.create(feed_forward) if feed_forward is not None else None
        self._parts = {"norm": self.norm, "mixer": self.mixer}
        if self.ffn is not None:
            self._parts["ffn"] = self.ffn

    def cache_spec(self):
        return self.mixer.cache_spec()

    def mixers(self):
        return [self.mixer]

    def subparts(self):
        return list(self._parts.values())

    def tensors(self):
        return {f"{p}.{name}": spec for p, part in self._parts.items() for name, spec in part.tensors().items()}

    def bind(self, weights, rt):
        self.rt = rt
        for p, part in self._parts.items():
            part.bind({k[len(p) + 1:]: v for k, v in weights.items() if k.startswith(p + ".")}, rt)

    def forward(self, stream, step, cache):
        # both read the same rows, so the norm's output is a tensor (never a norm left in factors); the
        # two deltas are added to the 32-bit stream one after the other
        h = stream.normed(self.norm)
        stream.push(self.mixer.forward(h, step, cache))
        if self.ffn is not None:
            stream.push(self.ffn.forward(h, step))


@BLOCKS.register("stream_reentry")
class StreamReentry(Block):
    """What stands before a stretch of layers that runs several times: x <- W [x ; x0] + b_t, x0 the
    embedding's output and t the number of the pass (``StepState.visit``: the block is one layer that the
    run order names once per pass).  The model must keep the embedding's output
    (``ModelSpec.keeps_embedding``).  No cache, no mixer."""
    replayable = True

    def __init__(self, hidden_size: int, times: int):
        self.hidden_size = hidden_size
        self.times = times

    def mixers(self):
        return []

    def tensors(self):
        W = self.hidden_size
        return {"in.weight": TensorSpec((W, 2 * W)), "step.weight": TensorSpec((self.times, W), "vector32", init="normal")}

    def bind(self, weights, rt):
        self.rt = rt
        self.w_in = rt.prepare_weight(weights["in.weight"])
        self.step_rows = [weights["step.weight"][t] for t in range(self.times)]

    def forward(self, stream, step, cache):
        rt, W = self.rt, self.hidden_size
        resid = stream.flush()
        x0 = step.scratch.get("embedding_output")
        if x0 is None:
            raise RuntimeError("stream_reentry: the model does not keep the embedding's output (ModelSpec.keeps_embedding)")
        if not 0 <= step.visit < self.times:
            raise RuntimeError(f"stream_reentry: pass {step.visit} of {self.times}")
        both = rt.buffer("reentry_in", resid.shape[0], 2 * W)
        ops.concat_cast(resid, x0, both)
        rt.gemm(both, self.w_in, resid)
        ops.add_rowvec(resid, self.step_rows[step.visit])
