"""The arrangement of a layer's parts around the residual stream.

``pre_norm``: x += mixer(norm(x)); x += feed_forward(norm(x)) (models/qwen3.py:254-287).  The residual
stream x is float32.  A branch's output is never added by a kernel of its own: it goes into a
``ResidualSink`` (parts/residual.py), and either the norm that reads x next adds it in the pass in which it
norms (the sum is made in 32-bit and written back to x), or the branch's last product does both.  So the
block gets its first norm's output from whoever ran before it, and returns the output of the norm that comes
after it.

``post_norm``: x += norm(mixer(x)); x += norm(feed_forward(x)): the norm sits on each branch's output, and the
branches read the stream itself (in the activation type).  A layer may have no feed-forward.  With
``depth_weights`` c (float32 [J + 1]) the layer's result R_J = x is kept beside the earlier ones (R_0: the embedding
rows) and what goes on is sum_j c[j] R_j: the model must say ``keeps_results``.  The norm, the add, the average and
the rounded copy for the next reader are one kernel.

``sandwich``: x += gain * norm_b(mixer(norm_a(x))); x += gain * norm_d(feed_forward(norm_c(x))): a norm on each side of
every branch and one multiplier on what is added.  A layer may have no feed-forward.  The norm of a branch's output, the
scaled add and the norm that reads the stream next are one kernel.

``pre_norm_scaled``: x += s1 * mixer(norm(x)); x += s2 * feed_forward(norm(x)) with learned vectors s1, s2 over the width
("layer scale").  A layer may have no feed-forward.  A branch may hand back a sum that is still to be made (the sides of
parallel mixers with their weights); the terms, the vector, the 32-bit add and the norm that reads the stream next are
one kernel.

``hyper_connections``: the residual stream runs in S copies x_1 .. x_S.  A sublayer reads u = sum_s in[s] x_s through its norm
(a ``streams_in`` reader), and its output y goes into all streams at once, x_t <- sum_s mix[s, t] x_s + out[t] y (every new
stream from the old ones).  A layer may have no feed-forward.  The write of one sublayer and the read of the next are one kernel.
"""
from __future__ import annotations

from ..kernels import ops
from .base import cache_needs, cache_needs_beside_shared, register_part
from .norm import PassThrough, StreamsReader
from .residual import ResidualSink, WeightedSum, as_tensor, run_branch


@register_part("block", "pre_norm")
class PreNormBlock:
    def __init__(self, spec, builder):
        self.mixer_norm = builder.build(spec.parts["mixer_norm"])
        self.mixer = builder.build(spec.parts["mixer"])
        self.feed_forward_norm = builder.build(spec.parts["feed_forward_norm"])
        self.feed_forward = builder.build(spec.parts["feed_forward"])

    @property
    def capturable(self) -> bool:
        return all(getattr(p, "capturable", False) for p in (self.mixer_norm, self.mixer, self.feed_forward_norm,
                                                              self.feed_forward))

    @staticmethod
    def cache_needs(spec):
        return cache_needs(spec.parts["mixer"])

    @property
    def entry_norm(self):
        return self.mixer_norm

    def forward(self, x, h, ctx, sink):
        h = run_branch(self.mixer, h, ctx, ResidualSink(x, self.feed_forward_norm))
        return run_branch(self.feed_forward, h, ctx, sink)


@register_part("block", "post_norm")
class PostNormBlock:
    def __init__(self, spec, builder):
        self.mixer = builder.build(spec.parts["mixer"])
        self.mixer_norm = builder.build(spec.parts["mixer_norm"])
        self.feed_forward = builder.build(spec.parts["feed_forward"]) if "feed_forward" in spec.parts else None
        self.feed_forward_norm = builder.build(spec.parts["feed_forward_norm"]) if self.feed_forward is not None else None
        self.depth_weights = builder.tensor(spec, "depth_weights") if "depth_weights" in spec.tensors else None
        self.dtype = builder.dtype
        self._reader = PassThrough(dtype=builder.dtype)
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and not getattr(norm, "folds_into_products", False):
                raise ValueError("a post_norm block norms its branches' outputs with RMS norms")

    @property
    def capturable(self) -> bool:
        parts = [self.mixer, self.mixer_norm] + ([self.feed_forward, self.feed_forward_norm] if self.feed_forward else [])
        return all(getattr(p, "capturable", False) for p in parts)

    @staticmethod
    def cache_needs(spec):
        return cache_needs(spec.parts["mixer"])

    @property
    def entry_norm(self):
        return self._reader

    def forward(self, x, h, ctx, sink):
        branches = [(self.mixer, self.mixer_norm)]
        if self.feed_forward is not None:
            branches.append((self.feed_forward, self.feed_forward_norm))
        for i, (part, norm) in enumerate(branches):
            y = part.forward(as_tensor(h), ctx)
            last = i + 1 == len(branches)
            if last and self.depth_weights is not None:
                if ctx.results is None:
                    raise RuntimeError("a block that averages over depth needs the earlier layers' results; the model keeps none")
                h = ops.add_normed(x, y, norm.weight, norm.eps, self.dtype, results=ctx.results, mix=self.depth_weights)
            else:
                h = ops.add_normed(x, y, norm.weight, norm.eps, self.dtype)
        if sink.rows is None and getattr(sink.norm, "passes_through", False):
            return h                                        # the next block reads the stream as it is
        return sink.norm(sink.x, rows=sink.rows)


@register_part("block", "sandwich")
class SandwichBlock:
    def __init__(self, spec, builder):
        self.gain = float(spec.params.get("residual_gain", 1.0))
        self.mixer_norm = builder.build(spec.parts["mixer_norm"])
        self.mixer = builder.build(spec.parts["mixer"])
        self.mixer_out_norm = builder.build(spec.parts["mixer_out_norm"])
        self.feed_forward = builder.build(spec.parts["feed_forward"]) if "feed_forward" in spec.parts else None
        self.feed_forward_norm = builder.build(spec.parts["feed_forward_norm"]) if self.feed_forward is not None else None
        self.feed_forward_out_norm = builder.build(spec.parts["feed_forward_out_norm"]) if self.feed_forward is not None else None
        self.dtype = builder.dtype
        for norm in (self.mixer_out_norm, self.feed_forward_out_norm):
            if norm is not None and not getattr(norm, "folds_into_products", False):
                raise ValueError("a sandwich block norms its branches' outputs with RMS norms")

    @property
    def capturable(self) -> bool:
        parts = [self.mixer_norm, self.mixer, self.mixer_out_norm]
        if self.feed_forward is not None:
            parts += [self.feed_forward_norm, self.feed_forward, self.feed_forward_out_norm]
        return all(getattr(p, "capturable", False) for p in parts)

    @staticmethod
    def cache_needs(spec):
        return cache_needs(spec.parts["mixer"])

    @property
    def entry_norm(self):
        return self.mixer_norm

    def _add(self, x, y, out_norm, reader, rows):
        """x += gain * out_norm(y); returns what ``reader`` (the norm that reads x next) makes of x, over ``rows``."""
        if rows is None and getattr(reader, "folds_into_products", False):
            return ops.add_normed_scaled(x, y, out_norm.weight, out_norm.eps, self.gain, reader.weight, reader.eps, self.dtype)
        ops.add_normed_scaled(x, y, out_norm.weight, out_norm.eps, self.gain)
        return reader(x, rows=rows)

    def forward(self, x, h, ctx, sink):
        y = self.mixer.forward(as_tensor(h), ctx)
        if self.feed_forward is None:
            return self._add(x, y, self.mixer_out_norm, sink.norm, sink.rows)
        h = self._add(x, y, self.mixer_out_norm, self.feed_forward_norm, None)
        y = self.feed_forward.forward(h, ctx)
        return self._add(x, y, self.feed_forward_out_norm, sink.norm, sink.rows)


@register_part("block", "pre_norm_scaled")
class ScaledPreNormBlock:
    def __init__(self, spec, builder):
        self.mixer_norm = builder.build(spec.parts["mixer_norm"])
        self.mixer = builder.build(spec.parts["mixer"])
        self.mixer_scale = builder.tensor(spec, "mixer_scale") if "mixer_scale" in spec.tensors else None
        self.feed_forward = builder.build(spec.parts["feed_forward"]) if "feed_forward" in spec.parts else None
        self.feed_forward_norm = builder.build(spec.parts["feed_forward_norm"]) if self.feed_forward is not None else None
        self.feed_forward_scale = builder.tensor(spec, "feed_forward_scale") if "feed_forward_scale" in spec.tensors else None
        self.dtype = builder.dtype
        width = int(spec.params["hidden_size"])
        for v in (self.mixer_scale, self.feed_forward_scale):
            if v is not None and v.shape != (width,):
                raise ValueError(f"a branch's scale is a vector over the width {width}, not {tuple(v.shape)}")

    @property
    def capturable(self) -> bool:
        parts = [self.mixer_norm, self.mixer] + ([self.feed_forward_norm, self.feed_forward] if self.feed_forward is not None else [])
        return all(getattr(p, "capturable", False) for p in parts)

    @staticmethod
    def cache_needs(spec):
        return cache_needs(spec.parts["mixer"])

    @property
    def entry_norm(self):
        return self.mixer_norm

    def _add(self, x, y, scale, reader, rows):
        """x += scale * y; returns what ``reader`` (the norm that reads x next) makes of x, over ``rows``."""
        terms, weights = (y.terms, y.weights) if isinstance(y, WeightedSum) else ([y], [1.0])
        while len(terms) > 2:                                   # the kernel adds two terms a pass
            ops.add_scaled_normed(x, terms[:2], weights[:2], scale, None, 0.0)
            terms, weights = terms[2:], weights[2:]
        if getattr(reader, "folds_into_products", False):
            if rows is not None:
                # the rows that are read next: their sums are made for the norm alone; the stream is not needed again
                return ops.add_scaled_normed(x, terms, weights, scale, reader.weight, reader.eps, self.dtype, rows=rows)
            return ops.add_scaled_normed(x, terms, weights, scale, reader.weight, reader.eps, self.dtype)
        ops.add_scaled_normed(x, terms, weights, scale, None, 0.0)
        return reader(x, rows=rows)

    def forward(self, x, h, ctx, sink):
        y = self.mixer.forward(as_tensor(h), ctx)
        if self.feed_forward is None:
            return self._add(x, y, self.mixer_scale, sink.norm, sink.rows)
        h = self._add(x, y, self.mixer_scale, self.feed_forward_norm, None)
        y = self.feed_forward.forward(h, ctx)
        return self._add(x, y, self.feed_forward_scale, sink.norm, sink.rows)


@register_part("block", "hyper_connections")
class HyperConnectionsBlock:
    def __init__(self, spec, builder):
        self.streams = int(spec.params["streams"])
        self.mixer_norm = builder.build(spec.parts["mixer_norm"])
        self.mixer = builder.build(spec.parts["mixer"])
        self.mixer_mix, self.mixer_out = builder.tensor(spec, "mixer_mix"), builder.tensor(spec, "mixer_out")
        self.feed_forward = builder.build(spec.parts["feed_forward"]) if "feed_forward" in spec.parts else None
        self.feed_forward_norm = builder.build(spec.parts["feed_forward_norm"]) if self.feed_forward is not None else None
        self.feed_forward_mix = builder.tensor(spec, "feed_forward_mix") if self.feed_forward is not None else None
        self.feed_forward_out = builder.tensor(spec, "feed_forward_out") if self.feed_forward is not None else None
        S = self.streams
        for mix, out_w in ((self.mixer_mix, self.mixer_out), (self.feed_forward_mix, self.feed_forward_out)):
            if mix is not None and (mix.shape != (S, S) or out_w.shape != (S,)):
                raise ValueError(f"{S} streams are written with weights [{S}, {S}] and [{S}], not {tuple(mix.shape)} and {tuple(out_w.shape)}")

    @property
    def capturable(self) -> bool:
        parts = [self.mixer_norm, self.mixer] + ([self.feed_forward_norm, self.feed_forward] if self.feed_forward is not None else [])
        return all(getattr(p, "capturable", False) for p in parts)

    @staticmethod
    def cache_needs(spec):
        return cache_needs(spec.parts["mixer"])

    @staticmethod
    def cache_needs_beside_shared(spec):
        return cache_needs_beside_shared(spec.parts["mixer"])

    @property
    def entry_norm(self):
        return self.mixer_norm

    @staticmethod
    def _write(x, y, mix, out_w, reader, rows):
        """The sublayer output y into the streams x; returns what ``reader`` makes of them, over ``rows``."""
        if isinstance(reader, StreamsReader):
            return reader.read(x, y, mix, out_w, rows=rows)
        xs = x.view(x.shape[0], 1, x.shape[1]) if x.dim() == 2 else x
        ops.streams_mix_norm(xs, y, mix, out_w, None, None, read=False)
        return reader(x, rows=rows)

    def forward(self, x, h, ctx, sink):
        y = as_tensor(self.mixer.forward(as_tensor(h), ctx))
        if self.feed_forward is None:
            return self._write(x, y, self.mixer_mix, self.mixer_out, sink.norm, sink.rows)
        h = self._write(x, y, self.mixer_mix, self.mixer_out, self.feed_forward_norm, None)
        y = as_tensor(self.feed_forward.forward(h, ctx))
        return self._write(x, y, self.feed_forward_mix, self.feed_forward_out, sink.norm, sink.rows)
