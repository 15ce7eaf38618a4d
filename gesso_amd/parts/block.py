"""A block: how a mixer, a feed-forward and their norms are arranged around the residual stream.

``prenorm``: ``h += mixer(norm_a(h)); h += ffn(norm_b(h))`` (reference
``src/Inference/Inference.jl:270-363``).  Each add is folded into the norm that follows it;
the model adds what is still pending after the last block.  A sub-layer may return a tensor or a
deferred product (its last projection, computed straight into the stream).  Another arrangement (post-norms on
sub-layer outputs, a parallel block) is another class registered under another kind.
"""
from __future__ import annotations

from .base import Part, sub_tensors
from .registry import build, part_class, register


class PreNormBlock(Part):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer_norm = build("norm", spec.mixer_norm, rt)
        self.mixer = build("mixer", spec.mixer, rt)
        self.ffn = self.ffn_norm = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, rt)
            self.ffn = build("ffn", spec.ffn, rt)

    @staticmethod
    def tensor_specs(spec):
        out = {}
        roles = [("mixer_norm", "norm", spec.mixer_norm), ("mixer", "mixer", spec.mixer)]
        if spec.ffn is not None:
            roles += [("ffn_norm", "norm", spec.ffn_norm), ("ffn", "ffn", spec.ffn)]
        for role, category, sub in roles:
            for name, ts in part_class(category, sub).tensor_specs(sub).items():
                out[f"{role}.{name}"] = ts
        return out

    @staticmethod
    def cache_need(spec):
        cls = part_class("mixer", spec.mixer)
        return cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None

    def bind(self, tensors):
        self.mixer_norm.bind(sub_tensors(tensors, "mixer_norm"))
        self.mixer.bind(sub_tensors(tensors, "mixer"))
        if self.ffn is not None:
            self.ffn_norm.bind(sub_tensors(tensors, "ffn_norm"))
            self.ffn.bind(sub_tensors(tensors, "ffn"))

    @property
    def first_norm(self):
        """The norm that reads the stream first when this block runs (a hint for whoever writes the stream before)."""
        return self.mixer_norm

    def forward(self, stream, ctx, cache):
        after, rt = stream.following, self.rt
        with rt.stage("norm"):
            x = self.mixer_norm.add_norm(stream)
        # a stage per kind of mixer (the profiler's names: conv_mixer, attn_mixer, ...); a sub-layer's last product
        # runs inside push, straight into the stream, and belongs to its stage
        with rt.stage(getattr(self.mixer, "stage", "mixer")):
            out = self.mixer.forward(x, ctx, cache)
            with rt.stage(getattr(self.mixer, "out_stage", "mixer_out")):
                stream.push(out, rt, next_norm=self.ffn_norm if self.ffn is not None else after)
        if self.ffn is not None:
            with rt.stage("norm"):
                x = self.ffn_norm.add_norm(stream)
            with rt.stage(getattr(self.ffn, "stage", "ffn")):
                out = self.ffn.forward(x, ctx)
                with rt.stage(getattr(self.ffn, "out_stage", "ffn_out")):
                    stream.push(out, rt, next_norm=after)

    @property
    def portions_recordable(self) -> bool:
        """Whether a step of prompt portions through this block may be recorded for replay (see ``Model``)."""
        parts = [self.mixer_norm, self.mixer] + ([self.ffn_norm, self.ffn] if self.ffn is not None else [])
        return all(getattr(p, "portions_recordable", False) for p in parts)

    def replay_key(self, q_lens, max_kv_len):
        f = getattr(self.mixer, "replay_key", None)
        return f(q_lens, max_kv_len) if f is not None else None

    @property
    def graph_safe(self) -> bool:
        """Whether a step through this block may be recorded into a HIP graph (no host round trips inside)."""
        parts = [self.mixer_norm, self.mixer] + ([self.ffn_norm, self.ffn] if self.ffn is not None else [])
        return all(getattr(p, "graph_safe", False) for p in parts)


class OutNormBlock(PreNormBlock):
    """``h += mult * norm_a(mixer(h)); h += mult * norm_b(ffn(h))``: the norms stand on the sub-layers' outputs, the
    sub-layers read the stream itself (in the activation type).  The add, the norm and the rows for the next
    sub-layer are one kernel."""

    first_norm = None           # nothing norms the stream before this block's mixer reads it

    def forward(self, stream, ctx, cache):
        rt, ops, s = self.rt, self.rt.ops, self.spec
        rows_dtype = None if rt.dtype == stream.res.dtype else rt.dtype
        stream.flush(rt)
        x = stream.rows
        if x is None:
            x = stream.res if rows_dtype is None else ops.norm_scaled_add(stream.res, None, None, 0.0, 0.0, rows_dtype)
        with rt.stage(getattr(self.mixer, "stage", "mixer")):
            y = rt.dense(self.mixer.forward(x, ctx, cache))
        with rt.stage("norm"):
            x = ops.norm_scaled_add(stream.res, y, self.mixer_norm.weight, self.mixer_norm.spec.eps, s.mult, rows_dtype)
        if self.ffn is not None:
            with rt.stage(getattr(self.ffn, "stage", "ffn")):
                y = rt.dense(self.ffn.forward(stream.res if rows_dtype is None else x, ctx))
            with rt.stage("norm"):
                x = ops.norm_scaled_add(stream.res, y, self.ffn_norm.weight, self.ffn_norm.spec.eps, s.mult, rows_dtype)
        # what earlier writers left beside the stream (sums of squares, pre-weighted rows) no longer describes it
        stream.pending = stream.ssq = stream.xs = stream.xs_for = stream.normed = None
        stream.rows = x

    @property
    def portions_recordable(self) -> bool:
        return False


class ParallelBlock(PreNormBlock):
    """``h += mixer(norm_a(h)) + ffn(norm_b(h))``: both sub-layers read the stream as it enters the block, each
    through its own norm.  One kernel adds what the block before left (its two results) and norms the row for both
    readers; the block's own two results stay beside the stream for whoever norms it next."""

    def forward(self, stream, ctx, cache):
        rt, ops = self.rt, self.rt.ops
        held = stream.pending if isinstance(stream.pending, tuple) else (stream.pending, None)
        with rt.stage("norm"):
            second = self.ffn_norm if self.ffn is not None else None
            x1, x2 = ops.add_rmsnorm_pair(stream.res, held[0], held[1], self.mixer_norm.weight,
                                          None if second is None else second.weight, self.mixer_norm.spec.eps, rt.dtype,
                                          bias=stream.bias)
        stream.pending = stream.ssq = stream.xs = stream.xs_for = stream.normed = stream.rows = stream.bias = None
        with rt.stage(getattr(self.mixer, "stage", "mixer")):
            a = rt.dense(self.mixer.forward(x1, ctx, cache))
        b = None
        if self.ffn is not None:
            with rt.stage(getattr(self.ffn, "stage", "ffn")):
                if getattr(self.ffn, "defers_bias", False):
                    # the last product's bias waits for the pass that adds the product to the stream
                    b, stream.bias = self.ffn.forward(x2, ctx, defer_bias=True)
                    b = rt.dense(b)
                else:
                    b = rt.dense(self.ffn.forward(x2, ctx))
        stream.pending = (a, b)

    @property
    def first_norm(self):
        return None                 # the block norms the stream itself, twice in one pass

    @property
    def portions_recordable(self) -> bool:
        return False


class SharedNormBlock(Part):
    """``h += mixer(a + conv(a)) + ffn(a)`` with ``a = norm(h)``: one norm, read by both sub-layers; the mixer's input
    may get a causal convolution over time added to it (``spec.input_taps``), whose last inputs are the request's state,
    kept in its slot beside whatever the mixer keeps.  The norm's pass adds the two results that the block before left;
    this block's own two results stay beside the stream for whoever norms it next."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.norm = build("norm", spec.norm, rt)
        self.mixer = build("mixer", spec.mixer, rt)
        self.ffn = build("ffn", spec.ffn, rt) if spec.ffn is not None else None
        self.taps = None

    @staticmethod
    def _width(spec) -> int:
        return int(spec.norm.size)

    @staticmethod
    def tensor_specs(spec):
        from .base import VECTOR, TensorSpec
        out = {}
        roles = [("norm", "norm", spec.norm), ("mixer", "mixer", spec.mixer)]
        if spec.ffn is not None:
            roles.append(("ffn", "ffn", spec.ffn))
        for role, category, sub in roles:
            for name, ts in part_class(category, sub).tensor_specs(sub).items():
                out[f"{role}.{name}"] = ts
        if spec.input_taps is not None:
            out["input_conv.weight"] = TensorSpec((SharedNormBlock._width(spec), spec.input_taps), VECTOR)
        return out

    @staticmethod
    def _mixer_needs(spec) -> tuple:
        cls = part_class("mixer", spec.mixer)
        need = cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None
        return tuple(need) if isinstance(need, (tuple, list)) else (need,)

    @staticmethod
    def cache_need(spec):
        from .base import SlotState
        mixer = SharedNormBlock._mixer_needs(spec)
        if spec.input_taps is None:
            return mixer if len(mixer) > 1 else mixer[0]
        # (a single tap has no history; a row is kept all the same, which nobody reads)
        own = SlotState((("input_history", (max(spec.input_taps - 1, 1), SharedNormBlock._width(spec)), "float32"),))
        return (own,) + mixer

    def bind(self, tensors):
        self.norm.bind(sub_tensors(tensors, "norm"))
        self.mixer.bind(sub_tensors(tensors, "mixer"))
        if self.ffn is not None:
            self.ffn.bind(sub_tensors(tensors, "ffn"))
        if self.spec.input_taps is not None:
            self.taps = tensors["input_conv.weight"].contiguous()

    @property
    def first_norm(self):
        return None                 # the norm's pass is the block's own business

    def forward(self, stream, ctx, cache):
        rt, ops, s = self.rt, self.rt.ops, self.spec
        with rt.stage("norm"):
            a = self.norm.add_norm(stream)
        x = a
        mixer_cache = cache
        if s.input_taps is not None:
            with rt.stage("input_conv"):
                history = cache[0].state["input_history"]
                rest = cache[1:]
                mixer_cache = rest if len(rest) > 1 else rest[0]
                x = ops.channel_conv(a, self.taps, None, history, ctx.seq_of_token, ctx.q_start, ctx.slots, ctx.nseq,
                                     ctx.all_single, rt.dtype, residual=True)
        with rt.stage(getattr(self.mixer, "stage", "mixer")):
            m = rt.dense(self.mixer.forward(x, ctx, mixer_cache))
        f = None
        if self.ffn is not None:
            with rt.stage(getattr(self.ffn, "stage", "ffn")):
                f = rt.dense(self.ffn.forward(a, ctx))
        stream.pending = (m, f)

    @property
    def graph_safe(self) -> bool:
        parts = [self.norm, self.mixer] + ([self.ffn] if self.ffn is not None else [])
        return all(getattr(p, "graph_safe", False) for p in parts)

    portions_recordable = False


register("block", "prenorm", PreNormBlock)
register("block", "shared_norm", SharedNormBlock)
register("block", "parallel", ParallelBlock)
register("block", "outnorm", OutNormBlock)
