"""Arrangements of parts into a layer."""
from __future__ import annotations

from ..ops import kernels
from .base import Block, DeferredNorm
from .registry import register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += ff(norm2(x))   (pico_vllm/model.py:361-374).

    Each residual sum is fused into the norm that follows it: the block hands
    its last delta on as ``pending`` and the next block's (or the model's
    final) norm adds it.  The sums are float32."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ff": "feed_forward"}
    graph_safe_prompts = True

    @staticmethod
    def _normed(norm, consumer, resid, delta):
        """The normed activations for ``consumer``, or the norm left to it where both sides can."""
        if getattr(consumer, "takes_deferred_norm", False):
            later = norm.deferred(resid, delta)
            if later is not None:
                return later
        return norm.add_norm(resid, delta)

    @staticmethod
    def _after(h, resid):
        if isinstance(h, DeferredNorm):
            if h.resid is None:
                raise RuntimeError("a part took a deferred norm and neither ran nor fused it")
            return h.resid
        return resid

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        h = self._normed(p["norm1"], p["mixer"], resid, pending)
        a = p["mixer"].forward(h, ctx, cache)
        resid = self._after(h, resid)
        h = self._normed(p["norm2"], p["ff"], resid, a)
        f = p["ff"].forward(h, ctx)
        return self._after(h, resid), f


@register_part("block", "parallel")
class ParallelBlock(Block):
    """h = norm1(x); x += mixer(h) + ff(h): one norm, and both sublayers read its output.  A layer without a
    feed-forward names the part "none" in that slot.  The sums are float32: the mixer's output joins the residual stream
    at once (a mixer with ``forward_into(h, ctx, cache, resid)`` adds it itself, as the last step of its output
    projection), the feed-forward's is handed on as ``pending`` and the next norm adds it."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "ff": "feed_forward"}
    graph_safe_prompts = True

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        h = p["norm1"].add_norm(resid, pending)
        into = getattr(p["mixer"], "forward_into", None)
        if into is not None:
            into(h, ctx, cache, resid)                         # the mixer adds its output to the stream itself
            return resid, p["ff"].forward(h, ctx)
        a = p["mixer"].forward(h, ctx, cache)
        f = p["ff"].forward(h, ctx)
        if f is None:
            return resid, a
        for delta in (a if a.dim() == 3 else (a,)):            # a stack of partial sums: each in turn
            kernels.residual_add(resid, delta)
        return resid, f


@register_part("block", "parallel_two_norms")
class ParallelTwoNormBlock(Block):
    """x += mixer(norm1(x)) + ff(norm2(x)): both sublayers read the same x, each through a norm of its own.  The sums
    are float32.  A delta that is still pending joins the stream in the norms' launch (one launch makes both norms where
    they differ in their weights only).  The mixer's output joins the stream at once (a mixer with
    ``forward_into(h, ctx, cache, resid)`` adds it itself, as the last step of its output projection); so does what a
    feed-forward with ``forward_into(h, ctx, resid)`` adds itself; the feed-forward's last delta is handed on as
    ``pending`` (a feed-forward may return a list of deltas: all but the last are added here).  A layer without a
    feed-forward names the part "none" in that slot."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ff": "feed_forward"}
    graph_safe_prompts = True

    @staticmethod
    def _add(resid, delta):
        for d in (delta if delta.dim() == 3 else (delta,)):    # a stack of partial sums: each in turn
            kernels.residual_add(resid, d)

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        if pending is not None and pending.dim() == 3 and pending.shape[0] > kernels.MAX_SLABS:
            self._add(resid, pending)                          # more partial sums than a norm's launch takes
            pending = None
        pair = getattr(p["norm1"], "add_norm_pair", None)
        both = pair(p["norm2"], resid, pending) if pair is not None else None
        if both is None:
            both = (p["norm1"].add_norm(resid, pending), p["norm2"].add_norm(resid, None))
        h1, h2 = both
        into = getattr(p["mixer"], "forward_into", None)
        if into is not None:
            into(h1, ctx, cache, resid)
        else:
            self._add(resid, p["mixer"].forward(h1, ctx, cache))
        into = getattr(p["ff"], "forward_into", None)
        f = into(h2, ctx, resid) if into is not None else p["ff"].forward(h2, ctx)
        if isinstance(f, (list, tuple)):
            for d in f[:-1]:
                self._add(resid, d)
            f = f[-1]
        return resid, f


@register_part("block", "prenorm_scaled")
class ScaledPreNormBlock(Block):
    """x += m * s1 * mixer(norm1(x));  x += m * s2 * ff(norm2(x)): the pre-norm arrangement with a constant ``mult`` and
    a stored vector a sublayer (``scale_names``, behind the layer's prefix) on what joins the residual stream.  The
    products m * s are made once at load; the sums are float32.  The mixer's scaled output joins the stream in the
    launch of norm2 where that norm takes a scale on its addend (``takes_delta_scale``); the feed-forward's joins at
    once (a feed-forward with ``forward_scaled_into(h, ctx, resid, scale)`` adds it itself, in the launch that puts its
    pieces together), so nothing is handed on as pending.  A layer without a feed-forward names the part "none"."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ff": "feed_forward"}
    graph_safe_prompts = True

    def __init__(self, parts, size: int, mult: float = 1.0, scale_names=("ls1", "ls2")):
        super().__init__(parts)
        self.size, self.mult, self.scale_names = int(size), float(mult), tuple(scale_names)
        self.s1 = self.s2 = None

    def own_param_specs(self):
        from .spec import ParamSpec
        return [ParamSpec(n, (self.size,), role="norm") for n in self.scale_names]

    def load_own(self, tensors, device, dtype) -> None:
        import torch
        self.s1, self.s2 = ((tensors[n].to(device=device, dtype=torch.float32) * self.mult).contiguous() for n in self.scale_names)

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        h = p["norm1"].add_norm(resid, pending)
        a = p["mixer"].forward(h, ctx, cache)
        if getattr(p["norm2"], "takes_delta_scale", False) and not (a.dim() == 3 and a.shape[0] > kernels.LN_MAX_SLABS):
            h = p["norm2"].add_norm(resid, a, delta_scale=self.s1)
        else:
            kernels.scaled_add(resid, a, scale=self.s1)
            h = p["norm2"].add_norm(resid, None)
        into = getattr(p["ff"], "forward_scaled_into", None)
        if into is not None:
            into(h, ctx, resid, self.s2)
            return resid, None
        f = p["ff"].forward(h, ctx)
        for d in (f if isinstance(f, (list, tuple)) else (f,)):
            if d is not None:
                kernels.scaled_add(resid, d, scale=self.s2)
        return resid, None


@register_part("block", "prenorm_scaled_mixer_only")
class ScaledMixerOnlyBlock(ScaledPreNormBlock):
    """x += m * s1 * mixer(norm1(x)) and nothing else: the arrangement above for a layer without a feed-forward (and so
    without a second norm and a second vector)."""
    slot_categories = {"norm1": "norm", "mixer": "mixer"}

    def __init__(self, parts, size: int, mult: float = 1.0, scale_names=("ls1",)):
        super().__init__(parts, size, mult, tuple(scale_names)[:1])

    def load_own(self, tensors, device, dtype) -> None:
        import torch
        self.s1 = (tensors[self.scale_names[0]].to(device=device, dtype=torch.float32) * self.mult).contiguous()

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        h = p["norm1"].add_norm(resid, pending)
        kernels.scaled_add(resid, p["mixer"].forward(h, ctx, cache), scale=self.s1)
        return resid, None


@register_part("block", "postnorm")
class PostNormBlock(Block):
    """x += norm1(mixer(x)); x += norm2(ff(x)): the sublayers read the residual stream itself, and the norm stands on
    what a sublayer returns.  Each sum happens inside its norm's launch, in float32 (the next sublayer needs the new
    stream, so nothing is handed on as pending), and the same launch leaves the stream's rows in the activations' dtype
    for the next sublayer.  A mixer that offers ``forward_pair(h, ctx, cache) -> (a, wa, b, wb)`` (two mixers side by
    side) has both outputs normed with their own weights and averaged inside that launch too."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ff": "feed_forward"}
    graph_safe_prompts = True

    def _rows(self, resid, ctx):
        from .norm import stream_rows
        return stream_rows(resid, ctx, self.parts["norm1"].act_dtype)

    def _join(self, norm, resid, y, ctx, pair=None):
        from .norm import STREAM_COPY
        act = norm.act_dtype
        want = None if act == resid.dtype else act
        if pair is None:
            copy = kernels.norm_add(resid, y, norm.weight, norm.eps, want)
        else:
            a, wa, b, wb = pair
            copy = kernels.norm_add(resid, a, norm.weight, norm.eps, want, y2=b, weight1=wa, weight2=wb)
        if copy is not None:
            ctx.shared[STREAM_COPY] = (resid, copy)

    def _mixer(self, resid, pending, ctx, cache):
        p = self.parts
        if pending is not None:                                   # a block in front that hands a delta on
            for d in (pending if pending.dim() == 3 else (pending,)):
                kernels.residual_add(resid, d)
            from .norm import STREAM_COPY
            ctx.shared.pop(STREAM_COPY, None)                     # the stream's copy in the activations' type is stale now
        h = self._rows(resid, ctx)
        pair = getattr(p["mixer"], "forward_pair", None)
        if pair is not None:
            self._join(p["norm1"], resid, None, ctx, pair=pair(h, ctx, cache))
        else:
            self._join(p["norm1"], resid, p["mixer"].forward(h, ctx, cache), ctx)

    def forward(self, resid, pending, ctx, cache):
        self._mixer(resid, pending, ctx, cache)
        p = self.parts
        self._join(p["norm2"], resid, p["ff"].forward(self._rows(resid, ctx), ctx), ctx)
        return resid, None


@register_part("block", "postnorm_mixer_only")
class PostNormMixerOnlyBlock(PostNormBlock):
    """x += norm1(mixer(x)) and nothing else: the arrangement above for a layer without a feed-forward."""
    slot_categories = {"norm1": "norm", "mixer": "mixer"}

    def forward(self, resid, pending, ctx, cache):
        self._mixer(resid, pending, ctx, cache)
        return resid, None
