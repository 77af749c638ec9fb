"""How the parts of one layer are arranged.

"pre_norm" is rollout/monkey_patch/qwen3.py:59-68: h = h + attn(norm(h));
h = h + mlp(norm(h)). The addition of a part's output into the residual stream is
left to the next norm, which does it in 32-bit in the same kernel.

An arrangement is a class with
    __init__(self, spec: BlockSpec, build)      build(name) -> the built part spec.parts[name]
    cache_spec(self)                            what the layer keeps between steps (its mixer's
                                                PagedKVSpec or StateSpec), or None
    step_needs(self) -> dict                    what its parts ask of the step's tables (may be {})
    forward(self, h, pending, step, cache, write_cache) -> (h, pending)
        h: fp32 residual stream [T, H]; pending: the last part's output, not yet added to h
        (or None); cache: the cache manager's view for this call's cache layer (or None).
    Optional: first_norm / first_product attributes and an after= argument of forward (see PreNormBlock),
    with which the norm between two blocks can be finished inside their products.
It is registered with register_arrangement(name, cls) and named in BlockSpec.arrangement.
"""
from __future__ import annotations

import inspect

from .runtime import Normed, NormSink, Pair, ResidualSink, Scaled


_TAKES_SINK = {}


def takes_sink(part):
    """Whether the part's forward has a ``sink`` parameter (a part may note its last product for the
    kernel set's measurement and still form it itself: then it is never handed a sink)."""
    cls = type(part)
    hit = _TAKES_SINK.get(cls)
    if hit is None:
        try:
            hit = "sink" in inspect.signature(cls.forward).parameters
        except (AttributeError, TypeError, ValueError):
            hit = False
        _TAKES_SINK[cls] = hit
    return hit


def norm_sink(h, producer, norm, consumer_first_product):
    """The sink for the last product of ``producer``, whose result goes through ``norm`` into the next
    part, or None. A NormSink when the producer ends in one product and the consumer begins with one
    (their last_product / first_product attributes), the norm is a plain RMSNorm part, and the kernel
    set says that it can finish the norm inside these two products for this many rows
    (can_defer_norm); else a ResidualSink when the norm takes a product's result in every form
    (takes_slabs); else None: the part forms its product as it does for anyone."""
    ops = getattr(getattr(norm, "rt", None), "ops", None)
    last = getattr(producer, "last_product", None)
    if last is None or ops is None or norm is None or not takes_sink(producer):
        return None
    if consumer_first_product is not None and hasattr(ops, "can_defer_norm") and \
            hasattr(norm, "weight") and hasattr(norm, "eps"):
        first, gated = consumer_first_product
        if ops.can_defer_norm(h.shape[0], last, first, gated):
            return NormSink(ops, h, norm)
    return ResidualSink(ops) if getattr(norm, "takes_slabs", False) else None


class PreNormBlock:
    def __init__(self, spec, build):
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.feed_forward_norm = build("feed_forward_norm")
        self.feed_forward = build("feed_forward")
        # what the block before may fuse into: this block's first norm and the product behind it
        self.first_norm = self.mixer_norm
        self.first_product = getattr(self.mixer, "first_product", None)
        self.last_product = getattr(self.feed_forward, "last_product", None)

    def norm_pairs(self):
        """(product before, norm weight, eps, product after, gated) of the norm inside the block, if it sits
        between two products."""
        last, first = getattr(self.mixer, "last_product", None), getattr(self.feed_forward, "first_product", None)
        if last is None or first is None or not hasattr(self.feed_forward_norm, "weight"):
            return []
        return [(last, self.feed_forward_norm.weight, self.feed_forward_norm.eps, *first)]

    def cache_spec(self):
        return self.mixer.cache_spec()

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

    def forward(self, h, pending, step, cache, write_cache=True, after=None):
        """h: fp32 residual; pending: output of the last part, not yet added. Returns (h, pending).
        after: (norm, first product) of what takes this block's pending output, the next block's
        first_norm and first_product or the model's last norm and None; None: unknown. The norm may be
        finished inside this block's last product and that first one, or take the product in shares."""
        x = self.mixer_norm.forward(h, pending)
        sink = norm_sink(h, self.mixer, self.feed_forward_norm, getattr(self.feed_forward, "first_product", None))
        a = self.mixer.forward(x, step, cache, write_cache, sink) if sink is not None else \
            self.mixer.forward(x, step, cache, write_cache)
        x = self.feed_forward_norm.forward(h, a)
        sink = norm_sink(h, self.feed_forward, after[0], after[1]) if after is not None else None
        f = self.feed_forward.forward(x, step, sink) if sink is not None else self.feed_forward.forward(x, step)
        return h, f


class ConvSideBlock:
    """Pre-norm layer with a causal convolution in front of every sublayer and a token input at its end:

        h += mixer(conv_m(norm_m(h)));  h += feed_forward(conv_f(norm_f(h)));  h += token_input(h, token)

    where conv(x) = x + filter(x) over time (an "input_conv" part). Parts by name: mixer_norm, mixer and,
    each optional, mixer_conv, feed_forward_norm + feed_forward (both or neither), feed_forward_conv,
    token_input. What the layer keeps between steps is what its mixer keeps plus, if it has
    convolutions, one state of their tails: cache_spec() is the tuple (mixer's spec(s)..., tails)."""

    def __init__(self, spec, build):
        has = lambda name: name in spec.parts
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.mixer_conv = build("mixer_conv") if has("mixer_conv") else None
        self.feed_forward = build("feed_forward") if has("feed_forward") else None
        self.feed_forward_norm = build("feed_forward_norm") if self.feed_forward is not None else None
        self.feed_forward_conv = build("feed_forward_conv") if has("feed_forward_conv") and self.feed_forward is not None \
            else None
        self.token_input = build("token_input") if has("token_input") else None
        mixer_spec = self.mixer.cache_spec()
        self._mixer_specs = () if mixer_spec is None else \
            tuple(mixer_spec) if isinstance(mixer_spec, (tuple, list)) else (mixer_spec,)
        tails = []
        for name, conv in (("mixer_tail", self.mixer_conv), ("feed_forward_tail", self.feed_forward_conv)):
            if conv is not None:
                tails.append((name, tuple(conv.state_shape()), conv.rt.dtype_name))
        from ..cache.spec import StateSpec
        self._tails = StateSpec(tuple(tails)) if tails else None

    def cache_spec(self):
        specs = self._mixer_specs + ((self._tails,) if self._tails is not None else ())
        return None if not specs else specs[0] if len(specs) == 1 else specs

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

    @staticmethod
    def _normed(norm, conv, h, pending, step, tails, tail_name):
        """What a sublayer reads: the norm of the stream (pending added first) and, if there is one, the
        convolution behind it."""
        x = norm.forward(h, pending)
        return x if conv is None else conv.forward(x, step, tails[tail_name])

    def forward(self, h, pending, step, cache, write_cache=True):
        views = () if cache is None else tuple(cache) if isinstance(cache, (tuple, list)) else (cache,)
        n = len(self._mixer_specs)
        mixer_cache = None if n == 0 else views[0] if n == 1 else views[:n]
        tails = views[n].tensors if self._tails is not None else None
        x = self._normed(self.mixer_norm, self.mixer_conv, h, pending, step, tails, "mixer_tail")
        pending = self.mixer.forward(x, step, mixer_cache, write_cache)
        if self.feed_forward is not None:
            x = self._normed(self.feed_forward_norm, self.feed_forward_conv, h, pending, step, tails, "feed_forward_tail")
            pending = self.feed_forward.forward(x, step)
        if self.token_input is not None:
            self.token_input.forward(h, pending, step)
            pending = None
        return h, pending


class ScaledPreNormBlock:
    """Pre-norm layer whose sublayers enter the stream times a factor m, the feed-forward optional:

        h += m * mixer(mixer_norm(h));  h += m * feed_forward(feed_forward_norm(h))

    Parts by name: mixer_norm, mixer and, both or neither, feed_forward_norm + feed_forward. The factor is
    the BlockSpec's part "residual" (category "norm", kind "factor": a constant, no tensors) or 1. A
    sublayer's output is handed on as Scaled rows, which whatever adds it into the stream multiplies."""

    def __init__(self, spec, build):
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.feed_forward = build("feed_forward") if "feed_forward" in spec.parts else None
        self.feed_forward_norm = build("feed_forward_norm") if self.feed_forward is not None else None
        self.factor = float(build("residual").factor) if "residual" in spec.parts else 1.0

    def cache_spec(self):
        return self.mixer.cache_spec()

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

    def _out(self, y):
        return y if self.factor == 1.0 else Scaled(y, self.factor)

    def forward(self, h, pending, step, cache, write_cache=True):
        x = self.mixer_norm.forward(h, pending)
        pending = self._out(self.mixer.forward(x, step, cache, write_cache))
        if self.feed_forward is not None:
            x = self.feed_forward_norm.forward(h, pending)
            pending = self._out(self.feed_forward.forward(x, step))
        return h, pending


class PrePostNormBlock:
    """A layer with a norm on both sides of each sublayer, the feed-forward optional:

        h += mixer_post_norm(mixer(mixer_norm(h)));  h += feed_forward_post_norm(feed_forward(feed_forward_norm(h)))

    Parts by name: mixer_norm, mixer, mixer_post_norm and, all or none, feed_forward_norm, feed_forward,
    feed_forward_post_norm. A post norm's result stays 32-bit: the kernel set adds it into the stream as it forms
    it (post_norm_add), and where the next norm of the layer follows at once, that one is formed in the same kernel.
    The block leaves nothing pending unless asked to (defer_last)."""

    def __init__(self, spec, build):
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.mixer_post_norm = build("mixer_post_norm")
        self.feed_forward = build("feed_forward") if "feed_forward" in spec.parts else None
        self.feed_forward_norm = build("feed_forward_norm") if self.feed_forward is not None else None
        self.feed_forward_post_norm = build("feed_forward_post_norm") if self.feed_forward is not None else None
        for norm in (self.mixer_norm, self.mixer_post_norm, self.feed_forward_norm, self.feed_forward_post_norm):
            if norm is not None and not (hasattr(norm, "weight") and hasattr(norm, "eps")):
                raise ValueError("a layer with norms on both sides of its sublayers takes plain RMS norms")
        self.first_norm_part = self.mixer_norm
        self.defers_last = True                        # forward(..., defer_last=True) hands the last output back as a Normed

    def cache_spec(self):
        return self.mixer.cache_spec()

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

    def forward(self, h, pending, step, cache, write_cache=True, normed=None, defer_last=False):
        """normed: mixer_norm(h) where whatever made h has formed it already (pending is then None).
        defer_last: the last sublayer's output is handed back as pending (a Normed: its post norm and the addition
        are left to whatever forms the stream next)."""
        ops, rt = self.mixer_norm.rt.ops, self.mixer_norm.rt
        x = normed if normed is not None else self.mixer_norm.forward(h, pending)
        y = self.mixer.forward(x, step, cache, write_cache)
        post = self.mixer_post_norm
        if self.feed_forward is None:
            if defer_last:
                return h, Normed(y, post.weight, post.eps)
            ops.post_norm_add(h, y, post.weight, post.eps)
            return h, None
        nxt = self.feed_forward_norm
        x = rt.empty(h.shape[0], h.shape[1])
        ops.post_norm_add(h, y, post.weight, post.eps, nxt.weight, nxt.eps, x)
        y = self.feed_forward.forward(x, step)
        post = self.feed_forward_post_norm
        if defer_last:
            return h, Normed(y, post.weight, post.eps)
        ops.post_norm_add(h, y, post.weight, post.eps)
        return h, None


class ParallelPreNormBlock:
    """A layer whose two sublayers run side by side on the same stream, each behind a norm of its own, the
    feed-forward optional:

        h += mixer(mixer_norm(h)) + feed_forward(feed_forward_norm(h))

    Parts by name: mixer_norm, mixer and, both or neither, feed_forward_norm + feed_forward. Both norms are formed in
    one pass over the rows, which also adds what the layer before left pending; the layer's own two outputs are
    handed on as a Pair for whatever forms the stream next."""

    def __init__(self, spec, build):
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.feed_forward = build("feed_forward") if "feed_forward" in spec.parts else None
        self.feed_forward_norm = build("feed_forward_norm") if self.feed_forward is not None else None
        self._plain = all(n is None or (hasattr(n, "weight") and hasattr(n, "eps") and getattr(n, "size", None))
                          for n in (self.mixer_norm, self.feed_forward_norm))

    def cache_spec(self):
        return self.mixer.cache_spec()

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

    def forward(self, h, pending, step, cache, write_cache=True):
        rt = self.mixer_norm.rt
        if self.feed_forward is None:
            return h, self.mixer.forward(self.mixer_norm.forward(h, pending), step, cache, write_cache)
        if self._plain and hasattr(rt.ops, "add_rmsnorm_pair") and (pending is None or isinstance(pending, Pair)
                                                                    or hasattr(pending, "dtype")):
            a, b = (pending.first, pending.second) if isinstance(pending, Pair) else (pending, None)
            x1, x2 = rt.empty(h.shape[0], h.shape[1]), rt.empty(h.shape[0], h.shape[1])
            rt.ops.add_rmsnorm_pair(h, a, b, self.mixer_norm.weight, self.mixer_norm.eps, x1,
                                    self.feed_forward_norm.weight, self.feed_forward_norm.eps, x2)
        else:
            x1 = self.mixer_norm.forward(h, pending)
            x2 = self.feed_forward_norm.forward(h, None)
        y = self.mixer.forward(x1, step, cache, write_cache)
        f = self.feed_forward.forward(x2, step)
        return h, Pair(y, f)


BLOCKS = {"parallel_pre_norm": ParallelPreNormBlock, "pre_post_norm": PrePostNormBlock, "pre_norm": PreNormBlock, "pre_norm_conv_side": ConvSideBlock, "pre_norm_scaled": ScaledPreNormBlock}


def register_arrangement(name, cls):
    BLOCKS[name] = cls
