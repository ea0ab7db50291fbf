"""Arrangements of norm, mixer and feed-forward in a block."""
from __future__ import annotations

import torch

from .. import ops
from .base import Part, PendingSum, as_tensor, register_part, run_norm


@register_part("block", "prenorm")
class PreNormBlock(Part):
    """h <- h + mixer(norm(h)); h <- h + ffn(norm(h)), with the sums carried in
    ``residual`` and made by the next norm (lite_llama/models/llama.py:138-162:
    the layer returns the feed-forward output and the residual without adding
    them; the next layer's first norm, or the final norm at :219, adds)."""

    def __init__(self, input_norm: Part, mixer: Part, post_norm: Part, feed_forward: Part):
        self.input_norm, self.mixer = input_norm, mixer
        self.post_norm, self.feed_forward = post_norm, feed_forward
        libs = ()
        for p in self.children().values():
            libs += tuple(p.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(libs))

    def children(self):
        """Sub-parts by the role the model's naming scheme addresses them with."""
        return {"input_norm": self.input_norm, "mixer": self.mixer,
                "post_norm": self.post_norm, "feed_forward": self.feed_forward}

    def cache_spec(self):
        return self.mixer.cache_spec() if hasattr(self.mixer, "cache_spec") else None

    def work_lists(self):
        """The work lists its parts want (parts.base.WorkList)."""
        lists = ()
        for p in self.children().values():
            if hasattr(p, "work_lists"):
                lists += tuple(p.work_lists())
        return tuple(dict.fromkeys(lists))

    can_defer_output = True

    @property
    def takes_pending_product(self) -> bool:
        """Whether the block before this one may leave its last product to this block's first
        norm (parts/base.py): what the model asks when it runs two blocks in a row."""
        return bool(getattr(self.input_norm, "takes_pending_product", False))

    def make_decode_copies(self) -> int:
        return sum(p.make_decode_copies() for p in self.children().values()
                   if hasattr(p, "make_decode_copies"))

    @property
    def graph_capturable(self) -> bool:
        return all(getattr(p, "graph_capturable", True) for p in self.children().values())

    def forward(self, h, residual, ctx, cache, defer_output: bool = False):
        """``h`` may be pending work of the block before (parts/base.py); with ``defer_output``
        the feed-forward may leave its last product to whoever normalises next."""
        mixer, ffn = self.mixer, self.feed_forward
        h, residual = run_norm(self.input_norm, h, residual, mixer)
        if not getattr(mixer, "takes_pending_scale", False):
            h = as_tensor(h)
        if (getattr(mixer, "can_defer_output", False)
                and getattr(self.post_norm, "takes_pending_product", False)):
            h = mixer.forward(h, ctx, cache, defer_output=True)
        else:
            h = mixer.forward(h, ctx, cache)
        h, residual = run_norm(self.post_norm, h, residual, ffn)
        if not getattr(ffn, "takes_pending_scale", False):
            h = as_tensor(h)
        if defer_output and getattr(ffn, "can_defer_output", False):
            h = ffn.forward(h, defer_output=True)
        else:
            h = ffn.forward(h)
        return h, residual


@register_part("block", "sandwich")
class SandwichBlock(Part):
    """A norm in front of and behind every sublayer, on a residual stream kept in float32:

        x <- x + post1(mixer(pre1(x)));   x <- x + post2(ffn(pre2(x)));   x <- side(x, tokens)

    The feed-forward (with its two norms) and the side input are optional. The stream is the
    block's ``h`` (float32 [T, hidden], updated in place); ``residual`` stays None. With
    Dynamic-Tanh norms the norm behind a sublayer, the sum and the norm in front of the next
    one are one kernel (ops.stream_add_dyt); other norms run through their own ``forward``
    and a plain sum into the stream. Sublayers read and return the engine's dtype (a
    feed-forward may return float32).

    ``next_norm`` (set by the model's builder): the Dynamic-Tanh norm in front of the mixer of
    the block that runs next. The block's last kernel then applies it as well and the second
    value it returns, where other blocks carry a residual, is the stream normed for that mixer;
    a block that is handed such a value starts from it instead of norming the stream itself."""

    def __init__(self, pre_mixer_norm: Part, mixer: Part, post_mixer_norm: Part,
                 pre_ffn_norm: Part = None, feed_forward: Part = None, post_ffn_norm: Part = None,
                 side: Part = None):
        if (feed_forward is None) != (pre_ffn_norm is None) or (feed_forward is None) != (post_ffn_norm is None):
            raise ValueError("a feed-forward comes with both of its norms, or none of the three")
        self.norm1, self.mixer, self.norm1b = pre_mixer_norm, mixer, post_mixer_norm
        self.norm2, self.feed_forward, self.norm2b = pre_ffn_norm, feed_forward, post_ffn_norm
        self.side = side
        libs = ("stream",)
        for p in self.children().values():
            libs += tuple(p.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(libs))
        self.dtype = None
        self.next_norm = None

    def children(self):
        roles = {"norm1": self.norm1, "mixer": self.mixer, "norm1b": self.norm1b, "norm2": self.norm2,
                 "feed_forward": self.feed_forward, "norm2b": self.norm2b, "side": self.side}
        return {k: p for k, p in roles.items() if p is not None}

    def cache_spec(self):
        return self.mixer.cache_spec() if hasattr(self.mixer, "cache_spec") else None

    def work_lists(self):
        lists = ()
        for p in self.children().values():
            if hasattr(p, "work_lists"):
                lists += tuple(p.work_lists())
        return tuple(dict.fromkeys(lists))

    def make_decode_copies(self) -> int:
        return sum(p.make_decode_copies() for p in self.children().values()
                   if hasattr(p, "make_decode_copies"))

    @property
    def graph_capturable(self) -> bool:
        return all(getattr(p, "graph_capturable", True) for p in self.children().values())

    @staticmethod
    def _fusable(norm) -> bool:
        return norm is None or hasattr(norm, "params")

    def _add(self, stream, y, post, pre, dtype, want_copy=False):
        """stream += post(y); returns (pre(stream) or None, copy or None)."""
        if self._fusable(post) and self._fusable(pre):
            return ops.stream_add_dyt(stream, y, post.params() if post is not None else None,
                                      pre.params() if pre is not None else None, dtype, want_copy)
        if y is not None:
            if post is not None:
                y = post.forward(y if y.dtype == dtype else y.to(dtype), None)[0]
            ops.stream_add_dyt(stream, y, None, None, dtype)
        copy = None
        if want_copy or pre is not None:
            _, copy = ops.stream_add_dyt(stream, None, None, None, dtype, True)
        out = pre.forward(copy, None)[0] if pre is not None else None
        return out, copy

    def forward(self, h, residual, ctx, cache):
        if h.dtype != torch.float32:
            raise ops.KernelError("a sandwich block runs on a float32 residual stream")
        stream = h
        dtype = self.mixer_dtype()
        if residual is not None:            # the stream, normed for this mixer by the block before
            a = residual
        else:
            a, _ = self._add(stream, None, None, self.norm1, dtype)
        y = self.mixer.forward(a, ctx, cache)
        nxt = self.next_norm if self._fusable(self.next_norm) else None
        want_copy = self.side is not None and dtype != torch.float32
        last_pre = None if self.side is not None else nxt
        if self.feed_forward is not None:
            a, _ = self._add(stream, y, self.norm1b, self.norm2, dtype)
            y = self.feed_forward.forward(a)
            ahead, copy = self._add(stream, y, self.norm2b, last_pre, dtype, want_copy)
        else:
            ahead, copy = self._add(stream, y, self.norm1b, last_pre, dtype, want_copy)
        if self.side is not None:
            ahead = self.side.forward(stream, copy if want_copy else stream, ctx.token_ids,
                                      nxt.params() if nxt is not None else None, dtype)
        return stream, ahead

    def mixer_dtype(self):
        """The engine's dtype, as the parts hold it after loading."""
        if self.dtype is None:
            self.dtype = getattr(self.norm1, "dtype", None)
        if self.dtype is None:
            for p in self.children().values():
                for t in vars(p).values():
                    if isinstance(t, torch.Tensor) and t.dim() >= 2 and t.is_floating_point():
                        self.dtype = t.dtype
                        return self.dtype
            raise RuntimeError("the block's parts hold no weights yet")
        return self.dtype


@register_part("block", "output_norm")
class OutputNormBlock(Part):
    """A norm on every sublayer's output only, on a residual stream kept in float32:

        x <- x + norm1(mixer(x));   x <- x + norm2(ffn(x))

    The sublayers read x itself (in the engine's dtype); the feed-forward with its norm is
    optional. The norms are RMS norms: the norm, the sum into the stream and the copy of the new
    stream in the engine's dtype for the next sublayer are one kernel, which also adds up a
    sublayer's result that arrives as a weighted sum not yet made (parts.base.PendingSum). The
    stream is the block's ``h`` (float32 [T, hidden], updated in place); what the block returns
    where others carry a residual is that copy, and a block that is handed one starts from it.
    ``last`` (set by the model's builder): nobody reads the copy after this block."""

    def __init__(self, mixer: Part, mixer_norm: Part, feed_forward: Part = None, ffn_norm: Part = None):
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with its norm, or neither")
        for n in (mixer_norm, ffn_norm):
            if n is not None and not (hasattr(n, "weight") and hasattr(n, "eps")):
                raise ValueError("the norms of this block are RMS norms (a weight and an eps)")
        self.mixer, self.norm1 = mixer, mixer_norm
        self.feed_forward, self.norm2 = feed_forward, ffn_norm
        libs = ("stream",)
        for p in self.children().values():
            libs += tuple(p.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(libs))
        self.last = False

    def children(self):
        roles = {"mixer": self.mixer, "norm1": self.norm1, "feed_forward": self.feed_forward,
                 "norm2": self.norm2}
        return {k: p for k, p in roles.items() if p is not None}

    def cache_spec(self):
        return self.mixer.cache_spec() if hasattr(self.mixer, "cache_spec") else None

    def work_lists(self):
        lists = ()
        for p in self.children().values():
            if hasattr(p, "work_lists"):
                lists += tuple(p.work_lists())
        return tuple(dict.fromkeys(lists))

    def make_decode_copies(self) -> int:
        return sum(p.make_decode_copies() for p in self.children().values()
                   if hasattr(p, "make_decode_copies"))

    @property
    def graph_capturable(self) -> bool:
        return all(getattr(p, "graph_capturable", True) for p in self.children().values())

    @staticmethod
    def _add(stream, y, norm, dtype, want_copy):
        """stream += norm(y); returns the new stream in ``dtype`` when asked (the stream itself
        when that is float32)."""
        copy = want_copy and dtype != torch.float32
        if isinstance(y, PendingSum):
            (y1, a), (y2, b) = y.terms[0], (y.terms[1] if len(y.terms) > 1 else (None, 0.0))
            bias, c = y.bias if y.bias is not None else (None, 0.0)
            out = ops.stream_add_rmsnorm_sum(stream, y1, a, y2, b, bias, c, norm.weight, norm.eps, dtype, copy)
        else:
            _, out = ops.stream_add_rmsnorm(stream, as_tensor(y), norm.weight, norm.eps, None, dtype, copy)
        return out if copy else (stream if want_copy else None)

    def forward(self, h, residual, ctx, cache):
        if h.dtype != torch.float32:
            raise ops.KernelError("an output-norm block runs on a float32 residual stream")
        stream, dtype = h, self.norm1.dtype
        a = residual
        if a is None:
            a = stream if dtype == torch.float32 else ops.stream_add_dyt(stream, None, None, None, dtype, True)[1]
        y = self.mixer.forward(a, ctx, cache)
        if self.feed_forward is None:
            return stream, self._add(stream, y, self.norm1, dtype, not self.last)
        a = self._add(stream, y, self.norm1, dtype, True)
        y = self.feed_forward.forward(a)
        return stream, self._add(stream, y, self.norm2, dtype, not self.last)
