"""Arrangements of norm, mixer and feed-forward in a block."""
from __future__ import annotations

import torch

from .. import ops
from .base import ParamSource, Part, PendingSum, as_tensor, place, register_part, run_norm


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


@register_part("block", "hyper_connections")
class HyperConnectionBlock(Part):
    """Pre-norm sublayers on several residual streams a token (hyper-connections; Zhu et al.,
    "Hyper-Connections"): the block's ``h`` is float32 [T, streams * hidden], stream after stream
    in a row. For the mixer and then the feed-forward (which is optional), with the sublayer's
    coefficients ``in`` [streams], ``mix`` [streams, streams] (from, to) and ``out`` [streams]:

        u = sum_s in[s] x_s;   y = sublayer(rmsnorm(u) w);   x_t <- sum_s mix[s, t] x_s + out[t] y

    all streams at once from the old ones. ``learned`` False: no coefficients in the checkpoint;
    one stream with in = mix = out = 1, which is x <- x + sublayer(rmsnorm(x) w) on a float32
    stream. The update behind a sublayer and the read-out with the norm in front of the next one
    are one kernel (ops.hyper_mix), also across blocks: the model tells the block which block runs
    next (``next_block``), the block's last kernel reads and norms for that block's mixer, and the
    result travels where other blocks carry a residual. Sublayers read the engine's dtype and may
    return float32."""
    takes_next_block = True

    def __init__(self, hidden_size: int, streams: int, mixer: Part, mixer_norm: Part, feed_forward: Part = None,
                 ffn_norm: Part = None, learned: bool = True, mixer_hc: str = "hc1.", ffn_hc: str = "hc2.",
                 in_name: str = "in", mix_name: str = "mix", out_name: str = "out"):
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with its norm, or neither")
        if not 1 <= streams <= ops.HYPER_MAX_STREAMS or (not learned and streams != 1):
            raise ValueError(f"1 to {ops.HYPER_MAX_STREAMS} streams (one when no coefficients are learned), "
                             f"got {streams}")
        for n in (mixer_norm, ffn_norm):
            if n is not None and not (hasattr(n, "weight") and hasattr(n, "eps")):
                raise ValueError("the norms of this block are RMS norms (a weight and an eps)")
        self.hidden_size, self.streams, self.learned = int(hidden_size), int(streams), bool(learned)
        self.mixer, self.norm1 = mixer, mixer_norm
        self.feed_forward, self.norm2 = feed_forward, ffn_norm
        self.hc_prefixes = (mixer_hc, ffn_hc)
        self.hc_names = (in_name, mix_name, out_name)
        self.coef = [None, None]            # per sublayer (in, mix, out) on the device, or None
        libs = ("stream",)
        for p in self._parts():
            libs += tuple(p.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(libs))

    def children(self):
        roles = {"mixer": self.mixer, "norm1": self.norm1, "feed_forward": self.feed_forward,
                 "norm2": self.norm2, "connections": self if self.learned else None}
        return {k: p for k, p in roles.items() if p is not None}

    def _parts(self):
        return [p for p in (self.mixer, self.norm1, self.feed_forward, self.norm2) if p is not None]

    def cache_spec(self):
        return self.mixer.cache_spec() if hasattr(self.mixer, "cache_spec") else None

    def work_lists(self):
        lists = ()
        for p in self._parts():
            if hasattr(p, "work_lists"):
                lists += tuple(p.work_lists())
        return tuple(dict.fromkeys(lists))

    def make_decode_copies(self) -> int:
        return sum(p.make_decode_copies() for p in self._parts() if hasattr(p, "make_decode_copies"))

    @property
    def graph_capturable(self) -> bool:
        return all(getattr(p, "graph_capturable", True) for p in self._parts())

    # the block's own tensors: the coefficients of its sublayers
    def param_sources(self):
        if not self.learned:
            return []
        S = self.streams
        i, m, o = self.hc_names
        out = []
        for q, prefix in enumerate(self.hc_prefixes):
            if q == 1 and self.feed_forward is None:
                continue
            out += [ParamSource(prefix + i, (S,), "vector", init=("normal", 1.0 / S, 0.1)),
                    ParamSource(prefix + o, (S,), "vector", init=("normal", 1.0, 0.1)),
                    ParamSource(prefix + m, (S, S), "vector", init=("normal", 1.0 / S, 0.15))]
        return out

    def load(self, tensors, dtype, device) -> None:
        if not self.learned:
            return
        i, m, o = self.hc_names
        for q, prefix in enumerate(self.hc_prefixes):
            if prefix + i in tensors:
                self.coef[q] = tuple(place(tensors[prefix + n], "vector", dtype, device) for n in (i, m, o))

    def read_args(self):
        """(in coefficients or None, norm weight, eps) of the read-out in front of the mixer."""
        c = self.coef[0]
        return (c[0] if c is not None else None, self.norm1.weight, self.norm1.eps)

    def _step(self, streams, y, q, nxt, dtype):
        """The update behind sublayer ``q`` (y None: none) and the read-out ``nxt`` = (in, weight,
        eps) in front of what follows (None: none)."""
        c = self.coef[q] if y is not None else None
        if isinstance(y, PendingSum) and len(y.terms) == 1 and y.terms[0][1] == 1.0 and y.bias is None:
            y = y.terms[0][0]
        if y is not None:
            y = as_tensor(y)
        inc, w, eps = nxt if nxt is not None else (None, None, 0.0)
        return ops.hyper_mix(streams, self.streams, y, c[1] if c is not None else None,
                             c[2] if c is not None else None, inc, w, eps, dtype)

    def forward(self, h, residual, ctx, cache, next_block=None):
        if h.dtype != torch.float32 or h.shape[1] != self.streams * self.hidden_size:
            raise ops.KernelError(f"a hyper-connection block runs on float32 rows of {self.streams} streams")
        streams, dtype = h, self.norm1.dtype
        a = residual if residual is not None else self._step(streams, None, 0, self.read_args(), dtype)
        y = self.mixer.forward(a, ctx, cache)
        after = next_block.read_args() if isinstance(next_block, HyperConnectionBlock) else None
        if self.feed_forward is None:
            return streams, self._step(streams, y, 0, after, dtype)
        c = self.coef[1]
        a = self._step(streams, y, 0, (c[0] if c is not None else None, self.norm2.weight, self.norm2.eps), dtype)
        y = self.feed_forward.forward(a)
        return streams, self._step(streams, y, 1, after, dtype)
