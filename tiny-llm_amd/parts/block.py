"""Block arrangements.  "pre_norm" is Llama's: x + mixer(norm(x)), then
x + ffn(norm(x)) (tiny_llm/parser/llama_parser.cpp:194-255).  "output_norm" puts the norm on each
sublayer's result instead: x + scale * norm(mixer(x)), then x + scale * norm(ffn(x)); the
sublayers read the residual stream itself.  "sum_norm" puts the norm behind the sum:
x <- norm(alpha * x + mixer(x)), then x <- norm(alpha * x + ffn(x)), alpha a constant of the model.
"sandwich" has a norm in front of and behind every sublayer: x <- x + mult * norm_b(mixer(norm_a(x))), then
x <- x + mult * norm_d(ffn(norm_c(x))), mult a constant of the model."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Block, register_block


class StreamCopyWanted:
    """What an arrangement whose sublayers read the stream itself shows as its `first_norm`: the block
    in front may hand over the copy of x in the engine's element type instead of a prepared norm."""


class PreNormBlock(Block):
    """x + mixer(norm(x)), then x + ffn(norm(x)); a layer may have no feed-forward (and then no second norm)."""
    roles = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}
    optional = ("ffn_norm", "ffn")

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.mixer = parts["mixer_norm"], parts["mixer"]
        self.ffn_norm, self.ffn = parts.get("ffn_norm"), parts.get("ffn")
        if (self.ffn is None) != (self.ffn_norm is None):
            raise ValueError("pre_norm: a feed-forward comes with its norm, and the norm with a feed-forward")

    def forward(self, x, ctx, caches, states):
        return self.forward_chained(x, ctx, caches, states)[0]

    @property
    def first_norm(self):
        """The norm that reads this block's input, for whoever writes that input."""
        return self.mixer_norm if getattr(self.mixer, "accepts_lazy_norm", False) else None

    def forward_chained(self, x, ctx, caches, states, prepared=None, next_norm=None):
        """As `forward`, between neighbours: `prepared` is this block's first norm as prepared by the
        product that wrote x (or None); `next_norm` is the norm that will read this block's result
        (or None).  Returns (x, that norm prepared or None)."""
        h = self._normed(self.mixer_norm, self.mixer, x, prepared)
        mixer_args = (h, ctx, caches.get("mixer"), states.get("mixer"), x)
        if self.ffn is None:
            return self._run(self.mixer, mixer_args, next_norm)
        ffn_norm = self.ffn_norm if getattr(self.ffn, "accepts_lazy_norm", False) else None
        x, prep = self._run(self.mixer, mixer_args, ffn_norm)
        h = self._normed(self.ffn_norm, self.ffn, x, prep)
        return self._run(self.ffn, (h, ctx, x), next_norm)

    @staticmethod
    def _run(part, args, next_norm):
        if next_norm is not None and getattr(part, "prepares_next_norm", False):
            out = part.forward(*args, next_norm=next_norm)
            return out if isinstance(out, tuple) else (out, None)
        return part.forward(*args), None

    @staticmethod
    def _normed(norm, consumer, x, prepared=None):
        # a consumer that says so may receive the norm unevaluated and fuse it into its first product
        if getattr(consumer, "accepts_lazy_norm", False) and hasattr(norm, "lazy"):
            return norm.lazy(x, prepared=prepared) if prepared is not None else norm.lazy(x)
        return norm.forward(x)


class OutputNormBlock(Block):
    """x <- x + s1 * norm1(mixer(x)); x <- x + s2 * norm2(ffn(x)).  The channel scales and the
    feed-forward (with its norm and scale) may be left out.  The sublayers are called with
    `residual=None` and return their result by itself in float32; norm, scale and the sum in float32
    are one kernel, which also writes the copy of x in the engine's element type that the next
    sublayer's products read (in float32 they read x itself)."""
    roles = {"mixer": "mixer", "mixer_norm": "norm", "mixer_scale": "scale",
             "ffn": "feed_forward", "ffn_norm": "norm", "ffn_scale": "scale"}
    optional = ("mixer_scale", "ffn", "ffn_norm", "ffn_scale")

    _WantsCopy = StreamCopyWanted

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer, self.mixer_norm = parts["mixer"], parts["mixer_norm"]
        self.mixer_scale = parts.get("mixer_scale")
        self.ffn, self.ffn_norm, self.ffn_scale = parts.get("ffn"), parts.get("ffn_norm"), parts.get("ffn_scale")
        if (self.ffn is None) != (self.ffn_norm is None) or (self.ffn is None and self.ffn_scale is not None):
            raise ValueError("output_norm: a feed-forward comes with its norm, and a scale only with both")
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and not hasattr(n, "add_normed"):
                raise ValueError(f"output_norm: the norm {type(n).__name__} cannot sit on a sublayer's output (no add_normed)")
        self.first_norm = self._WantsCopy()

    def forward(self, x, ctx, caches, states):
        return self.forward_chained(x, ctx, caches, states)[0]

    def _input(self, x, name):
        if x.dtype == self.mixer.dtype:
            return x
        return ops.cast_rows(x, ops.scratch(name, x.shape, self.mixer.dtype, x.device, rotate=2))

    def forward_chained(self, x, ctx, caches, states, prepared=None, next_norm=None):
        """`prepared`: the copy of x in the engine's element type, if the block in front was of this
        kind; returned likewise for the block behind (`next_norm` is then its `first_norm`)."""
        low = x.dtype != self.mixer.dtype          # the products read a copy in the engine's type
        h = prepared if (low and isinstance(prepared, torch.Tensor)) else self._input(x, "stream_copy")
        y = self.mixer.forward(h, ctx, caches.get("mixer"), states.get("mixer"), None)
        want_after = low and (self.ffn is not None or isinstance(next_norm, self._WantsCopy))
        copy = ops.scratch("stream_copy", x.shape, self.mixer.dtype, x.device, rotate=2) if want_after else None
        self.mixer_norm.add_normed(y, x, self.mixer_scale.weight if self.mixer_scale is not None else None, copy)
        if self.ffn is None:
            return x, copy
        y = self.ffn.forward(copy if low else x, ctx, None)
        copy = None
        if low and isinstance(next_norm, self._WantsCopy):
            copy = ops.scratch("stream_copy", x.shape, self.mixer.dtype, x.device, rotate=2)
        self.ffn_norm.add_normed(y, x, self.ffn_scale.weight if self.ffn_scale is not None else None, copy)
        return x, copy


class SumNormBlock(Block):
    """x <- norm1(alpha * x + mixer(x)); x <- norm2(alpha * x + ffn(x)).  The sublayers read x itself, are
    called with `residual=None` and return their result by itself in float32; scaling, sum and norm in
    float32 are one kernel, which also writes the copy of x in the engine's element type that the next
    sublayer's products read (in float32 they read x itself).  A layer may have no feed-forward; if it
    still has a second norm, that norm runs on alpha * x."""
    roles = {"mixer": "mixer", "mixer_norm": "norm", "ffn": "feed_forward", "ffn_norm": "norm"}
    optional = ("ffn", "ffn_norm")

    _WantsCopy = StreamCopyWanted

    def __init__(self, parts, alpha: float = 1.0):
        super().__init__(parts)
        self.alpha = float(alpha)
        self.mixer, self.mixer_norm = parts["mixer"], parts["mixer_norm"]
        self.ffn, self.ffn_norm = parts.get("ffn"), parts.get("ffn_norm")
        if self.ffn is not None and self.ffn_norm is None:
            raise ValueError("sum_norm: a feed-forward comes with its norm")
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and not hasattr(n, "sum_normed"):
                raise ValueError(f"sum_norm: the norm {type(n).__name__} cannot follow a sum (no sum_normed)")
        self.first_norm = self._WantsCopy()

    def forward(self, x, ctx, caches, states):
        return self.forward_chained(x, ctx, caches, states)[0]

    def _copy(self, x):
        return ops.scratch("stream_copy", x.shape, self.mixer.dtype, x.device, rotate=2)

    def forward_chained(self, x, ctx, caches, states, prepared=None, next_norm=None):
        """`prepared`: the copy of x in the engine's element type, if the block in front hands one over;
        returned likewise for the block behind (when `next_norm` says it takes one)."""
        low = x.dtype != self.mixer.dtype          # the products read a copy in the engine's type
        wanted_behind = low and isinstance(next_norm, StreamCopyWanted)
        h = x
        if low:
            h = prepared if isinstance(prepared, torch.Tensor) else ops.cast_rows(x, self._copy(x))
        y = self.mixer.forward(h, ctx, caches.get("mixer"), states.get("mixer"), None)
        second = self.ffn_norm is not None
        copy = self._copy(x) if low and (self.ffn is not None or (not second and wanted_behind)) else None
        self.mixer_norm.sum_normed(y, x, self.alpha, copy)
        if not second:
            return x, copy
        y = self.ffn.forward(copy if low else x, ctx, None) if self.ffn is not None else None
        copy = self._copy(x) if wanted_behind else None
        self.ffn_norm.sum_normed(y, x, self.alpha, copy)
        return x, copy


class NormedRows:
    """What a sandwich block hands to the block behind it: the stream as that block's first norm sees it,
    formed by the kernel that wrote the stream."""

    def __init__(self, norm, rows: torch.Tensor):
        self.norm, self.rows = norm, rows


class SandwichBlock(Block):
    """x <- x + mult * LNb(mixer(LNa(x))); x <- x + mult * LNd(ffn(LNc(x))): a norm in front of and behind every
    sublayer.  The sublayers are called with `residual=None` and return their result by itself in float32; the norm
    behind a sublayer, the scaled sum and the norm in front of whatever reads the stream next (this block's
    feed-forward, or the next block's mixer if that block says which norm it begins with) are ONE kernel.  A layer
    may have no feed-forward (and then neither of its norms)."""
    roles = {"mixer_norm": "norm", "mixer": "mixer", "mixer_out_norm": "norm",
             "ffn_norm": "norm", "ffn": "feed_forward", "ffn_out_norm": "norm"}
    optional = ("ffn_norm", "ffn", "ffn_out_norm")

    def __init__(self, parts, mult: float = 1.0):
        super().__init__(parts)
        self.mult = float(mult)
        self.mixer_norm, self.mixer, self.mixer_out_norm = parts["mixer_norm"], parts["mixer"], parts["mixer_out_norm"]
        self.ffn_norm, self.ffn, self.ffn_out_norm = parts.get("ffn_norm"), parts.get("ffn"), parts.get("ffn_out_norm")
        if len({self.ffn is None, self.ffn_norm is None, self.ffn_out_norm is None}) != 1:
            raise ValueError("sandwich: a feed-forward comes with both of its norms, and they with a feed-forward")
        for n in (self.mixer_out_norm, self.ffn_out_norm):
            if n is not None and not hasattr(n, "add_scaled_norm"):
                raise ValueError(f"sandwich: the norm {type(n).__name__} cannot sit on a sublayer's result (no add_scaled_norm)")

    @property
    def first_norm(self):
        """The norm that reads this block's input, for whoever writes that input."""
        return self.mixer_norm

    def forward(self, x, ctx, caches, states):
        return self.forward_chained(x, ctx, caches, states)[0]

    @staticmethod
    def _fusable(out_norm, next_norm):
        """Whether `out_norm.add_scaled_norm` can also produce `next_norm` of the new stream."""
        return type(next_norm) is type(out_norm) and getattr(next_norm, "hidden_size", None) == out_norm.hidden_size

    def forward_chained(self, x, ctx, caches, states, prepared=None, next_norm=None):
        """`prepared`: NormedRows of this block's first norm if the block in front formed them; returned likewise
        for the block behind when `next_norm` is a norm this block's last kernel can form."""
        if isinstance(prepared, NormedRows) and prepared.norm is self.mixer_norm:
            h = prepared.rows
        else:
            h = self.mixer_norm.forward(x)
        y = self.mixer.forward(h, ctx, caches.get("mixer"), states.get("mixer"), None)
        if self.ffn is None:
            return x, self._add(self.mixer_out_norm, y, x, next_norm)
        handed = self._add(self.mixer_out_norm, y, x, self.ffn_norm)
        h = handed.rows if handed is not None else self.ffn_norm.forward(x)
        y = self.ffn.forward(h, ctx, None)
        return x, self._add(self.ffn_out_norm, y, x, next_norm)

    def _add(self, out_norm, y, x, next_norm):
        if next_norm is not None and self._fusable(out_norm, next_norm):
            rows = out_norm.add_scaled_norm(y, x, self.mult, then=next_norm)
            return NormedRows(next_norm, rows) if rows is not None else None
        out_norm.add_scaled_norm(y, x, self.mult)
        return None


register_block("pre_norm", PreNormBlock)
register_block("sandwich", SandwichBlock)
register_block("sum_norm", SumNormBlock)
register_block("output_norm", OutputNormBlock)
