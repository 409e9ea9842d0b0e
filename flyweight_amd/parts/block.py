"""The arrangement of parts in a layer.

``pre_norm_residual``: x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x)), the residual
stream x in float32 (native/src/v2_runtime.cpp:28077,28282,28774,29133-29136). Another
arrangement (post-norm, parallel mixer and feed-forward) is another class registered here.

``output_norm_residual``: x <- x + m * norm1(mixer(x)); x <- x + m * norm2(ffn(x)). The sublayers
read x itself (rounded to the activation dtype for their products), the norm stands on a
sublayer's OUTPUT, and m is a fixed factor. The feed-forward may be absent.

``sandwich_norm_residual``: x <- x + post1(mixer(pre1(x))); x <- x + post2(ffn(pre2(x))), a norm before
and a norm behind every sublayer; then, where the layer has one, the tokens' own input
(``parts/token_input.py``): x <- x + rms(y(x, token)) * w. The feed-forward may be absent. Every sum into
x also forms what reads x next (the next norm's output, or x rounded) in the same kernel.


``parallel_residual``: with h = norm1(x), x <- x + (mixer(h) + ffn(h)): one norm, and both sublayers read its
output. The feed-forward may be absent.
"""

from __future__ import annotations

from ..config.spec import ConfigError
from ..kernels import ops
from .base import Block, build_part, register_block
from .norm import LazyNorm, NormedRows
from .token_input import TokenInput


@register_block("pre_norm_residual")
class PreNormResidualBlock(Block):
    def __init__(self, spec):
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm)
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn_norm = build_part("norm", spec.ffn_norm)
        self.ffn = build_part("ffn", spec.ffn)

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def first_norm(self):
        return self.mixer_norm

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        position = getattr(self.mixer, "position", None)
        return all(part.graph_safe for part in self.parts()) and (position is None or position.graph_safe)

    def forward(self, x, ctx, cache, prepared=None, norm_after=None):
        """``x`` [rows, hidden] float32 is updated in place."""
        # A part that can take the norm into its own first kernel gets it unevaluated. A part is
        # told which norm reads the residual after it (ctx.upcoming_norm) and may return what its
        # last product prepared for that norm; a part that returns nothing costs a plain norm.
        h = LazyNorm(self.mixer_norm, x, ctx, prepared=prepared)
        ctx.upcoming_norm = self.ffn_norm
        prepared = self.mixer.forward(h if getattr(self.mixer, "accepts_lazy_norm", False) else h.tensor(), x, ctx, cache)
        h = LazyNorm(self.ffn_norm, x, ctx, prepared=prepared)
        ctx.upcoming_norm = norm_after
        prepared = self.ffn.forward(h if getattr(self.ffn, "accepts_lazy_norm", False) else h.tensor(), x, ctx)
        ctx.upcoming_norm = None
        return prepared


class RoundedRows:
    """The residual rows once more in the activation dtype, left by the kernel that last changed
    them, for the block that reads them next. (``norm`` is None: a block that looks for a prepared
    norm finds none here.)"""
    norm = None

    def __init__(self, activations):
        self.activations = activations


@register_block("output_norm_residual")
class OutputNormResidualBlock(Block):
    def __init__(self, spec):
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm)
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        self.ffn_norm = build_part("norm", spec.ffn_norm) if spec.ffn is not None else None
        self.mult = float(spec.params.get("residual_mult", 1.0))
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and not hasattr(norm, "rms_parameters"):
                raise ConfigError("the output-norm arrangement takes RMS norms")

    def parts(self):
        return tuple(part for part in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if part is not None)

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        position = getattr(self.mixer, "position", None)
        return all(part.graph_safe for part in self.parts()) and (position is None or position.graph_safe)

    def _terms(self, part, *args):
        """A sublayer's output as [(float32 rows, scale)]: from the part itself if it can say so,
        else by letting it add into rows of zeros."""
        if hasattr(part, "output_terms"):
            return part.output_terms(*args)
        if hasattr(part, "output"):
            return [(part.output(*args), 1.0)]
        raise ConfigError(f"part '{part.spec.kind}' cannot give its output apart from the residual stream")

    def _join(self, x, terms, norm, dtype):
        """x += m * norm(sum of the terms); returns the new x rounded for the next reader."""
        weight, eps, one_centered = norm.rms_parameters()
        while len(terms) > 2:       # more than two branches: the last two are summed first
            (a, sa), (b, sb) = terms[-2], terms[-1]
            a = a * sa
            a.add_(b, alpha=sb)
            terms = terms[:-2] + [(a, 1.0)]
        (a, scale_a), (b, scale_b) = terms[0], terms[1] if len(terms) > 1 else (None, 1.0)
        return ops.norm_scale_add_(x, a, weight, eps, self.mult, b=b, scale_a=scale_a, scale_b=scale_b,
                                   one_centered=one_centered, rounded_dtype=None if dtype == x.dtype else dtype)

    def forward(self, x, ctx, cache, prepared=None, norm_after=None):
        """``x`` [rows, hidden] float32 is updated in place."""
        dtype = self.mixer_norm.dtype
        if isinstance(prepared, RoundedRows) and prepared.activations.shape == x.shape and prepared.activations.dtype == dtype:
            h = prepared.activations
        else:
            h = ops.round_rows(x, dtype)
        rounded = self._join(x, self._terms(self.mixer, h, ctx, cache), self.mixer_norm, dtype)
        if self.ffn is not None:
            h = x if rounded is None else rounded
            rounded = self._join(x, self._terms(self.ffn, h, ctx), self.ffn_norm, dtype)
        return None if rounded is None else RoundedRows(rounded)


@register_block("sandwich_norm_residual")
class SandwichNormResidualBlock(Block):
    """``LayerSpec.params``: ``mixer_post_norm`` and ``ffn_post_norm`` (PartSpecs of norms), ``token_input``
    (PartSpec of a :class:`TokenInput`, or absent). The norms may be RMS or layer norms, each on its own."""

    def __init__(self, spec):
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm)
        self.mixer = build_part("mixer", spec.mixer)
        self.mixer_post_norm = build_part("norm", spec.params["mixer_post_norm"])
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        self.ffn_norm = build_part("norm", spec.ffn_norm) if spec.ffn is not None else None
        self.ffn_post_norm = build_part("norm", spec.params["ffn_post_norm"]) if spec.ffn is not None else None
        given = spec.params.get("token_input")
        self.token_input = TokenInput(given) if given is not None else None
        for part in (self.mixer, self.ffn):
            if part is not None and not hasattr(part, "output"):
                raise ConfigError(f"part '{part.spec.kind}' cannot give its output apart from the residual stream")
        for norm in (self.mixer_norm, self.mixer_post_norm, self.ffn_norm, self.ffn_post_norm):
            if norm is not None and (not hasattr(norm, "row_norm") or getattr(norm, "one_centered", False)):
                raise ConfigError("the sandwich arrangement takes RMS norms with a plain weight and layer norms")

    def parts(self):
        return tuple(part for part in (self.mixer_norm, self.mixer, self.mixer_post_norm, self.ffn_norm, self.ffn,
                                       self.ffn_post_norm, self.token_input) if part is not None)

    def first_norm(self):
        return self.mixer_norm

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        position = getattr(self.mixer, "position", None)
        return all(part.graph_safe for part in self.parts()) and (position is None or position.graph_safe)

    @staticmethod
    def _reader(reader, dtype) -> dict:
        """What a kernel that sums into x is told about the next reader of x: a norm (its output), "rounded"
        (x in the activation dtype) or None."""
        if reader is None:
            return {}
        if reader == "rounded":
            return {"next_kind": ops.NEXT_ROUNDED, "next_dtype": dtype}
        next_weight, next_eps, next_centered = reader.row_norm()
        return {"next_kind": ops.NEXT_CENTERED if next_centered else ops.NEXT_RMS, "next_weight": next_weight, "next_eps": next_eps,
                "next_dtype": dtype}

    def _join(self, x, rows, norm, reader, dtype):
        """x += norm(rows); returns what ``reader`` sees of the new x (None for no reader)."""
        weight, eps, centered = norm.row_norm()
        return ops.norm_add_norm_(x, rows, weight, centered, eps, **self._reader(reader, dtype))

    def forward(self, x, ctx, cache, prepared=None, norm_after=None):
        """``x`` [rows, hidden] float32 is updated in place."""
        dtype = self.mixer_norm.dtype
        # a norm that follows this block is formed with the block's last sum only if it is of a form the kernel knows
        after = norm_after if hasattr(norm_after, "row_norm") and norm_after.row_norm() is not None else None
        h = LazyNorm(self.mixer_norm, x, ctx, prepared=prepared).tensor()
        last = self.ffn is None and self.token_input is None
        reader = after if last else (self.ffn_norm if self.ffn is not None else "rounded")     # the token input's product reads x rounded
        h = self._join(x, self.mixer.output(h, ctx, cache), self.mixer_post_norm, reader, dtype)
        if self.ffn is not None:
            reader = after if self.token_input is None else "rounded"
            h = self._join(x, self.ffn.output(h, ctx), self.ffn_post_norm, reader, dtype)
        if self.token_input is not None:
            h = self._join(x, self.token_input.output(h, ctx), self.token_input, after, dtype)
        return NormedRows(after, h) if after is not None and h is not None else None


@register_block("parallel_residual")
class ParallelResidualBlock(Block):
    """One norm whose output both sublayers read; their outputs join the residual stream together. Both
    sublayers add into the float32 stream in their last product's epilogue, the mixer first."""

    def __init__(self, spec):
        self.spec = spec
        self.norm = build_part("norm", spec.mixer_norm)
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        if spec.ffn_norm is not None:
            raise ConfigError("the parallel arrangement has one norm; its feed-forward reads the mixer's")

    def parts(self):
        return tuple(part for part in (self.norm, self.mixer, self.ffn) if part is not None)

    def first_norm(self):
        return self.norm

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        position = getattr(self.mixer, "position", None)
        return all(part.graph_safe for part in self.parts()) and (position is None or position.graph_safe)

    def forward(self, x, ctx, cache, prepared=None, norm_after=None):
        """``x`` [rows, hidden] float32 is updated in place."""
        # Both sublayers must see the norm of x as it was: the feed-forward may not take the norm into a
        # kernel of its own once the mixer has added to x, so it gets the rows normed beforehand unless the
        # mixer needs none of them (a mixer that takes the norm into its own first kernel reads x before it
        # writes it, and so does the feed-forward's product only if it runs first: it does not).
        h = LazyNorm(self.norm, x, ctx, prepared=prepared if isinstance(prepared, NormedRows) else None)
        normed = h.tensor() if self.ffn is not None or not getattr(self.mixer, "accepts_lazy_norm", False) else None
        ctx.upcoming_norm = None
        if normed is None or getattr(self.mixer, "wants_unnormed_rows", False):
            self.mixer.forward(h, x, ctx, cache)
        else:
            self.mixer.forward(normed, x, ctx, cache)
        if self.ffn is not None:
            self.ffn.forward(normed, x, ctx)
        return None
