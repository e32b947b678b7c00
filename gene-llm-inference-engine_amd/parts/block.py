"""Arrangements of a layer's parts around the residual stream.

"prenorm" (reference: src/model/transformer.cpp:385-450):
    x += mixer(norm_1(x));  x += feed_forward(norm_2(x))
"sandwich": a norm before and a norm after each half; the feed-forward half may be absent:
    x += post_1(mixer(norm_1(x)));  x += post_2(feed_forward(norm_2(x)))
"parallel": one norm, read by the mixer and by the feed-forward (which may be absent):
    h = norm_1(x);  x += mixer(h) + feed_forward(h)
The residual stream x is float32 [T, hidden] and is changed in place."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import feed_forward_class, mixer_class, norm_class, register_block
from .linear import linear, takes_handed_norm
from .norm import NormedRows, norm_to_hand_on


class PreNormBlock:
    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec
        self.mixer_norm = norm_class(spec.mixer_norm)(spec.mixer_norm, tensors, dtype, device)
        self.mixer = mixer_class(spec.mixer)(spec.mixer, tensors, dtype, device)
        self.feed_forward_norm = norm_class(spec.feed_forward_norm)(spec.feed_forward_norm, tensors, dtype, device)
        self.feed_forward = feed_forward_class(spec.feed_forward)(spec.feed_forward, tensors, dtype, device)

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward))

    @classmethod
    def tensor_needs(cls, spec):
        return (norm_class(spec.mixer_norm).tensor_needs(spec.mixer_norm) + mixer_class(spec.mixer).tensor_needs(spec.mixer) +
                norm_class(spec.feed_forward_norm).tensor_needs(spec.feed_forward_norm) +
                feed_forward_class(spec.feed_forward).tensor_needs(spec.feed_forward))

    @classmethod
    def cache_need(cls, spec):
        return mixer_class(spec.mixer).cache_need(spec.mixer)

    @staticmethod
    def _normed(norm, part, x, ctx):
        """The part's input: the normed rows, or the norm handed on unapplied if both sides can."""
        dtype = getattr(part, "in_dtype", ctx.dtype)
        if getattr(part, "accepts_deferred_norm", False) and hasattr(norm, "deferred"):
            return norm.deferred(x, dtype)
        return norm(x, dtype)

    # A part that adds onto the residual may do the next norm's share on the way (`HandedRows` in parts/norm.py), if that
    # norm can be applied so (`handed_weight`), its reader takes rows so normed (`takes_handed_norm`) and the part knows how
    # (`hands_norm_on`: its `forward` takes `then` and returns the handed rows, or None where its product could not).
    hands_norm_on = True

    def first_reader(self):
        """The norm that reads the residual first in this block, and the part that reads the normed rows."""
        return self.mixer_norm, self.mixer

    @staticmethod
    def _then(part, reader, n_rows):
        return norm_to_hand_on(reader, n_rows) if getattr(part, "hands_norm_on", False) else None

    def forward(self, x, ctx, cache, handed=None, next_reader=None):
        """handed: this block's first norm as whoever wrote x last left it, or None.  next_reader: `first_reader()` of whatever
        reads x after this block, or None.  Returns that reader's norm handed on, or None."""
        if handed is None or handed.norm is not self.mixer_norm:
            handed = self._normed(self.mixer_norm, self.mixer, x, ctx)
        then = self._then(self.mixer, (self.feed_forward_norm, self.feed_forward), ctx.n_rows)
        handed = self.mixer.forward(handed, x, ctx, cache) if then is None else self.mixer.forward(handed, x, ctx, cache, then=then)
        if ctx.trace is not None:
            ctx.trace("attn_out", x)
        if handed is None or then is None:
            handed = self._normed(self.feed_forward_norm, self.feed_forward, x, ctx)
        then = self._then(self.feed_forward, next_reader, ctx.n_rows)
        handed = self.feed_forward.forward(handed, x, ctx) if then is None else self.feed_forward.forward(handed, x, ctx, then=then)
        if ctx.trace is not None:
            ctx.trace("ffn_out", x)
        return handed if then is not None else None


register_block("prenorm", PreNormBlock)


class SandwichBlock:
    """x += post_1(mixer(norm_1(x))), then, if the layer has a feed-forward, x += post_2(feed_forward(norm_2(x))).  A half's
    result goes into rows of its own (a part that `can_overwrite` stores it there, any other part adds onto zeros), and the
    norm behind the half adds the normed rows onto x in one kernel where it is an RMS norm with weights."""

    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec
        build = lambda s: None if s is None else norm_class(s)(s, tensors, dtype, device)
        if spec.mixer_post_norm is None or (spec.feed_forward is not None and (spec.feed_forward_norm is None or spec.feed_forward_post_norm is None)):
            raise ValueError("a sandwich layer needs a norm before and behind each of its halves")
        self.mixer_norm, self.mixer_post_norm = build(spec.mixer_norm), build(spec.mixer_post_norm)
        self.mixer = mixer_class(spec.mixer)(spec.mixer, tensors, dtype, device)
        self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward_norm, self.feed_forward_post_norm = build(spec.feed_forward_norm), build(spec.feed_forward_post_norm)
            self.feed_forward = feed_forward_class(spec.feed_forward)(spec.feed_forward, tensors, dtype, device)

    def _parts(self):
        halves = [self.mixer_norm, self.mixer, self.mixer_post_norm]
        return halves + ([self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm] if self.feed_forward is not None else [])

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in self._parts())

    @classmethod
    def tensor_needs(cls, spec):
        needs = []
        for s in (spec.mixer_norm, spec.mixer_post_norm) + ((spec.feed_forward_norm, spec.feed_forward_post_norm) if spec.feed_forward is not None else ()):
            needs += norm_class(s).tensor_needs(s)
        needs += mixer_class(spec.mixer).tensor_needs(spec.mixer)
        if spec.feed_forward is not None:
            needs += feed_forward_class(spec.feed_forward).tensor_needs(spec.feed_forward)
        return needs

    @classmethod
    def cache_need(cls, spec):
        return mixer_class(spec.mixer).cache_need(spec.mixer)

    # The norm behind a half and the norm that reads the rows next (this layer's second, or the next layer's first, or the
    # model's last when every row's logits are wanted) run as one kernel where both are RMS norms with weights of one dtype:
    # the block plays the model's game of handing a norm on (`hands_norm_on`, `first_reader`, `handed`, `next_reader`).
    hands_norm_on = True

    def first_reader(self):
        return self.mixer_norm, self.mixer

    @staticmethod
    def _half(h, part, post, x, ctx, reader, *cache):
        """x += post(part(h)); returns the rows `reader` = (norm, part) will read, if they were made on the way, else None."""
        if isinstance(h, NormedRows) and not getattr(part, "accepts_deferred_norm", False):
            h = h.materialize()
        if getattr(part, "can_overwrite", False):
            y = torch.empty_like(x)
            part.forward(h, y, ctx, *cache, overwrite=True)
        else:
            y = torch.zeros_like(x)
            part.forward(h, y, ctx, *cache)
        then, reads = reader if reader is not None else (None, None)
        if (then is not None and hasattr(post, "add_onto_then") and type(then) is type(post) and then.weight.dtype == post.weight.dtype
                and then.weight.shape == post.weight.shape):
            return post.add_onto_then(y, x, then, getattr(reads, "in_dtype", ctx.dtype))
        if hasattr(post, "add_onto"):
            post.add_onto(y, x)
        else:
            x += post(y, torch.float32)
        return None

    def forward(self, x, ctx, cache, handed=None, next_reader=None):
        """handed: this block's first norm as whoever wrote x last left it (rows ready to read), or None.  next_reader:
        `first_reader()` of whatever reads x after this block, or None.  Returns that reader's rows, or None."""
        if handed is None or handed.norm is not self.mixer_norm:
            handed = PreNormBlock._normed(self.mixer_norm, self.mixer, x, ctx)
        inner = (self.feed_forward_norm, self.feed_forward) if self.feed_forward is not None else next_reader
        handed = self._half(handed, self.mixer, self.mixer_post_norm, x, ctx, inner, cache)
        if ctx.trace is not None:
            ctx.trace("attn_out", x)
        if self.feed_forward is not None:
            if handed is None:
                handed = PreNormBlock._normed(self.feed_forward_norm, self.feed_forward, x, ctx)
            handed = self._half(handed, self.feed_forward, self.feed_forward_post_norm, x, ctx, next_reader)
        if ctx.trace is not None:
            ctx.trace("ffn_out", x)
        return handed


register_block("sandwich", SandwichBlock)


class _Readers:
    """The parts that read one norm's rows, asked as one whether they take that norm half applied."""

    def __init__(self, parts, first_weight=None):
        self.parts, self.first_weight = parts, first_weight          # first_weight(n_rows): the one matrix all of them read at this number of rows, or None
        self.accepts_deferred_norm = all(getattr(p, "accepts_deferred_norm", False) for p in parts)
        dtypes = {getattr(p, "in_dtype", None) for p in parts}
        self.in_dtype = dtypes.pop() if len(dtypes) == 1 else None

    def takes_handed_norm(self, n_rows: int) -> bool:
        common = self.first_weight(n_rows) if self.first_weight is not None else None
        if common is not None:                    # (one product for all of them)
            return self.in_dtype == torch.bfloat16 and takes_handed_norm(common, n_rows)
        return self.in_dtype is not None and all(hasattr(p, "takes_handed_norm") and p.takes_handed_norm(n_rows) for p in self.parts)


class ParallelBlock:
    """x += mixer(h) + feed_forward(h) with h = norm_1(x): both halves read the same normed rows, which are made once, and each
    adds its result onto x (the two sums reach x one after the other; neither half reads x).  The block plays the game of
    handing a norm on (`hands_norm_on`, `first_reader`, `handed`, `next_reader`): the half that writes x last does the next
    norm's first share, and a norm so handed to this block is finished by the first products of both halves, where both can
    (asked beforehand: the second half must not fall back on rows that the first has changed by then)."""
    hands_norm_on = True
    STACK = True                     # the two halves' first products as one (off: each half makes its own)
    # ... in steps of up to so many rows and with both matrices together up to so many bytes: one launch less a layer where launches
    # are what a step costs (8 decoded rows, 8 layers: 0.563 -> 0.536 ms a step with 44 MB a layer); with 160 MB a layer the one product
    # took longer than the two (1.142 -> 1.169 ms), and so did it for the rows of prompts at both sizes (5.19 -> 5.28, 11.28 -> 11.37 ms).
    STACK_MAX_ROWS, STACK_MAX_BYTES = 128, 64 << 20

    def _stacked(self, n_rows: int):
        """The common matrix of both halves' first products, if a step of this many rows makes them as one; else None."""
        if self.w_first is None or n_rows > self.STACK_MAX_ROWS or self.w_first.numel() * self.w_first.element_size() > self.STACK_MAX_BYTES:
            return None
        return self.w_first

    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec
        if spec.feed_forward_norm is not None or spec.mixer_post_norm is not None or spec.feed_forward_post_norm is not None:
            raise ValueError("a parallel layer has one norm, before its mixer and its feed-forward")
        self.mixer_norm = norm_class(spec.mixer_norm)(spec.mixer_norm, tensors, dtype, device)
        self.mixer = mixer_class(spec.mixer)(spec.mixer, tensors, dtype, device)
        self.feed_forward = None if spec.feed_forward is None else feed_forward_class(spec.feed_forward)(spec.feed_forward, tensors, dtype, device)
        # Both halves begin with a product of the same rows: where both say which matrix that is (`input_weight`), the two are laid
        # one behind the other, the block makes one product of them and hands each half its columns (`projected=`); the halves keep
        # views of the common matrix, so nothing lies in memory twice.
        self.w_first, self._split = None, 0
        first = [getattr(p, "input_weight", lambda: None)() for p in (self.mixer, self.feed_forward)] if self.feed_forward is not None else []
        if (self.STACK and len(first) == 2 and all(w is not None for w in first) and first[0].dtype == first[1].dtype and first[0].shape[1] == first[1].shape[1]
                and getattr(self.mixer, "in_dtype", None) == getattr(self.feed_forward, "in_dtype", None)):
            self._split = first[0].shape[0]
            if (self._split * first[0].shape[1] * first[0].element_size()) % 16 == 0:          # (the second matrix starts as aligned as the first)
                self.w_first = torch.cat(first, dim=0).contiguous()
                self.mixer.use_input_weight(self.w_first[:self._split])
                self.feed_forward.use_input_weight(self.w_first[self._split:])
        self._readers = _Readers(self._parts()[1:], self._stacked)

    def _parts(self):
        return [self.mixer_norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in self._parts())

    @classmethod
    def tensor_needs(cls, spec):
        needs = norm_class(spec.mixer_norm).tensor_needs(spec.mixer_norm) + mixer_class(spec.mixer).tensor_needs(spec.mixer)
        if spec.feed_forward is not None:
            needs += feed_forward_class(spec.feed_forward).tensor_needs(spec.feed_forward)
        return needs

    @classmethod
    def cache_need(cls, spec):
        return mixer_class(spec.mixer).cache_need(spec.mixer)

    def first_reader(self):
        return self.mixer_norm, self._readers

    def forward(self, x, ctx, cache, handed=None, next_reader=None):
        """handed: this block's norm as whoever wrote x last left it (half applied), or None.  next_reader: `first_reader()` of
        whatever reads x after this block, or None.  Returns that reader's norm handed on, or None."""
        if handed is not None and handed.norm is self.mixer_norm and self._readers.takes_handed_norm(ctx.n_rows):
            rows = lambda part: handed
        elif self._readers.in_dtype is not None:      # one set of normed rows serves both halves
            h = self.mixer_norm(x, self._readers.in_dtype)
            rows = lambda part: h
        else:
            made = {part: self.mixer_norm(x, getattr(part, "in_dtype", ctx.dtype)) for part in self._parts()[1:]}      # (before anything changes x)
            rows = made.__getitem__
        last = self.feed_forward if self.feed_forward is not None else self.mixer
        then = norm_to_hand_on(next_reader, ctx.n_rows) if getattr(last, "hands_norm_on", False) else None
        own = [{}, {}]                            # what each half is told beyond its rows
        w_first = self._stacked(ctx.n_rows)
        if w_first is not None:
            both = torch.empty((ctx.n_rows, w_first.shape[0]), dtype=torch.float32, device=x.device)
            linear(rows(self.mixer), w_first, both)
            own[0]["projected"], own[1]["projected"] = both[:, :self._split], both[:, self._split:]
        if then is not None:
            own[0 if last is self.mixer else 1]["then"] = then
        out = self.mixer.forward(rows(self.mixer), x, ctx, cache, **own[0])
        if ctx.trace is not None:
            ctx.trace("attn_out", x)
        if self.feed_forward is not None:
            out = self.feed_forward.forward(rows(self.feed_forward), x, ctx, **own[1])
        if ctx.trace is not None:
            ctx.trace("ffn_out", x)
        return out if then is not None else None


register_block("parallel", ParallelBlock)
