from __future__ import annotations

from typing import Dict

import torch

from ..config.specs import (ParallelBlockSpec, PostNormBlockSpec, PreNormBlockSpec,
                            SandwichNormBlockSpec, StreamBlockSpec)
from ..errors import ConfigError
from .base import Block, TensorDecl, build_part, register_part
from .linear import place_gain


class PreNormBlock(Block):
    """x += mixer(norm(x)); x += feed_forward(norm(x)): the residual is the un-normed input
    (`src/model/runtime/optimized_decoder/layer.zig:108,188-201`).  The residual stream ``x``
    is float32; both sums happen in 32-bit inside the parts."""

    def __init__(self, spec: PreNormBlockSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx, prefix + spec.mixer_norm_prefix)
        self.mixer = build_part("mixer", spec.mixer, ctx, prefix + spec.mixer_prefix)
        self.ff_norm = build_part("norm", spec.ff_norm, ctx, prefix + spec.ff_norm_prefix)
        self.feed_forward = build_part("feed_forward", spec.feed_forward, ctx,
                                       prefix + spec.ff_prefix)
        self.parts = (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)
        # the norm that reads the residual stream first, if what a sum leaves for it is of use
        self.entry_norm = self._lazy(self.mixer_norm, self.mixer)
        self.graph_safe = all(p.graph_safe for p in self.parts)
        self.kernel_modules = tuple(sorted({m for p in self.parts for m in p.kernel_modules}))

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)

    def cache_need(self):
        return self.mixer.cache_need()

    def accept_cache(self, cache) -> None:
        self.mixer.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def _normed(self, norm, consumer, x, step):
        """The consumer's input: the normed activations, or, for a consumer that says it can
        take a norm that has not run, the norm's stand-in (``Norm.deferred``)."""
        make = lambda: step.scratch("normed", x.shape, self.ctx.act_dtype)
        left, step.norm_ready, step.norm_after = step.norm_ready, None, None
        if getattr(consumer, "accepts_lazy_norm", False):
            lazy = norm.deferred(x, make, left)
            if lazy is not None:
                return lazy
        return norm.forward(x, make())

    def _lazy(self, norm, consumer):
        """``norm`` if its reader takes a norm that has not run (and so what a residual sum
        leaves for it), else None."""
        return norm if norm.defers and getattr(consumer, "accepts_lazy_norm", False) else None

    def forward(self, x, step, cache) -> None:
        after_block = step.norm_after_block
        h = self._normed(self.mixer_norm, self.mixer, x, step)
        step.norm_after = self._lazy(self.ff_norm, self.feed_forward)
        self.mixer.forward(h, x, step, cache)
        h = self._normed(self.ff_norm, self.feed_forward, x, step)
        step.norm_after = after_block
        self.feed_forward.forward(h, x, step)
        step.norm_after = None


class SandwichNormBlock(Block):
    """x += post1(mixer(norm1(x))); x += post2(ff(norm2(x))): a norm before every sublayer and
    one behind it, ahead of the residual sum.  A sublayer's output is a float32 branch of its
    own (a part that says ``stores_output`` stores it there; any other part adds it to a
    branch that was cleared first); the norm behind it reads the branch and adds its result to
    the stream in one kernel, in 32-bit.  Without a feed-forward the block is its first line."""

    def __init__(self, spec: SandwichNormBlockSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx, prefix + spec.mixer_norm_prefix)
        self.mixer = build_part("mixer", spec.mixer, ctx, prefix + spec.mixer_prefix)
        self.mixer_post_norm = build_part("norm", spec.mixer_post_norm, ctx,
                                          prefix + spec.mixer_post_norm_prefix)
        self.parts = [self.mixer_norm, self.mixer, self.mixer_post_norm]
        self.feed_forward = self.ff_norm = self.ff_post_norm = None
        if spec.feed_forward is not None:
            self.ff_norm = build_part("norm", spec.ff_norm, ctx, prefix + spec.ff_norm_prefix)
            self.feed_forward = build_part("feed_forward", spec.feed_forward, ctx,
                                           prefix + spec.ff_prefix)
            self.ff_post_norm = build_part("norm", spec.ff_post_norm, ctx,
                                           prefix + spec.ff_post_norm_prefix)
            self.parts += [self.ff_norm, self.feed_forward, self.ff_post_norm]
        self.parts = tuple(self.parts)
        # the norm that reads the stream first: the block before may already have run it, in
        # the kernel of its own last norm (``NormedRows`` in ``step.norm_ready``)
        self.entry_norm = self.mixer_norm
        self.graph_safe = all(p.graph_safe for p in self.parts)
        self.kernel_modules = tuple(sorted({m for p in self.parts for m in p.kernel_modules}))

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)

    def cache_need(self):
        return self.mixer.cache_need()

    def accept_cache(self, cache) -> None:
        self.mixer.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def _sublayer(self, norm, part, post, x, step, args, then, ready):
        """One sublayer; ``args``: what the part takes behind the step (a mixer its cache).
        ``ready``: the rows ``norm`` would give, if whoever summed into the
        stream last has run it already.  ``then``: the norm that reads the stream next; if the
        closing norm's kernel can run it too, its rows come back (else None)."""
        if ready is not None:
            h = ready
        else:
            h = norm.forward(x, step.scratch("normed", x.shape, self.ctx.act_dtype))
        branch = step.scratch("branch", x.shape, torch.float32)
        if getattr(part, "stores_output", False):
            part.forward(h, branch, step, *args, accumulate=False)
        else:
            branch.zero_()
            part.forward(h, branch, step, *args)
        step.norm_ready = None
        fused = getattr(post, "forward_add_then", None)
        if then is not None and fused is not None:
            # (the mixer or feed-forward is done with the buffer its input lay in)
            out = step.scratch("normed", x.shape, self.ctx.act_dtype)
            if fused(branch, x, then, out):
                return out
        post.forward_add(branch, x)
        return None

    def forward(self, x, step, cache) -> None:
        after_block = step.norm_after_block
        left, step.norm_ready, step.norm_after = step.norm_ready, None, None
        ready = left.normed if isinstance(left, NormedRows) and left.fits(self.mixer_norm, x) \
            else None
        then = self.ff_norm if self.feed_forward is not None else after_block
        h = self._sublayer(self.mixer_norm, self.mixer, self.mixer_post_norm, x, step,
                           (cache,), then, ready)
        if self.feed_forward is not None:
            h = self._sublayer(self.ff_norm, self.feed_forward, self.ff_post_norm, x, step, (),
                               after_block, h)
        step.norm_after = None
        # what the next block's first norm would compute is there already
        step.norm_ready = NormedRows(after_block, x, h) if h is not None else None


class NormedRows:
    """The rows ``normed`` = ``norm(x)`` that a block's last kernel already made for the norm
    that reads the stream next."""

    def __init__(self, norm, x: torch.Tensor, normed: torch.Tensor):
        self.norm, self.x, self.normed = norm, x, normed

    def fits(self, norm, x: torch.Tensor) -> bool:
        return self.norm is norm and self.x.data_ptr() == x.data_ptr() and self.x.shape == x.shape


class StreamRows:
    """The residual rows ``x`` in the activations' type, left by the kernel that last added
    into them for a sublayer that reads the stream as it is."""

    def __init__(self, x: torch.Tensor, rows: torch.Tensor):
        self.x, self.rows = x, rows

    def fits(self, x: torch.Tensor) -> bool:
        return self.x.data_ptr() == x.data_ptr() and self.x.shape == x.shape


class PostNormBlock(Block):
    """x += norm1(mixer(x)); x += norm2(ff(x)): the sublayers read the stream itself, and each
    one's output goes through a norm before it joins the stream.  A sublayer stores its output
    in a float32 branch; the norm behind it reads the branch and adds its result to the stream
    in 32-bit, and the same kernel leaves the sum in the type the next sublayer's products take
    (``StreamRows``, handed across the layer's edge in ``step.norm_ready``).  In a 32-bit build
    the sublayers read the stream's own rows.  Without a feed-forward the block is its first
    line."""

    def __init__(self, spec: PostNormBlockSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.mixer = build_part("mixer", spec.mixer, ctx, prefix + spec.mixer_prefix)
        self.mixer_post_norm = build_part("norm", spec.mixer_post_norm, ctx,
                                          prefix + spec.mixer_post_norm_prefix)
        self.parts = [self.mixer, self.mixer_post_norm]
        self.feed_forward = self.ff_post_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = build_part("feed_forward", spec.feed_forward, ctx,
                                           prefix + spec.ff_prefix)
            self.ff_post_norm = build_part("norm", spec.ff_post_norm, ctx,
                                           prefix + spec.ff_post_norm_prefix)
            self.parts += [self.feed_forward, self.ff_post_norm]
        self.parts = tuple(self.parts)
        self.graph_safe = all(p.graph_safe for p in self.parts)
        # (the cast of the stream's rows is the elementwise module's)
        self.kernel_modules = tuple(sorted({"elementwise"}
                                           | {m for p in self.parts for m in p.kernel_modules}))

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)

    def cache_need(self):
        return self.mixer.cache_need()

    def accept_cache(self, cache) -> None:
        self.mixer.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def _rows(self, x, step):
        """The stream's rows as a sublayer's products take them."""
        if self.ctx.act_dtype == torch.float32:
            return x
        from .. import ops
        rows = step.scratch("stream_rows", x.shape, self.ctx.act_dtype)
        ops.cast(x, rows)
        return rows

    def _sublayer(self, part, post, x, h, step, args):
        """One sublayer on the rows ``h`` of the stream ``x``; returns the rows of the new
        stream if the closing norm's kernel left them, else None."""
        branch = step.scratch("branch", x.shape, torch.float32)
        if getattr(part, "stores_output", False):
            part.forward(h, branch, step, *args, accumulate=False)
        else:
            branch.zero_()
            part.forward(h, branch, step, *args)
        step.norm_ready = None
        fused = getattr(post, "forward_add_store", None)
        if self.ctx.act_dtype != torch.float32 and fused is not None:
            # (the sublayer is done with the buffer its input lay in)
            out = step.scratch("stream_rows", x.shape, self.ctx.act_dtype)
            if fused(branch, x, out):
                return out
        post.forward_add(branch, x)
        return None

    def forward(self, x, step, cache) -> None:
        left, step.norm_ready, step.norm_after = step.norm_ready, None, None
        h = left.rows if isinstance(left, StreamRows) and left.fits(x) else self._rows(x, step)
        h = self._sublayer(self.mixer, self.mixer_post_norm, x, h, step, (cache,))
        if self.feed_forward is not None:
            if h is None:
                h = self._rows(x, step)
            h = self._sublayer(self.feed_forward, self.ff_post_norm, x, h, step, ())
        step.norm_after = None
        step.norm_ready = StreamRows(x, h) if h is not None else None


class ParallelBlock(Block):
    """x += mixer(norm1(x)) + feed_forward(norm2(x)): both norms read the stream before either
    sublayer has added to it; the sublayers then add their outputs into the stream one after
    the other, in 32-bit.  Without a feed-forward the block is its mixer's line."""

    def __init__(self, spec: ParallelBlockSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx, prefix + spec.mixer_norm_prefix)
        self.mixer = build_part("mixer", spec.mixer, ctx, prefix + spec.mixer_prefix)
        self.parts = [self.mixer_norm, self.mixer]
        self.ff_norm = self.feed_forward = None
        if spec.feed_forward is not None:
            self.ff_norm = build_part("norm", spec.ff_norm, ctx, prefix + spec.ff_norm_prefix)
            self.feed_forward = build_part("feed_forward", spec.feed_forward, ctx,
                                           prefix + spec.ff_prefix)
            self.parts += [self.ff_norm, self.feed_forward]
        self.parts = tuple(self.parts)
        self.graph_safe = all(p.graph_safe for p in self.parts)
        self.kernel_modules = tuple(sorted({m for p in self.parts for m in p.kernel_modules}))

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)

    def cache_need(self):
        return self.mixer.cache_need()

    def accept_cache(self, cache) -> None:
        self.mixer.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def forward(self, x, step, cache) -> None:
        step.norm_ready = step.norm_after = None
        h1 = self.mixer_norm.forward(x, step.scratch("normed", x.shape, self.ctx.act_dtype))
        h2 = None
        if self.feed_forward is not None:
            # (before the mixer adds into the stream: both sublayers read the same rows)
            h2 = self.ff_norm.forward(x, step.scratch("normed_ff", x.shape, self.ctx.act_dtype))
        self.mixer.forward(h1, x, step, cache)
        if self.feed_forward is not None:
            self.feed_forward.forward(h2, x, step)
        step.norm_ready = step.norm_after = None


class StreamRead:
    """What the kernel that last wrote the copies ``x`` of the stream left for the block that
    reads them next: the rows ``normed`` its first sublayer takes."""

    def __init__(self, block, x: torch.Tensor, normed: torch.Tensor):
        self.block, self.x, self.normed = block, x, normed

    def fits(self, block, x: torch.Tensor) -> bool:
        return self.block is block and self.x.data_ptr() == x.data_ptr() \
            and self.x.shape == x.shape


class StreamBlock(Block):
    """A layer over several copies of the residual stream (``StreamBlockSpec``): x is float32
    [S, T, W] (or [T, W] for one copy).  One kernel a sublayer: it lets the sublayer before join
    every copy (the copies mixed among themselves, the output added with a weight a copy) and
    forms the next sublayer's input, the weighted sum of the new copies through the norm.  That
    holds across layers too: the last kernel of a block already reads for the block behind it
    (``StreamRead`` in ``step.norm_ready``), which the decoder names in
    ``step.norm_after_block``.  A sublayer stores its output in a float32 branch; a mixer that
    is two side by side may bring two branches with a factor each (``forward_branches``), which
    the same kernel adds.  The norms' work is done by that kernel: they must be RMS norms
    without a bias (``LayerNormSpec`` not centred)."""

    def __init__(self, spec: StreamBlockSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        from .. import ops
        if not 1 <= spec.streams <= ops.STREAMS_MAX:
            raise ConfigError(f"streams={spec.streams}: 1 to {ops.STREAMS_MAX} copies of the "
                              "residual stream")
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx, prefix + spec.mixer_norm_prefix)
        self.mixer = build_part("mixer", spec.mixer, ctx, prefix + spec.mixer_prefix)
        self.parts = [self.mixer_norm, self.mixer]
        self.ff_norm = self.feed_forward = None
        if spec.feed_forward is not None:
            self.ff_norm = build_part("norm", spec.ff_norm, ctx, prefix + spec.ff_norm_prefix)
            self.feed_forward = build_part("feed_forward", spec.feed_forward, ctx,
                                           prefix + spec.ff_prefix)
            self.parts += [self.ff_norm, self.feed_forward]
        self.parts = tuple(self.parts)
        for norm in (self.mixer_norm, self.ff_norm):
            ns = getattr(norm, "spec", None)
            if norm is not None and (getattr(ns, "centred", True) or
                                     getattr(ns, "bias_name", "") is not None):
                raise ConfigError("the norms of a layer over several copies of the stream are "
                                  "RMS norms without a bias")
        # the block that runs before this one may read the copies for it
        self.entry_norm = self
        self.defers = False
        self.graph_safe = all(p.graph_safe for p in self.parts)
        self.kernel_modules = tuple(sorted({"norms"}
                                           | {m for p in self.parts for m in p.kernel_modules}))

    def _coef_names(self, c: int):
        s = self.spec
        base = self.prefix + s.coef_prefix.format(c)
        return base + s.in_name, base + s.mix_name, base + s.out_name

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        S = self.spec.streams
        if self.spec.learned:
            for c in (1, 2) if self.feed_forward is not None else (1,):
                a, m, b = self._coef_names(c)
                d[a] = TensorDecl((S,), init="gain")
                d[m] = TensorDecl((S, S))
                d[b] = TensorDecl((S,), init="gain")
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)
        S = self.spec.streams
        self.coefs = []
        for c in (1, 2) if self.feed_forward is not None else (1,):
            if self.spec.learned:
                a, m, b = (place_gain(tensors[n], self.ctx) for n in self._coef_names(c))
            else:
                a, b = (place_gain(torch.ones(S), self.ctx) for _ in range(2))
                m = place_gain(torch.eye(S), self.ctx)
            self.coefs.append((a, m, b))

    def cache_need(self):
        return self.mixer.cache_need()

    def accept_cache(self, cache) -> None:
        self.mixer.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def read_args(self, c: int = 0):
        """What the kernel that reads the copies for sublayer ``c`` needs."""
        norm = self.mixer_norm if c == 0 else self.ff_norm
        return dict(in_coef=self.coefs[c][0], gain=norm.gain, eps=float(norm.spec.eps))

    def _run(self, part, h, step, args):
        """The sublayer's output as [(float32 branch, factor)]."""
        branches = getattr(part, "forward_branches", None)
        if branches is not None:
            return branches(h, step, *args)
        y = step.scratch("branch", h.shape, torch.float32)
        if getattr(part, "stores_output", False):
            part.forward(h, y, step, *args, accumulate=False)
        else:
            y.zero_()
            part.forward(h, y, step, *args)
        return [(y, 1.0)]

    def forward(self, x, step, cache) -> None:
        from .. import ops
        xs = x if x.dim() == 3 else x.unsqueeze(0)
        T, W = xs.shape[1], xs.shape[2]
        act = self.ctx.act_dtype
        after = step.norm_after_block
        left, step.norm_ready, step.norm_after = step.norm_ready, None, None
        if isinstance(left, StreamRead) and left.fits(self, x):
            h = left.normed
        else:
            h = step.scratch("normed", (T, W), act)
            ops.streams_step(xs, read=True, out=h, **self.read_args(0))
        sublayers = [(self.mixer, (cache,))]
        if self.feed_forward is not None:
            sublayers.append((self.feed_forward, ()))
        handed = None
        for c, (part, args) in enumerate(sublayers):
            branches = self._run(part, h, step, args)
            _, mix, out_coef = self.coefs[c]
            if c + 1 < len(sublayers):
                reader = self.read_args(c + 1)
            else:
                reader = after.read_args(0) if isinstance(after, StreamBlock) else None
            if reader is not None:
                # (the sublayer is done with the buffer its input lay in)
                h = step.scratch("normed_ff" if c % 2 == 0 else "normed", (T, W), act)
                ops.streams_step(xs, branches, mix, out_coef, read=True, out=h, **reader)
                if c + 1 == len(sublayers):
                    handed = StreamRead(after, x, h)
            else:
                ops.streams_step(xs, branches, mix, out_coef)
        step.norm_after = None
        step.norm_ready = handed


register_part("block", StreamBlockSpec, StreamBlock)
register_part("block", ParallelBlockSpec, ParallelBlock)
register_part("block", PostNormBlockSpec, PostNormBlock)
register_part("block", PreNormBlockSpec, PreNormBlock)
register_part("block", SandwichNormBlockSpec, SandwichNormBlock)
