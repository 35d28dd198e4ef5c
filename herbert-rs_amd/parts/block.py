"""How a layer's parts are arranged.

"parallel": with h = norm(x), x += mult * (mixer(h) + feed_forward(h)): one norm, both parts read it,
and their sum joins the residual stream times a constant.

"postnorm": x <- norm_post_mixer(alpha x + mixer(x)); x <- norm_post_ff(alpha x + feed_forward(x)): the parts
take x as it is, and each norm comes after its sum.

"prenorm": x += mixer(norm_input(x)); x += feed_forward(norm_post_mixer(x)), the
arrangement of the reference's two-norm layer
(crates/backends/backend_common/src/generic_layer.rs:1149-1151, 1234-1236,
1246-1248, 1272-1274).
"""
import torch

from ..kernels import ops
from .base import Part
from .registry import register


@register("block", "prenorm")
class PreNormBlock(Part):
    graph_safe = True

    norm_roles = ("input", "post_mixer")

    def __init__(self, mixer, feed_forward, norms):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        missing = [r for r in self.norm_roles if r not in norms]
        if missing:
            raise ValueError(f"prenorm block needs norms {missing}")

    def parts(self):
        return [self.norms["input"], self.mixer, self.norms["post_mixer"], self.feed_forward]

    def first_norm(self):
        """The norm that the residual stream meets first in this block."""
        return self.norms["input"]

    def forward(self, ctx, x):
        after = ctx.norm_after_block
        self._run(ctx, x, self.norms["input"], self.mixer, (self.norms["post_mixer"], ctx.entry))
        self._run(ctx, x, self.norms["post_mixer"], self.feed_forward, after)

    @staticmethod
    def _run(ctx, x, norm, part, ahead):
        """part(norm(x)) added to x. A part may offer forward_from_residual(ctx, x, norm), which
        returns True if it has done the norm itself inside its first kernel, or has used what the
        part before left of it (ctx.handed). `ahead` is (the norm that x meets next, its entry)."""
        left, ctx.left = ctx.left, None
        valid = (left is not None and left.norm is norm and left.entry == ctx.entry
                 and left.x.data_ptr() == x.data_ptr() and left.x.shape == x.shape)
        ctx.norm_ahead = ahead
        if valid and left.squares is None:          # the product before has normed the rows as well
            ctx.handed = None
            part.forward(ctx, left.xg, x)
            return
        ctx.handed = left if valid else None
        fused = getattr(part, "forward_from_residual", None)
        if fused is not None and fused(ctx, x, norm):
            return
        ctx.handed = None
        part.forward(ctx, norm.forward(ctx, x), x)


@register("block", "parallel")
class ParallelBlock(Part):
    """x <- x + mult * (mixer(h) + feed_forward(h)) with h = norm(x). The parts add their outputs, as they
    always do, to float32 rows of their own (cleared first) instead of to x. Where the next layer is such
    a block with a norm that can take a sum on, the sum is left for that norm's kernel, which adds it to x
    and norms the result in one pass; otherwise it is added here."""
    graph_safe = True

    norm_roles = ("input",)

    def __init__(self, mixer, feed_forward, norms, mult=1.0, fuse_sum=True):
        self.mixer = mixer
        self.feed_forward = feed_forward
        if "input" not in norms:
            raise ValueError("parallel block needs the norm 'input'")
        self.norm = norms["input"]
        self.mult = float(mult)
        self.fuse_sum = bool(fuse_sum)

    def parts(self):
        return [self.norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    def first_norm(self):
        return self.norm

    def takes_sum(self):
        """True if this block's norm adds a sum that the block before left (ctx.pending_sum)."""
        return self.fuse_sum and getattr(self.norm, "adds_sum", False)

    def forward(self, ctx, x):
        pending, ctx.pending_sum = ctx.pending_sum, None
        if pending is not None and pending[0].data_ptr() == x.data_ptr() and self.takes_sum():
            h = self.norm.forward(ctx, x, delta=pending[1], mult=pending[2])
        else:
            if pending is not None:
                ops.layernorm_free_sum(x, pending[1], pending[2])
            h = self.norm.forward(ctx, x)
        # the two parts' outputs meet in rows of their own (free again: the norm above has taken the sum
        # of the layer before)
        total = ctx.rt.buffer("parallel_sum", tuple(x.shape), torch.float32)
        ctx.handed = ctx.norm_ahead = None
        # a mixer that can store its rows instead of adding them says so (`stores_fresh_rows`) and finds the
        # rows in ctx.fresh_rows; for any other the rows are cleared first
        if getattr(self.mixer, "stores_fresh_rows", False):
            ctx.fresh_rows = total
        else:
            ops.fill_u32(total, 0)
        self.mixer.forward(ctx, h, total)
        ctx.fresh_rows = None
        if self.feed_forward is not None:
            self.feed_forward.forward(ctx, h, total)
        nxt = ctx.next_block
        if isinstance(nxt, ParallelBlock) and nxt.takes_sum():
            ctx.pending_sum = (x, total, self.mult)
        else:
            ops.layernorm_free_sum(x, total, self.mult)


@register("block", "postnorm")
class PostNormBlock(Part):
    """x <- norm_post_mixer(alpha x + mixer(x)), then x <- norm_post_ff(alpha x + feed_forward(x)) (the second
    step only where the layer has a feed-forward). The parts take x as it is, in the compute dtype, and add
    their outputs, as they always do, to float32 rows: rows that already hold alpha x. One kernel between
    two parts norms those rows into x, writes the copy that the next part reads and alpha x where it adds;
    the one after a layer's last part does so for the next layer too, if that is such a block."""
    graph_safe = True

    norm_roles = ("post_mixer", "post_ff")

    def __init__(self, mixer, feed_forward, norms, alpha=1.0):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.alpha = float(alpha)
        missing = [r for r in self.norm_roles[:1 if feed_forward is None else 2] if r not in norms]
        if missing:
            raise ValueError(f"postnorm block needs norms {missing}")
        if self.alpha == 0.0:
            raise ValueError("postnorm block: alpha must not be zero")
        for role in self.norm_roles:
            if role in norms and not getattr(norms[role], "hands_on", False):
                raise ValueError("postnorm block: its norms are of the form x * w / rms(x)")

    def parts(self):
        parts = [self.mixer, self.norms["post_mixer"]]
        if self.feed_forward is not None:
            parts += [self.feed_forward, self.norms["post_ff"]]
        return parts

    def forward(self, ctx, x):
        rt = ctx.rt
        shape = tuple(x.shape)
        acc = rt.buffer("postnorm_sum", shape, torch.float32)
        y = None if rt.exact else rt.buffer("postnorm_rows", shape)       # (float32: the parts take x as it is)
        pending, ctx.pending_post = ctx.pending_post, None
        if pending != (x.data_ptr(), self.alpha):
            ops.postnorm(x, None, None, y, 0.0, self.alpha, acc=acc)
        nxt = ctx.next_block
        alpha_after = nxt.alpha if isinstance(nxt, PostNormBlock) else 0.0
        steps = [(self.mixer, self.norms["post_mixer"])]
        if self.feed_forward is not None:
            steps.append((self.feed_forward, self.norms["post_ff"]))
        for i, (part, norm) in enumerate(steps):
            ctx.handed = ctx.norm_ahead = ctx.left = ctx.fresh_rows = None
            part.forward(ctx, x if y is None else y, acc)
            last = i + 1 == len(steps)
            ops.postnorm(acc, norm.w, x, None if last and alpha_after == 0.0 else y, norm.eps,
                         alpha_after if last else self.alpha)
        if alpha_after != 0.0:
            ctx.pending_post = (x.data_ptr(), alpha_after)
