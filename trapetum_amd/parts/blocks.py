"""How a layer's parts are arranged around the residual stream.

sandwich  x += post_mixer_norm(mixer(pre_mixer_norm(x)));
          x += post_ff_norm(ff(pre_ff_norm(x)))          (runtime/src/lib.rs:4527-4540)
pre_norm  x += mixer(pre_mixer_norm(x));  x += ff(pre_ff_norm(x))
          (the reference's other layer type, runtime/src/lib.rs:721-730)

The stream is fp32 and the sum is formed in fp32 (the reference adds in fp32 and
stores fp16: runtime/cuda/codebook_gemv.cu:539-542).  Where a norm of a sub-layer's
output is followed by the add and by the next norm, one kernel does all three; that
includes the first norm of the block that runs next (`next_norm`), whose result the
next block receives as `normed`.
"""
from ..registry import register_part
from .base import Block


def add_then_norm(ctx, stream, rows, post, nxt):
    """stream += post(rows) (or rows); returns nxt(stream) (or None).  One kernel when both norms
    expose an RMS gain, else the norms' own forward around a plain add."""
    fusable = all(n is None or n.gain is not None for n in (post, nxt))
    if fusable:
        return ctx.ops.add_rms_norm(stream, rows,
                                    post.gain if post else None, post.eps if post else 0.0,
                                    nxt.gain if nxt else None, nxt.eps if nxt else 0.0, ctx.dtype)
    rows = ctx.ops.rows(rows, ctx.dtype)
    if post is not None:
        rows = post.forward(ctx, rows)
    ctx.ops.add_rms_norm(stream, rows, None, 0.0, None, 0.0, ctx.dtype)
    return nxt.forward(ctx, stream) if nxt is not None else None


class SandwichBlock(Block):
    @classmethod
    def norm_sites(cls):
        return ("pre_mixer_norm", "post_mixer_norm", "pre_ff_norm", "post_ff_norm")

    def entry_norm(self):
        return self.norms["pre_mixer_norm"]

    def forward(self, ctx, stream, site, normed=None, next_norm=None):
        n = self.norms
        x = normed if normed is not None else n["pre_mixer_norm"].forward(ctx, stream)
        ctx.dump("mixer_in", x)
        a = self.mixer.forward(ctx, x, site)
        ctx.dump("mixer_out", a)
        x = add_then_norm(ctx, stream, a, n["post_mixer_norm"], n["pre_ff_norm"])
        ctx.dump("after_mixer", stream)
        m = self.feed_forward.forward(ctx, x)
        ctx.dump("ff_out", m)
        normed_next = add_then_norm(ctx, stream, m, n["post_ff_norm"], next_norm)
        ctx.dump("layer_out", stream)
        return stream, normed_next


class PreNormBlock(Block):
    @classmethod
    def norm_sites(cls):
        return ("pre_mixer_norm", "pre_ff_norm")

    def entry_norm(self):
        return self.norms["pre_mixer_norm"]

    def forward(self, ctx, stream, site, normed=None, next_norm=None):
        n = self.norms
        x = normed if normed is not None else n["pre_mixer_norm"].forward(ctx, stream)
        ctx.dump("mixer_in", x)
        a = self.mixer.forward(ctx, x, site)
        ctx.dump("mixer_out", a)
        x = add_then_norm(ctx, stream, a, None, n["pre_ff_norm"])
        ctx.dump("after_mixer", stream)
        m = self.feed_forward.forward(ctx, x)
        ctx.dump("ff_out", m)
        normed_next = add_then_norm(ctx, stream, m, None, next_norm)
        ctx.dump("layer_out", stream)
        return stream, normed_next


register_part("block", "sandwich", SandwichBlock)
register_part("block", "pre_norm", PreNormBlock)
