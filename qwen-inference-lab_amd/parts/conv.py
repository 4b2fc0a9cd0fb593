"""A short causal convolution over time on every channel, added to its input."""
from .base import Part, ParamSpec, StateNeed
from .. import ops


class ShortConvolution(Part):
    """h_t = x_t + sum_(j < taps) w[:, j] * x_(t - taps + 1 + j), zeros before a sequence's start; ``weight``
    [width, taps], no bias.  It reads the float32 residual stream and computes in float32; the result is rounded once
    to the type the consumer's products read.  The last taps - 1 inputs of a sequence are its state between steps:
    ``cache_need()`` is a ``StateNeed`` of [taps - 1, width] float32 (None for a single tap), and ``forward`` gets the
    ``StateView`` of the schedule entry.  ``finalize`` turns the stored weight to [taps, width], a tap's factors side
    by side, which is how the kernel reads them."""

    def __init__(self, width, taps):
        super().__init__()
        if type(taps) is not int or taps < 1:
            raise ops.UnsupportedShape(f'taps must be a positive integer, not {taps!r}')
        self.width, self.taps = int(width), taps

    def param_specs(self):
        return {'weight': ParamSpec((self.width, self.taps), 'vector', 'normal')}

    def cache_need(self):
        return StateNeed((self.taps - 1, self.width), 'float32') if self.taps > 1 else None

    def finalize(self):
        self.p['weight'] = self.p['weight'].t().contiguous()

    def forward(self, stream, ctx, cache, out_dtype):
        return ops.short_conv(stream, self.p['weight'], state=cache.state if cache is not None else None,
                              cu_seqlens=ctx.cu_seqlens, seq_starts=ctx.seq_starts, seq_slots=ctx.seq_slots,
                              row_seq=ctx.row_seq, n_seqs=ctx.n_seqs, out_dtype=out_dtype)
