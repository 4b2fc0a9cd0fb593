"""A selective state-space mixer: a short convolution, then a recurrence whose step size and input and output maps
depend on the token."""
import torch

from .base import Mixer, ParamSpec, StateNeed, CompoundNeed
from .. import ops


class SelectiveScan(Mixer):
    """With h the mixer's input, ``inner`` channels and ``state`` numbers per channel:

        [x | z] = W_in h;   u = silu(conv(x) + b_conv)       (causal, per channel, ``taps`` taps, zeros before the start)
        [low | B | C] = W_x u;   dt = softplus(W_dt low + b_dt)
        S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c u_c B_n;   y_c = sum_n S[c, n] C_n + D_c u_c
        result = W_o (y * silu(z))

    with A = -exp(A_log).  The projections and the convolution with its activation run in the model's type; the step
    size from the softplus on, the decays, the state and everything that touches it are float32.  A request keeps two
    things between steps, each in a slot of its own kind: the convolution's last ``taps - 1`` inputs and the state S
    [inner, state] (``cache_need`` is a ``CompoundNeed`` of two ``StateNeed``; one when there is a single tap).  A
    sequence that begins (``seq_starts`` 0) starts from zeros whatever its slot holds.

    ``finalize`` splits W_x into the rows that make ``low`` and those that make B and C (two products read u), turns
    the convolution's weight to [taps, inner] and makes A once, in float32.
    """
    graph_safe = True

    def __init__(self, *, width, inner, state, taps, dt_rank, dtype=torch.bfloat16):
        super().__init__()
        for name, value in (('inner', inner), ('state', state), ('taps', taps), ('dt_rank', dt_rank)):
            if type(value) is not int or value < 1:
                raise ops.UnsupportedShape(f'{name} must be a positive integer, not {value!r}')
        self.width, self.inner, self.state, self.taps, self.dt_rank, self.dtype = int(width), inner, state, taps, dt_rank, dtype
        ops.check_selective_scan_geometry(inner=inner, state=state, taps=taps)

    def param_specs(self):
        i, n, r = self.inner, self.state, self.dt_rank
        return {'in_proj.weight': ParamSpec((2 * i, self.width)),
                'conv.weight': ParamSpec((i, self.taps), 'vector'), 'conv.bias': ParamSpec((i,), 'vector'),
                'x_proj.weight': ParamSpec((r + 2 * n, i)),
                'dt_proj.weight': ParamSpec((i, r)), 'dt_proj.bias': ParamSpec((i,), 'vector'),
                'A_log': ParamSpec((i, n), 'vector'), 'D': ParamSpec((i,), 'vector', 'one_plus_normal'),
                'o_proj.weight': ParamSpec((self.width, i))}

    def cache_need(self):
        scan = StateNeed((self.inner, self.state), 'float32')
        if self.taps == 1:
            return scan
        return CompoundNeed((StateNeed((self.taps - 1, self.inner), 'float32'), scan))

    def finalize(self):
        p = self.p
        x_proj = p.pop('x_proj.weight')
        p['low_proj.weight'] = x_proj[:self.dt_rank].contiguous()
        p['bc_proj.weight'] = x_proj[self.dt_rank:].contiguous()
        p['conv.weight'] = p['conv.weight'].t().contiguous()
        p['A'] = (-torch.exp(p.pop('A_log').to(torch.float32))).contiguous()

    def forward(self, h, ctx, cache):
        p = self.p
        conv_cache, scan_cache = (None, cache) if self.taps == 1 else cache
        sequences = dict(cu_seqlens=ctx.cu_seqlens, seq_starts=ctx.seq_starts, seq_slots=ctx.seq_slots, n_seqs=ctx.n_seqs)
        xz = ops.linear(h, p['in_proj.weight'], None, partials=True)
        u = ops.channel_conv(xz, p['conv.weight'], p['conv.bias'], columns=self.inner,
                             state=conv_cache.state if conv_cache is not None else None, activation='silu',
                             out_dtype=self.dtype, row_seq=ctx.row_seq, **sequences)
        low = ops.linear(u, p['low_proj.weight'], None)
        dt = ops.linear(low, p['dt_proj.weight'], None, partials=True)
        bc = ops.linear(u, p['bc_proj.weight'], None, partials=True)
        y = ops.selective_scan(u, dt, bc, xz, dt_bias=p['dt_proj.bias'], a=p['A'], d=p['D'], state=scan_cache.state,
                               gate_offset=self.inner, max_query=ctx.max_query, out_dtype=self.dtype, **sequences)
        return ops.linear(y, p['o_proj.weight'], None, partials=True)
