"""Feed-forwards: gated, down(act(gate(x)) * up(x)) (formula: qil/model.py:71), and plain, down(act(up(x)))."""
import torch

from .base import FeedForward, ParamSpec
from .. import ops


class GatedMLP(FeedForward):
    """``activation`` names the gate's function (``ops.GATE_FUNCTIONS``): 'silu', silu(g) * u, or 'clamped_swish' with
    ``limit`` L and ``alpha`` a: g' = min(g, L), u' = clamp(u, -L, L), g' * sigmoid(a g') * (u' + 1).  Gate and up matrices become one [2 * intermediate, width] matrix at
    ``finalize`` (rows in turns of 16, or gate rows first where the sizes do not allow that): a pure re-layout."""

    def __init__(self, *, width, intermediate, activation='silu', limit=None, alpha=1.0, dtype=torch.bfloat16):
        super().__init__()
        self.dtype = dtype
        if activation not in ops.GATE_FUNCTIONS:
            raise ValueError(f'no kernel for activation {activation!r}')
        if activation == 'clamped_swish' and not (limit is not None and limit > 0):
            raise ValueError('clamped_swish needs a positive limit')
        self.width, self.intermediate, self.activation = width, intermediate, activation
        self.limit, self.alpha = float(limit or 0.0), float(alpha)

    def param_specs(self):
        return {'gate_proj.weight': ParamSpec((self.intermediate, self.width)),
                'up_proj.weight': ParamSpec((self.intermediate, self.width)),
                'down_proj.weight': ParamSpec((self.width, self.intermediate))}

    def finalize(self):
        p = self.p
        gate, up = p.pop('gate_proj.weight'), p.pop('up_proj.weight')
        # on the GPU, rows in turns of 16 where the sizes allow (the kernels read a gate tile and its up tile side by side)
        self.interleaved = self.intermediate % 16 == 0 and gate.is_cuda
        p['gate_up_proj.weight'] = ops.interleave_gate_up(gate, up) if self.interleaved else torch.cat([gate, up]).contiguous()

    adds_to_stream = True

    def forward(self, h, add_to=None):
        hidden = ops.gated_linear(h, self.p['gate_up_proj.weight'], self.dtype, interleaved=self.interleaved, lazy=True,
                                  activation=self.activation, limit=self.limit, alpha=self.alpha)
        if add_to is not None and hidden.is_cuda:              # few rows: the down product adds into the stream itself
            return ops.linear(hidden, self.p['down_proj.weight'], None, partials=True, add_to=add_to)
        return ops.linear(hidden, self.p['down_proj.weight'], None, partials=True)


class PlainMLP(FeedForward):
    """down(act(up(x))) without a gate branch and without biases.  ``activation`` names a function of
    ``ops.PLAIN_ACTIVATIONS``; 'xielu' has two stored numbers (p, q), the tensor ``act``, and is
    softplus(p) z^2 + z / 2 for z > 0, (1 / 2 + softplus(q)) (exp(z) - 1 - z) + z / 2 otherwise, in float32."""

    def __init__(self, *, width, intermediate, activation='xielu', dtype=torch.bfloat16):
        super().__init__()
        if activation not in ops.PLAIN_ACTIVATIONS:
            raise ValueError(f'no kernel for activation {activation!r}')
        self.width, self.intermediate, self.activation, self.dtype = width, intermediate, activation, dtype

    def param_specs(self):
        specs = {'up_proj.weight': ParamSpec((self.intermediate, self.width)),
                 'down_proj.weight': ParamSpec((self.width, self.intermediate))}
        if self.activation == 'xielu':
            specs['act'] = ParamSpec((2,), 'vector', 'normal')
        return specs

    def forward(self, h):
        hidden = ops.plain_act(ops.linear(h, self.p['up_proj.weight'], None, partials=True), self.dtype,
                               activation=self.activation, params=self.p.get('act'))
        return ops.linear(hidden, self.p['down_proj.weight'], None, partials=True)
