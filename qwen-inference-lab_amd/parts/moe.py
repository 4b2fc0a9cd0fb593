"""A routed feed-forward: a router chooses a few experts per token, each a small gated feed-forward."""
import torch

from .base import FeedForward, ParamSpec
from .. import ops


class RoutedExperts(FeedForward):
    """``experts`` gated feed-forwards (``GatedMLP``'s formula with ``activation``, ``limit``, ``alpha``; no biases) of
    which every token uses ``top``, and ``identity`` more router outputs that stand for experts without tensors whose
    output is their input.

    Router: logits over experts + identity outputs in float32 (the router matrix stays float32 in every model), plus
    a stored bias per output if ``bias``; softmax over all of them; the choice goes by score + ``correction`` (a stored vector, if ``correction``) among the
    outputs of the ``keep`` best of ``groups`` equal groups of neighbouring outputs, a group's score being its best
    choice score; the weights are the chosen outputs' softmax scores, divided by their sum only if ``renormalize``
    (which makes them the softmax over the chosen logits alone).
    The result is the weighted sum of the chosen experts' outputs, in float32.

    The experts' matrices are stacked at ``finalize`` into [experts, 2, ff, width] (gate rows, then up rows) and
    [experts, width, ff], ff padded with zeros to a multiple of 16 (a zero gate and up row give act = 0, which meets a
    zero column of the down matrix): pure re-layouts.
    """

    def __init__(self, *, width, experts, identity=0, top, groups=1, keep=1, intermediate, activation='silu', limit=None,
                 alpha=1.0, correction=False, renormalize=False, bias=False, dtype=torch.bfloat16):
        super().__init__()
        for name, value in (('experts', experts), ('top', top), ('groups', groups), ('keep', keep),
                            ('intermediate', intermediate)):
            if type(value) is not int or value < 1:
                raise ops.UnsupportedShape(f'{name} must be a positive integer, not {value!r}')
        if type(identity) is not int or identity < 0:
            raise ops.UnsupportedShape(f'identity must be a non-negative integer, not {identity!r}')
        outputs = experts + identity
        if outputs % groups or keep > groups or top > keep * (outputs // groups):
            raise ValueError(f'{outputs} router outputs do not split into {groups} groups of which {keep} hold {top} choices')
        if activation not in ops.GATE_FUNCTIONS:
            raise ValueError(f'no kernel for activation {activation!r}')
        if activation == 'clamped_swish' and not (limit is not None and limit > 0):
            raise ValueError('clamped_swish needs a positive limit')
        self.width, self.experts, self.identity, self.top, self.groups, self.keep = width, experts, identity, top, groups, keep
        self.outputs, self.intermediate, self.activation = outputs, intermediate, activation
        self.limit, self.alpha, self.correction, self.renormalize = float(limit or 0.0), float(alpha), bool(correction), bool(renormalize)
        self.dtype, self.bias = dtype, bool(bias)

    def param_specs(self):
        specs = {'router.weight': ParamSpec((self.outputs, self.width), 'vector')}
        if self.bias:
            specs['router.bias'] = ParamSpec((self.outputs,), 'vector')
        if self.correction:
            specs['router.correction'] = ParamSpec((self.outputs,), 'vector')
        for e in range(self.experts):
            specs[f'experts.{e}.gate_proj.weight'] = ParamSpec((self.intermediate, self.width))
            specs[f'experts.{e}.up_proj.weight'] = ParamSpec((self.intermediate, self.width))
            specs[f'experts.{e}.down_proj.weight'] = ParamSpec((self.width, self.intermediate))
        return specs

    def finalize(self):
        p = self.p
        ff, padded = self.intermediate, -(-self.intermediate // 16) * 16
        first = p['experts.0.gate_proj.weight']
        gate_up = first.new_zeros((self.experts, 2, padded, self.width))
        down = first.new_zeros((self.experts, self.width, padded))
        for e in range(self.experts):
            gate_up[e, 0, :ff].copy_(p.pop(f'experts.{e}.gate_proj.weight'))
            gate_up[e, 1, :ff].copy_(p.pop(f'experts.{e}.up_proj.weight'))
            down[e, :, :ff].copy_(p.pop(f'experts.{e}.down_proj.weight'))
        p['experts.gate_up_proj.weight'], p['experts.down_proj.weight'] = gate_up, down

    def forward(self, h, add_to=None):
        p = self.p
        chosen, weights = ops.moe_route(h, p['router.weight'], p.get('router.correction'), groups=self.groups,
                                        keep=self.keep, top=self.top, renormalize=self.renormalize, bias=p.get('router.bias'))
        out = ops.moe_experts(h, chosen, weights, p['experts.gate_up_proj.weight'], p['experts.down_proj.weight'],
                              activation=self.activation, limit=self.limit, alpha=self.alpha, lazy=True)
        if isinstance(out, ops.RoutedSum):              # the norm that follows makes the weighted sum as it loads the rows
            return out
        return ops.Partials(out.unsqueeze(0))           # complete float32 sums: one split
