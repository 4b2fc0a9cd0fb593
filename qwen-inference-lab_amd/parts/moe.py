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

    ``score='sigmoid'``: the scores are sigmoid(logit), each output by itself, instead of the softmax; the choice then
    goes by the score (+ correction).  ``group_score='top2'``: a group's score is the sum of its two largest choice
    scores instead of its largest.  With ``renormalize`` the chosen scores are divided by their sum +
    ``renormalize_eps``; ``weight_scale`` multiplies the weights last.
    ``shared``: a feed-forward part that every token passes and whose result is added to the routed sum (in float32,
    by one kernel); its tensors are this part's own under the prefix ``shared.``.

    The experts' matrices are stacked at ``finalize`` into [experts, 2, ff, width] (gate rows, then up rows) and
    [experts, width, ff], ff padded with zeros to a multiple of 16 (a zero gate and up row give act = 0, which meets a
    zero column of the down matrix): pure re-layouts.
    """

    def __init__(self, *, width, experts, identity=0, top, groups=1, keep=1, intermediate, activation='silu', limit=None,
                 alpha=1.0, correction=False, renormalize=False, bias=False, dtype=torch.bfloat16, score='softmax',
                 group_score='max', weight_scale=1.0, renormalize_eps=0.0, shared=None):
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
        if score not in ops.ROUTER_SCORES or group_score not in ops.ROUTER_GROUP_SCORES:
            raise ValueError(f'no router kernel for score {score!r} with group score {group_score!r}')
        self.score, self.group_score = score, group_score
        self.weight_scale, self.renormalize_eps, self.shared = float(weight_scale), float(renormalize_eps), shared

    def set_param(self, name, tensor):
        if name.startswith('shared.'):
            return self.shared.set_param(name[len('shared.'):], tensor)
        return super().set_param(name, tensor)

    def parameter_bytes(self):
        return super().parameter_bytes() + (self.shared.parameter_bytes() if self.shared is not None else 0)

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
        if self.shared is not None:
            specs.update({'shared.' + name: spec for name, spec in self.shared.param_specs().items()})
        return specs

    def finalize(self):
        if self.shared is not None:
            self.shared.finalize()
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
                                        keep=self.keep, top=self.top, renormalize=self.renormalize, bias=p.get('router.bias'),
                                        score=self.score, group_score=self.group_score, weight_scale=self.weight_scale,
                                        renormalize_eps=self.renormalize_eps)
        out = ops.moe_experts(h, chosen, weights, p['experts.gate_up_proj.weight'], p['experts.down_proj.weight'],
                              activation=self.activation, limit=self.limit, alpha=self.alpha, lazy=self.shared is None)
        if self.shared is not None:                     # routed sum + the shared expert's result, float32
            return ops.Partials(ops.scaled_sum(out, self.shared.forward(h), 1.0, 1.0).unsqueeze(0))
        if isinstance(out, ops.RoutedSum):              # the norm that follows makes the weighted sum as it loads the rows
            return out
        return ops.Partials(out.unsqueeze(0))           # complete float32 sums: one split
