"""Norms with float32 statistics: RMSNorm (formula: qil/model.py:15-23) and a layer norm with or without a bias."""
import torch

from .base import Norm, ParamSpec
from .. import ops


class RMSNorm(Norm):
    """y = cast(x * rsqrt(mean(x^2) + eps)) * (offset + weight).  ``offset`` 0: the weight multiplies as stored;
    ``offset`` 1: a weight that is stored around zero.  The sum is made once, in float32, at ``finalize`` (the stored
    weights are float32 on the device whatever the model's type), so the kernels see one factor per channel."""
    centre = False

    def __init__(self, width, eps, offset=0.0):
        super().__init__()
        self.width, self.eps, self.offset = int(width), float(eps), float(offset)

    def param_specs(self):
        return {'weight': ParamSpec((self.width,), 'vector', 'one_plus_normal' if self.offset == 0.0 else 'normal')}

    def finalize(self):
        if self.offset != 0.0:
            self.p['weight'] = (self.p['weight'] + self.offset).contiguous()

    def forward(self, stream, delta, out_dtype, delta_scale=1.0):
        if delta_scale != 1.0:                      # (the general kernel rounds once, after the weight)
            return ops.add_norm(stream, delta, self.p['weight'], self.eps, out_dtype, centre=False, delta_scale=delta_scale)
        return ops.add_rmsnorm(stream, delta, self.p['weight'], self.eps, out_dtype)

    def forward_lazy(self, stream, out_dtype, added):
        if stream.is_cuda and out_dtype == torch.bfloat16 and stream.shape[0] <= ops.NORMED_GEMM_MOST_ROWS:
            return ops.Normed(stream, self.p['weight'], self.eps, out_dtype, added)
        return None

    def forward_rows(self, stream, delta, rows, out_dtype, delta_scale=1.0):
        if delta_scale != 1.0:
            return ops.rows_norm(stream, delta, rows, self.p['weight'], self.eps, out_dtype, centre=False,
                                 delta_scale=delta_scale)
        return ops.rows_rmsnorm(stream, delta, rows, self.p['weight'], self.eps, out_dtype)


class LayerNorm(Norm):
    """y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * weight (+ bias, if ``bias``); float32 throughout and one
    rounding of the result.  ``delta_scale`` multiplies the sub-layer output that is added into the stream first."""
    centre = True

    def __init__(self, width, eps, bias=False):
        super().__init__()
        self.width, self.eps, self.bias = int(width), float(eps), bool(bias)

    def param_specs(self):
        specs = {'weight': ParamSpec((self.width,), 'vector', 'one_plus_normal')}
        if self.bias:
            specs['bias'] = ParamSpec((self.width,), 'vector', 'normal')
        return specs

    def forward(self, stream, delta, out_dtype, delta_scale=1.0):
        return ops.add_norm(stream, delta, self.p['weight'], self.eps, out_dtype, centre=True, delta_scale=delta_scale,
                            bias=self.p.get('bias'))

    def forward_rows(self, stream, delta, rows, out_dtype, delta_scale=1.0):
        return ops.rows_norm(stream, delta, rows, self.p['weight'], self.eps, out_dtype, centre=True,
                             delta_scale=delta_scale, bias=self.p.get('bias'))
