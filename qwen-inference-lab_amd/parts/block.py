"""Pre-norm residual arrangement: norm -> sub-layer -> add to the un-normalised stream.

Two sub-layers per block, mixer then feed-forward (qil/model.py:48-71), or the mixer alone (``ffn=None``).  The
stream is float32 and every residual sum is made in float32; the add of a
sub-layer's output is fused into the norm that follows it.  ``residual_scale`` m: x + m * sublayer(norm(x)); the
norms multiply what they add, and the model multiplies the last block's output (``CausalLM(residual_scale=)``).
"""
import torch

from .base import Block, ParamSpec, CompoundNeed
from .. import ops


class PreNormBlock(Block):
    def __init__(self, *, mixer_norm, mixer, ffn_norm=None, ffn=None, dtype, names=None, residual_scale=1.0):
        super().__init__()
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.dtype = mixer_norm, mixer, ffn_norm, ffn, dtype
        if (ffn is None) != (ffn_norm is None):
            raise ValueError('a feed-forward and its norm come together')
        self.residual_scale = float(residual_scale)
        self._names = names or dict(mixer_norm='mixer_norm', mixer='mixer', ffn_norm='ffn_norm', ffn='ffn')

    def parts(self):
        n = self._names
        out = {n['mixer_norm']: self.mixer_norm, n['mixer']: self.mixer}
        if self.ffn is not None:
            out.update({n['ffn_norm']: self.ffn_norm, n['ffn']: self.ffn})
        return out

    def forward(self, stream, pending, ctx, cache):
        if self.residual_scale != 1.0:
            return self._forward_scaled(stream, pending, ctx, cache)
        h = None
        if isinstance(pending, ops.Added):                     # the stream is complete
            if self.mixer.takes_lazy_norm:                     # the mixer's first product may make the norm itself
                h = self.mixer_norm.forward_lazy(stream, self.dtype, pending)
            pending = None
        if h is None:
            h = self.mixer_norm.forward(stream, pending, self.dtype)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return mixed
        h = self.ffn_norm.forward(stream, None if isinstance(mixed, ops.Added) else mixed, self.dtype)
        return self.ffn.forward(h, add_to=stream) if self.ffn.adds_to_stream else self.ffn.forward(h)

    def _forward_scaled(self, stream, pending, ctx, cache):
        """The same with every sub-layer output multiplied as it is added: nothing adds into the stream by itself."""
        m = self.residual_scale
        if isinstance(pending, ops.Added):
            pending = None
        h = self.mixer_norm.forward(stream, pending, self.dtype, delta_scale=m)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return mixed
        return self.ffn.forward(self.ffn_norm.forward(stream, mixed, self.dtype, delta_scale=m))


class SandwichBlock(Block):
    """A norm before and a norm after every sub-layer: x <- x + post(sublayer(pre(x))), mixer then feed-forward (or
    the mixer alone).  The stream and both norms' statistics are float32; a sub-layer's output leaves the block as an
    ``ops.PostNormed`` (not yet normed, not yet added), and the norm that follows, this block's or the next one's or
    the model's last, makes the post norm, the sum and its own norm in one kernel."""

    def __init__(self, *, mixer_norm, mixer, mixer_post_norm, ffn_norm=None, ffn=None, ffn_post_norm=None, dtype, names=None):
        super().__init__()
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ffn_norm, self.ffn, self.ffn_post_norm, self.dtype = ffn_norm, ffn, ffn_post_norm, dtype
        if len({ffn is None, ffn_norm is None, ffn_post_norm is None}) != 1:
            raise ValueError('a feed-forward and its two norms come together')
        self._names = names or dict(mixer_norm='mixer_norm', mixer='mixer', mixer_post_norm='mixer_post_norm',
                                    ffn_norm='ffn_norm', ffn='ffn', ffn_post_norm='ffn_post_norm')

    def parts(self):
        n = self._names
        out = {n['mixer_norm']: self.mixer_norm, n['mixer']: self.mixer, n['mixer_post_norm']: self.mixer_post_norm}
        if self.ffn is not None:
            out.update({n['ffn_norm']: self.ffn_norm, n['ffn']: self.ffn, n['ffn_post_norm']: self.ffn_post_norm})
        return out

    @staticmethod
    def _post(norm, value):
        return ops.PostNormed(value, norm.p['weight'], norm.eps)

    def forward(self, stream, pending, ctx, cache):
        if isinstance(pending, ops.Added):                     # the stream is complete
            pending = None
        h = self.mixer_norm.forward(stream, pending, self.dtype)
        mixed = self._post(self.mixer_post_norm, self.mixer.forward(h, ctx, cache))
        if self.ffn is None:
            return mixed
        h = self.ffn_norm.forward(stream, mixed, self.dtype)
        return self._post(self.ffn_post_norm, self.ffn.forward(h))


class PostNormBlock(Block):
    """The norm stands on the sub-layer's output only, and the sub-layers read the stream itself:

        x <- x + s1 * norm1(mixer(c(x))),   then   x <- x + s2 * norm2(ffn(x))      (or the mixer alone)

    ``input_conv``: a ``ShortConvolution`` c that the mixer's input passes first (None: the mixer reads x).
    ``layer_scale``: s1, s2 are stored vectors (tensors ``mixer_scale``, ``ffn_scale``), a factor per channel on the
    normed output; without it they are 1.
    ``depth``, ``depth_total``: the block is run ``depth - 2`` of a model whose blocks all average over depth; with X_0
    the embedding's output and X_(i+1) the result of run i, what leaves run i is sum_(j <= i+1) mix[j] X_j (tensor
    ``depth_mix`` [depth]).  The results travel from block to block as an ``ops.Averaged``; the first block makes
    the buffer for ``depth_total`` of them.
    The stream, the norms, the scale, the sums and the average are float32; the sub-layers' products read the stream
    (or the convolution's result) rounded once to the model's type.  The norm, the scale, the sum, the average and
    the rounding are one kernel a sub-layer.  A block with a convolution keeps pages (its mixer's) and a state (the
    convolution's): its ``cache_need`` is a ``CompoundNeed`` and its cache the pair of views."""

    def __init__(self, *, mixer, mixer_post_norm, ffn=None, ffn_post_norm=None, input_conv=None, layer_scale=False,
                 depth=None, depth_total=None, width, dtype, names=None):
        super().__init__()
        if (ffn is None) != (ffn_post_norm is None):
            raise ValueError('a feed-forward and its norm come together')
        if depth is not None and not (type(depth) is int and type(depth_total) is int and 2 <= depth <= depth_total):
            raise ValueError('depth counts the results averaged after this block: from 2 to depth_total')
        self.mixer, self.mixer_post_norm, self.ffn, self.ffn_post_norm = mixer, mixer_post_norm, ffn, ffn_post_norm
        self.input_conv, self.layer_scale, self.depth, self.depth_total = input_conv, bool(layer_scale), depth, depth_total
        self.width, self.dtype = int(width), dtype
        self._names = names or dict(mixer='mixer', mixer_post_norm='mixer_post_norm', ffn='ffn',
                                    ffn_post_norm='ffn_post_norm', input_conv='input_conv')

    def parts(self):
        n = self._names
        out = {n['mixer']: self.mixer, n['mixer_post_norm']: self.mixer_post_norm}
        if self.ffn is not None:
            out.update({n['ffn']: self.ffn, n['ffn_post_norm']: self.ffn_post_norm})
        if self.input_conv is not None:
            out[n['input_conv']] = self.input_conv
        return out

    def param_specs(self):
        specs = {}
        if self.layer_scale:
            specs['mixer_scale'] = ParamSpec((self.width,), 'vector', 'one_plus_normal')
            if self.ffn is not None:
                specs['ffn_scale'] = ParamSpec((self.width,), 'vector', 'one_plus_normal')
        if self.depth is not None:
            specs['depth_mix'] = ParamSpec((self.depth,), 'vector', 'normal')
        return specs

    def _conv_need(self):
        return self.input_conv.cache_need() if self.input_conv is not None else None

    def cache_need(self):
        mixer, conv = self.mixer.cache_need(), self._conv_need()
        if conv is None:
            return mixer
        return CompoundNeed((mixer, conv)) if mixer is not None else conv

    def _join(self, stream, value, norm, scale, out_dtype, history, last):
        averaging = last and self.depth is not None
        return ops.post_norm_scale_add(stream, value, weight=norm.p['weight'], bias=norm.p.get('bias'),
                                       channel_scale=self.p.get(scale), eps=norm.eps, centre=norm.centre,
                                       out_dtype=out_dtype, history=history if averaging else None,
                                       depth=self.depth if averaging else 0,
                                       mix=self.p['depth_mix'] if averaging else None)

    def forward(self, stream, pending, ctx, cache):
        if pending is not None and not isinstance(pending, ops.Added):
            raise TypeError('a post-norm block takes a complete stream')
        mixer_cache, conv_cache = cache, None
        if self._conv_need() is not None:
            mixer_cache, conv_cache = cache if self.mixer.cache_need() is not None else (None, cache)
        history = None
        if self.depth is not None:
            if isinstance(pending, ops.Averaged):
                history = pending.history
                if pending.count != self.depth - 1:
                    raise ValueError(f'run {self.depth - 2} of a depth average follows {pending.count - 1} runs')
            else:                                       # the first block: X_0 is the stream as the embedding left it
                if self.depth != 2:
                    raise ValueError('a depth average begins at the first block')
                history = torch.empty((self.depth_total, *stream.shape), dtype=torch.float32, device=stream.device)
                history[0].copy_(stream)
        rounded = None if self.dtype == torch.float32 else self.dtype       # float32 products read the stream itself
        if self.input_conv is not None:
            h = self.input_conv.forward(stream, ctx, conv_cache, self.dtype)
        else:
            h = stream if rounded is None else stream.to(rounded)
        mixed = self.mixer.forward(h, ctx, mixer_cache)
        h = self._join(stream, mixed, self.mixer_post_norm, 'mixer_scale', None if self.ffn is None else rounded, history,
                       self.ffn is None)
        if self.ffn is not None:
            self._join(stream, self.ffn.forward(stream if h is None else h), self.ffn_post_norm, 'ffn_scale', None, history,
                       True)
        return ops.Averaged(history, self.depth) if self.depth is not None else ops.Added(None)
