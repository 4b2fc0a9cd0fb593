"""Two mixers side by side on the same input."""
from .base import Mixer, CompoundNeed
from .. import ops


class ParallelMixers(Mixer):
    """result = left_scale * left(h) + right_scale * right(h): both mixers read the same h, each keeps what it keeps
    (the part's ``cache_need`` is the ``CompoundNeed`` of both, the left one's needs first; its cache is the tuple of
    their views and each mixer gets its own), and the weighted sum is made in float32 from their results (tensors of
    the model's type or float32 partial sums) by one kernel.  The children's tensors are the part's own, under the
    prefixes ``left.`` and ``right.``."""

    def __init__(self, *, left, right, left_scale=1.0, right_scale=1.0):
        super().__init__()
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.graph_safe = bool(left.graph_safe and right.graph_safe)

    def _children(self):
        return (('left.', self.left), ('right.', self.right))

    def param_specs(self):
        return {prefix + name: spec for prefix, child in self._children() for name, spec in child.param_specs().items()}

    def set_param(self, name, tensor):
        for prefix, child in self._children():
            if name.startswith(prefix):
                return child.set_param(name[len(prefix):], tensor)
        raise KeyError(name)

    def finalize(self):
        for _, child in self._children():
            child.finalize()

    def parameter_bytes(self):
        return sum(child.parameter_bytes() for _, child in self._children())

    @staticmethod
    def _single(need):
        return () if need is None else need.needs if isinstance(need, CompoundNeed) else (need,)

    def cache_need(self):
        needs = self._single(self.left.cache_need()) + self._single(self.right.cache_need())
        return None if not needs else needs[0] if len(needs) == 1 else CompoundNeed(needs)

    def _split(self, cache):
        """The children's caches out of the part's: None, one view, or a tuple, as each child would get it alone."""
        views = () if cache is None else cache if isinstance(cache, tuple) else (cache,)
        out, at = [], 0
        for _, child in self._children():
            count = len(self._single(child.cache_need()))
            mine = views[at:at + count]
            at += count
            out.append(None if count == 0 else mine[0] if count == 1 else tuple(mine))
        return out

    def forward(self, h, ctx, cache):
        left_cache, right_cache = self._split(cache)
        left = self.left.forward(h, ctx, left_cache)
        right = self.right.forward(h, ctx, right_cache)
        return ops.Partials(ops.scaled_sum(left, right, self.left_scale, self.right_scale).unsqueeze(0))
