"""Grouped-query attention over the paged cache.  Formulas: qil/model.py:48-69, :73-84."""
import torch

from .base import Mixer, ParamSpec, KVNeed
from .. import ops


class Attention(Mixer):
    """q/k/v projections (+bias), optional per-head RMSNorm of q and k, position
    encoding, write of k/v into the request's pages, attention of the step's
    queries over everything cached (key j visible iff j <= position, and
    j > position - window if a window is set), output projection (+bias).

    Query head h reads kv head h // (heads / kv_heads)  (qil/model.py:59-61).
    The three projection matrices are stacked at ``finalize`` into one
    [(heads + 2 kv_heads) head_dim, width] matrix: a pure re-layout, each output
    column is computed from the same row as before.

    The attention kernels take heads of a multiple of 8 elements.  Any other even size (qil/config.py:29-30 allows
    every even one) is padded at ``finalize`` to the next multiple of 8: zero rows at the end of every head of the
    q/k/v matrices (and biases), zero columns in the output matrix, zeros in the head norms' weights.  Padded elements
    of queries, keys and values are then exact zeros, which add nothing to a score or to the output; the head norm's
    mean runs over the true size (``norm_dim``), the rotation over the true size's pairs, and the scale is the
    caller's.  The cache holds the padded size.

    What a design may change beyond sizes: ``value_dim`` (values of another size than queries and keys: every head is
    padded with zeros to the larger of the two, so keys and values share the kernels' one head size; the output
    matrix gets zero columns for the padding); ``softcap`` c (scores become c * tanh(score / c) after the scale);
    ``qk_norm_weights=False`` (the head norms divide by the root mean square and multiply by nothing: the part
    declares no norm tensors); ``norm_after_rotation`` (queries and keys are rotated first and normed then).
    ``position`` may be a ``Rotary`` (tables) or a ``RotaryFrequencies`` (the kernels make the angles from the
    positions, which no table bounds).
    ``out_bias``: whether the output projection has a bias (default: as ``bias``).
    ``q_temperature`` (coef, every): the query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)
    after the head norm, in float32.
    ``sink``: a stored number per query head (tensor ``sinks``) whose exponential joins the softmax's denominator
    once: it has no key and no value and is not scaled.
    ``gate``: the heads' results are multiplied element by element by sigmoid(W_g h) before the output projection
    (tensor ``g_proj.weight`` [heads * value_dim, width], stacked under q/k/v: one product makes all four).
    ``own_kv=False``: the part has no key and value projections; its schedule entry reads another entry's cache
    (``ScheduleEntry.cache_of``), with its own queries, mask and everything else.
    """
    graph_safe = True
    takes_lazy_norm = True       # h goes into ops.linear only, which takes a norm not computed yet

    def __init__(self, *, width, heads, kv_heads, head_dim, bias, qk_norm_eps, scale,
                 position=None, window=None, dtype=torch.bfloat16, value_dim=None, softcap=None, qk_norm_weights=True,
                 norm_after_rotation=False, out_bias=None, q_temperature=None, sink=False, gate=False, own_kv=True):
        super().__init__()
        if heads % kv_heads:
            raise ValueError('heads must be a multiple of kv_heads')
        self.width, self.heads, self.kv_heads, self.head_dim = width, heads, kv_heads, head_dim
        self.bias, self.qk_norm_eps, self.scale = bool(bias), qk_norm_eps, float(scale)
        self.position, self.window, self.dtype = position, window, dtype
        self.value_dim = head_dim if value_dim is None else value_dim
        self.softcap = None if softcap is None else float(softcap)
        self.qk_norm_weights, self.norm_after_rotation = bool(qk_norm_weights), bool(norm_after_rotation)
        self.out_bias = self.bias if out_bias is None else bool(out_bias)
        self.sink, self.gate, self.own_kv = bool(sink), bool(gate), bool(own_kv)
        self.q_temperature = None
        if q_temperature is not None:
            coef, every = q_temperature
            if type(every) is not int or every < 1:
                raise ValueError('the query temperature grows every so many positions: a positive integer')
            self.q_temperature = (float(coef), every)
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError('softcap must be positive')
        if type(self.value_dim) is not int or self.value_dim < 1:
            raise ops.UnsupportedShape(f'value_dim {self.value_dim!r} must be a positive integer')
        rotated = getattr(position, 'rot_dim', 0) if position is not None else 0
        if type(head_dim) is not int or head_dim < 1 or rotated > head_dim or (value_dim is None and head_dim % 2):
            raise ops.UnsupportedShape(f'head_dim {head_dim} must be even (any size of at least the rotated width when '
                                       'the values have a size of their own)')
        self.padded_dim = -(-max(head_dim, self.value_dim) // 8) * 8    # what the kernels and the cache see
        ops.check_attention_geometry(heads=heads, kv_heads=kv_heads, head_dim=self.padded_dim, dtype=dtype)

    def param_specs(self):
        q, kv, d = self.heads * self.head_dim, self.kv_heads * self.head_dim, self.head_dim
        v, o = self.kv_heads * self.value_dim, self.heads * self.value_dim
        specs = {'q_proj.weight': ParamSpec((q, self.width)), 'o_proj.weight': ParamSpec((self.width, o))}
        if self.own_kv:
            specs.update({'k_proj.weight': ParamSpec((kv, self.width)), 'v_proj.weight': ParamSpec((v, self.width))})
        if self.bias:
            specs['q_proj.bias'] = ParamSpec((q,), 'vector')
            if self.own_kv:
                specs.update({'k_proj.bias': ParamSpec((kv,), 'vector'), 'v_proj.bias': ParamSpec((v,), 'vector')})
        if self.out_bias:   # o_proj gets a bias too (qil/model.py:35)
            specs['o_proj.bias'] = ParamSpec((self.width,), 'vector')
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            specs['q_norm.weight'] = ParamSpec((d,), 'vector', 'one_plus_normal')
            if self.own_kv:
                specs['k_norm.weight'] = ParamSpec((d,), 'vector', 'one_plus_normal')
        if self.gate:
            specs['g_proj.weight'] = ParamSpec((o, self.width))
        if self.sink:
            specs['sinks'] = ParamSpec((self.heads,), 'vector')
        return specs

    def cache_need(self):
        return KVNeed(self.kv_heads, self.padded_dim, self.window)

    def _pad_heads(self, tensor, axis=0, d=None):
        """``tensor`` with every head's ``d`` (default ``head_dim``) entries along ``axis`` followed by zeros up to
        ``padded_dim``."""
        d, dp = d or self.head_dim, self.padded_dim
        if d == dp:
            return tensor
        count = tensor.shape[axis] // d
        shape = list(tensor.shape)
        shape[axis:axis + 1] = [count, d]
        padded_shape = list(shape)
        padded_shape[axis + 1] = dp
        out = tensor.new_zeros(padded_shape)
        out.narrow(axis + 1, 0, d).copy_(tensor.reshape(shape))
        shape[axis:axis + 2] = [count * dp]
        return out.reshape(shape)

    def finalize(self):
        p = self.p
        stacked = [('q_proj', self.head_dim)]
        if self.own_kv:
            stacked += [('k_proj', self.head_dim), ('v_proj', self.value_dim)]
        matrices = [self._pad_heads(p.pop(f'{name}.weight'), d=d) for name, d in stacked]
        biases = [self._pad_heads(p.pop(f'{name}.bias'), d=d) for name, d in stacked] if self.bias else None
        if self.gate:                                    # the gate's rows come last and have no bias
            matrices.append(self._pad_heads(p.pop('g_proj.weight'), d=self.value_dim))
            if self.bias:
                biases.append(biases[0].new_zeros(self.heads * self.padded_dim))
        self.w_qkv = torch.cat(matrices).contiguous()
        self.b_qkv = torch.cat(biases).contiguous() if self.bias else None
        # the bias of q, k and v alone (the gate has none), as the q/k kernel takes it
        self.b_qkv_own = torch.cat(biases[:len(stacked)]).contiguous() if self.bias else None
        p['qkv_proj.weight'] = self.w_qkv
        if self.bias:
            p['qkv_proj.bias'] = self.b_qkv
        if self.padded_dim != self.value_dim:
            p['o_proj.weight'] = self._pad_heads(p['o_proj.weight'], axis=1, d=self.value_dim).contiguous()
        if self.padded_dim != self.head_dim:
            for name in ('q_norm.weight', 'k_norm.weight'):
                if name in p:
                    p[name] = self._pad_heads(p[name]).contiguous()
        if self.qk_norm_eps is not None and not self.qk_norm_weights:       # a norm that multiplies by nothing
            self._ones = torch.ones(self.padded_dim, dtype=torch.float32, device=self.w_qkv.device)
        if self.position is not None:
            self.position.rotation()                     # device tensors are made here, not in a step that may be captured

    def forward(self, h, ctx, cache):
        p = self.p
        if cache.writes and not self.own_kv:
            raise ValueError('an attention part without keys and values of its own reads another entry\'s cache')
        extended = self.gate or self.sink or self.q_temperature is not None or not self.own_kv
        # (the extended step's q/k kernel adds the bias itself: its product may then stay partial sums)
        qkv = ops.linear(h, self.w_qkv, None if extended else self.b_qkv, partials=True)
        rotation = self.position.rotation() if self.position is not None else None
        if self.qk_norm_eps is not None and not self.qk_norm_weights:
            norms = dict(q_weight=self._ones, k_weight=self._ones, eps=self.qk_norm_eps)
        else:
            norms = dict(q_weight=p.get('q_norm.weight'), k_weight=p.get('k_norm.weight', p.get('q_norm.weight')),
                         eps=self.qk_norm_eps if self.qk_norm_eps is not None else 0.0)
        sizes = dict(heads=self.heads, kv_heads=self.kv_heads, head_dim=self.padded_dim)
        if extended:
            return self._forward_extended(qkv, rotation, norms, sizes, ctx, cache)
        # (the kernel that makes its queries itself norms over the whole head it sees: not for padded heads)
        if ctx.max_query == 1 and self.padded_dim == self.head_dim and \
                ops.decode_attention_takes(qkv, page_size=cache.page_size, rotation=rotation, dtype=self.dtype, **sizes):
            # every row alone in its sequence: norm, rotation and cache write happen inside the attention kernel
            attended = ops.decode_attention(
                qkv, rotation=rotation, positions=ctx.positions, writes=cache.writes, k_cache=cache.k, v_cache=cache.v,
                page_size=cache.page_size, block_tables=cache.block_tables, row_seq=ctx.row_seq,
                max_context=ctx.max_context, scale=self.scale, window=self.window, unmerged=True,
                rotate_first=self.norm_after_rotation, softcap=self.softcap, **sizes, **norms)
            return ops.linear(attended, p['o_proj.weight'], p.get('o_proj.bias'), partials=True)
        q = ops.qk_norm_rope_store(
            qkv, rotation=rotation, positions=ctx.positions, slots=cache.slots if cache.writes else None,
            k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size, dtype=self.dtype, norm_dim=self.head_dim,
            rotate_first=self.norm_after_rotation, **sizes, **norms)
        attended = ops.paged_attention(
            q, k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size,
            block_tables=cache.block_tables, row_seq=ctx.row_seq, positions=ctx.positions,
            cu_seqlens=ctx.cu_seqlens, seq_starts=ctx.seq_starts, single_rows=ctx.single_rows, n_seqs=ctx.n_seqs,
            max_query=ctx.max_query, max_context=ctx.max_context, tile_seqs=ctx.tile_seqs,
            scale=self.scale, window=self.window, unmerged=True, softcap=self.softcap, **sizes)
        return ops.linear(attended, p['o_proj.weight'], p.get('o_proj.bias'), partials=True)

    def _forward_extended(self, qkv, rotation, norms, sizes, ctx, cache):
        """The step of a part with a query temperature, sinks, an output gate or another entry's keys and values:
        the q/k kernel skips the gate's columns of the stacked product (and finds no key and value columns when the
        part has none), the attention kernels take the sinks, and the gate multiplies what they return."""
        p = self.p
        gate_columns = self.heads * self.padded_dim if self.gate else 0
        stored = self.kv_heads if self.own_kv else 0
        if ctx.max_query == 1 and self.padded_dim == self.head_dim and \
                ops.decode_attention_takes(qkv, page_size=cache.page_size, rotation=rotation, dtype=self.dtype, **sizes):
            # every row alone in its sequence: bias, norm, rotation, temperature and cache write inside the attention kernel
            attended = ops.decode_attention(
                qkv, rotation=rotation, positions=ctx.positions, writes=cache.writes, k_cache=cache.k, v_cache=cache.v,
                page_size=cache.page_size, block_tables=cache.block_tables, row_seq=ctx.row_seq,
                max_context=ctx.max_context, scale=self.scale, window=self.window, unmerged=False,
                rotate_first=self.norm_after_rotation, softcap=self.softcap, has_kv=self.own_kv,
                extra_columns=gate_columns, bias=self.b_qkv_own, q_temperature=self.q_temperature, sinks=p.get('sinks'),
                **sizes, **norms)
            if self.gate:
                attended = ops.sigmoid_gate(attended, qkv, offset=(self.heads + 2 * stored) * self.padded_dim)
            return ops.linear(attended, p['o_proj.weight'], p.get('o_proj.bias'), partials=True)
        q = ops.qk_norm_rope_store(
            qkv, rotation=rotation, positions=ctx.positions, slots=cache.slots if cache.writes else None,
            k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size, dtype=self.dtype, norm_dim=self.head_dim,
            rotate_first=self.norm_after_rotation, heads=self.heads, kv_heads=stored, head_dim=self.padded_dim,
            extra_columns=gate_columns, q_temperature=self.q_temperature, bias=self.b_qkv_own, **norms)
        attended = ops.paged_attention(
            q, k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size,
            block_tables=cache.block_tables, row_seq=ctx.row_seq, positions=ctx.positions,
            cu_seqlens=ctx.cu_seqlens, seq_starts=ctx.seq_starts, single_rows=ctx.single_rows, n_seqs=ctx.n_seqs,
            max_query=ctx.max_query, max_context=ctx.max_context, tile_seqs=ctx.tile_seqs,
            scale=self.scale, window=self.window, unmerged=False, softcap=self.softcap, sinks=p.get('sinks'), **sizes)
        if self.gate:
            attended = ops.sigmoid_gate(attended, qkv, offset=(self.heads + 2 * stored) * self.padded_dim)
        return ops.linear(attended, p['o_proj.weight'], p.get('o_proj.bias'), partials=True)
