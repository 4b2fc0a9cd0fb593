"""Attention whose keys and values are expanded from one cached low-rank latent per token."""
import torch

from .base import Mixer, ParamSpec, PagedNeed
from .. import ops


class LatentAttention(Mixer):
    """Per token the cache holds a latent c [kv_rank] (RMS-normed, with a weight) and one rotated key part kr [rot_dim]
    that every head shares.  Head h's key is [W_uk,h c ; kr], its value W_uv,h c.  Queries pass through a latent of
    their own: cq = rmsnorm(W_dq x) [q_rank], q = W_uq cq, laid out head by head as [dim unrotated, rot_dim rotated].

        score(h, i, j) = scale * (q_h,i[:dim] . W_uk,h c_j  +  rotate(q_h,i[dim:], i) . kr_j),   j <= i
        p(h, i, .)     = exp(score) / (sum_j exp(score(h, i, j)) + exp(sink_h))      (``sink``: a logit per head
                         that has no key and no value; it only enlarges the denominator)
        out_i          = W_o concat_h(W_uv,h sum_j p(h, i, j) c_j)

    Keys and values are never expanded: the query is multiplied by W_uk,h^T once (``ops.latent_query``), the
    attention kernel works on the cached rows themselves, and W_uv,h is applied to the weighted sum of latents.
    ``position``: a ``RotaryFrequencies`` over ``rot_dim`` elements.
    ``window`` w: row i sees the keys j with 0 <= i - j < w only, and the cache gives pages back that no later row
    sees (None: every key j <= i).
    ``gate``: head h's result is multiplied by sigmoid(W_g x)_h (tensor ``g_proj.weight`` [heads, width]; the
    sigmoid in float32); W_g is stacked under the two down projections, so the gate costs no product of its own.
    ``pairing``: which elements of the rotated parts a rotation pairs: 'halves', (i, i + rot_dim / 2), which is what
    the kernels do, or 'neighbours', (2 i, 2 i + 1) with the same frequency f_i.  A score does not change when the
    elements of the query's and the key's rotated part are reordered alike, so for 'neighbours' the rows of W_uq
    (every head's rotated part) and of W_dkv (the shared rotated part) are reordered once at ``finalize``, even
    elements first, and the kernels run as they are.
    """
    graph_safe = True

    def __init__(self, *, width, heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, eps, position, sink=True,
                 window=None, gate=False, pairing='halves', dtype=torch.bfloat16):
        super().__init__()
        for name, value in (('heads', heads), ('dim', dim), ('vdim', vdim), ('kv_rank', kv_rank), ('q_rank', q_rank)):
            if type(value) is not int or value < 1:
                raise ops.UnsupportedShape(f'{name} must be a positive integer, not {value!r}')
        if type(rot_dim) is not int or rot_dim < 2 or rot_dim % 2:
            raise ops.UnsupportedShape(f'rot_dim {rot_dim!r} must be even and at least 2')
        if position is None or position.rot_dim != rot_dim:
            raise ValueError('the rotation must cover exactly the rotated part')
        self.width, self.heads, self.dim, self.rot_dim, self.vdim = width, heads, dim, rot_dim, vdim
        self.kv_rank, self.q_rank, self.scale, self.eps = kv_rank, q_rank, float(scale), float(eps)
        self.position, self.sink, self.dtype = position, bool(sink), dtype
        if window is not None and (type(window) is not int or window < 1):
            raise ops.UnsupportedShape(f'window must be a positive integer or None, not {window!r}')
        if pairing not in ('halves', 'neighbours'):
            raise ValueError(f"pairing must be 'halves' or 'neighbours', not {pairing!r}")
        self.window, self.gate, self.pairing = window, bool(gate), pairing

    def param_specs(self):
        h, d, r = self.heads, self.dim, self.rot_dim
        specs = {'q_down.weight': ParamSpec((self.q_rank, self.width)),
                 'q_norm.weight': ParamSpec((self.q_rank,), 'vector', 'one_plus_normal'),
                 'q_up.weight': ParamSpec((h * (d + r), self.q_rank)),
                 'kv_down.weight': ParamSpec((self.kv_rank + r, self.width)),
                 'kv_norm.weight': ParamSpec((self.kv_rank,), 'vector', 'one_plus_normal'),
                 'k_up.weight': ParamSpec((h * d, self.kv_rank)),
                 'v_up.weight': ParamSpec((h * self.vdim, self.kv_rank)),
                 'o_proj.weight': ParamSpec((self.width, h * self.vdim))}
        if self.sink:
            specs['sink'] = ParamSpec((h,), 'vector', 'normal')
        if self.gate:
            specs['g_proj.weight'] = ParamSpec((h, self.width))
        return specs

    def cache_need(self):
        return PagedNeed((('latent', (self.kv_rank,), 'model'), ('rope', (self.rot_dim,), 'model')), self.window)

    def finalize(self):
        p = self.p
        if self.pairing == 'neighbours':                # even elements of every rotated part first: (2 i, 2 i + 1) -> (i, i + r / 2)
            d, r = self.dim, self.rot_dim
            order = torch.cat([torch.arange(0, r, 2), torch.arange(1, r, 2)]).to(p['q_up.weight'].device)
            q_up = p['q_up.weight'].view(self.heads, d + r, self.q_rank)
            p['q_up.weight'] = torch.cat([q_up[:, :d], q_up[:, d:][:, order]], dim=1).reshape(-1, self.q_rank).contiguous()
            kv_down = p['kv_down.weight']
            p['kv_down.weight'] = torch.cat([kv_down[:self.kv_rank], kv_down[self.kv_rank:][order]]).contiguous()
        # the down products in one: [q_rank + kv_rank + rot_dim (+ heads), width]
        stacked = [p.pop('q_down.weight'), p.pop('kv_down.weight')] + ([p.pop('g_proj.weight')] if self.gate else [])
        self.w_down = torch.cat(stacked).contiguous()
        p['down.weight'] = self.w_down
        # W_uk as [heads, dim, kv_rank] is the layout the query's product reads (a pure view); W_uv per head transposed
        self.k_up = p['k_up.weight'].view(self.heads, self.dim, self.kv_rank)
        p['v_up.weight'] = p['v_up.weight'].view(self.heads, self.vdim, self.kv_rank).transpose(1, 2).contiguous()
        self.position.frequencies()                     # made here, not in a step that may be captured

    def forward(self, h, ctx, cache):
        p = self.p
        frequencies = self.position.frequencies()
        down = ops.linear(h, self.w_down, None, partials=True)
        cq = ops.latent_prepare(down, q_rank=self.q_rank, rank=self.kv_rank, rot=self.rot_dim, q_weight=p['q_norm.weight'],
                                c_weight=p['kv_norm.weight'], eps=self.eps, frequencies=frequencies,
                                positions=ctx.positions, slots=cache.slots if cache.writes else None,
                                latent=cache.tensors['latent'], rope=cache.tensors['rope'], dtype=self.dtype,
                                gates=self.heads if self.gate else 0)
        cq, gate = cq if self.gate else (cq, None)
        q = ops.linear(cq, p['q_up.weight'], None)
        q = ops.latent_query(q, self.k_up, heads=self.heads, dim=self.dim, rot=self.rot_dim, rank=self.kv_rank,
                             frequencies=frequencies, positions=ctx.positions)
        mixed = ops.latent_attention(q, latent=cache.tensors['latent'], rope=cache.tensors['rope'],
                                     page_size=cache.page_size, block_tables=cache.block_tables, row_seq=ctx.row_seq,
                                     positions=ctx.positions, sink=p.get('sink'), scale=self.scale, heads=self.heads,
                                     rank=self.kv_rank, rot=self.rot_dim, cu_seqlens=ctx.cu_seqlens,
                                     seq_starts=ctx.seq_starts, n_seqs=ctx.n_seqs, max_query=ctx.max_query,
                                     max_context=ctx.max_context, window=self.window, gate=gate)
        values = ops.head_product(mixed, p['v_up.weight'], heads=self.heads, out_dtype=self.dtype)
        return ops.linear(values, p['o_proj.weight'], None, partials=True)
