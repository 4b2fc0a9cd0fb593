"""A plain, slow restatement of the Zinesun design: one function per mechanism, whole sequences, no cache.

Test code only: it shares nothing with the engine.  Everything runs in one dtype (float64 by default) on the CPU.
Weights are a dict name -> tensor under the checkpoint's own names; ``config`` is the config.json dict.

Notation: x [T, width] is the residual stream of one sequence, h a sub-layer's input, H heads, t a position.
"""
import math

import torch


# ---------------------------------------------------------------------------------------------- small pieces
def layer_norm(y, weight, bias, eps):
    centred = y - y.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt(centred.square().mean(dim=-1, keepdim=True) + eps) * weight + bias


def rms_norm(y, weight, eps):
    return y / torch.sqrt(y.square().mean(dim=-1, keepdim=True) + eps) * weight


def softplus(v):
    return torch.log1p(torch.exp(v))


def rotate_neighbours(v, positions, base, dims):
    """v [T, ..., dims]: elements 2 i and 2 i + 1 are one pair, turned by the angle t * base^(-2 i / dims)."""
    frequency = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=v.dtype)
    angle = positions.to(v.dtype)[:, None] * frequency[None, :]
    while angle.dim() < v.dim():
        angle = angle.unsqueeze(1)
    even, odd = v[..., 0::2], v[..., 1::2]
    out = torch.empty_like(v)
    out[..., 0::2] = even * angle.cos() - odd * angle.sin()
    out[..., 1::2] = odd * angle.cos() + even * angle.sin()
    return out


def time_convolution(x, taps_weight):
    """x_t + sum_j w[:, j] x_(t - taps + 1 + j), nothing before the sequence's start.  taps_weight [width, taps]."""
    taps = taps_weight.shape[1]
    out = x.clone()
    for t in range(x.shape[0]):
        for j in range(taps):
            source = t - taps + 1 + j
            if source >= 0:
                out[t] += taps_weight[:, j] * x[source]
    return out


def xielu(z, numbers):
    above = softplus(numbers[0]) * z * z + z / 2
    below = (0.5 + softplus(numbers[1])) * (torch.exp(z.clamp(max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, above, below)


# ---------------------------------------------------------------------------------------------- the mixer
def latent_attention(h, w, pre, m, eps, positions, probabilities=None):
    """Keys and values of all heads from one normed latent per position, queries through a latent of their own, one
    rotated key part for all heads, a sliding window, a sigmoid gate per head on the result."""
    t = h.shape[0]
    heads, d, r, dv, rank = m['heads'], m['dim'], m['rot_dim'], m['vdim'], m['kv_rank']
    q = (rms_norm(h @ w[pre + 'dq'].t(), w[pre + 'dq.norm'], eps) @ w[pre + 'uq'].t()).reshape(t, heads, d + r)
    down = h @ w[pre + 'dkv'].t()
    latent = rms_norm(down[:, :rank], w[pre + 'dkv.norm'], eps)
    shared_key = rotate_neighbours(down[:, rank:], positions, m['rot']['base'], m['rot']['dims'])          # [T, r]
    keys = (latent @ w[pre + 'uk'].t()).reshape(t, heads, d)
    values = (latent @ w[pre + 'uv'].t()).reshape(t, heads, dv)
    turned = rotate_neighbours(q[:, :, d:], positions, m['rot']['base'], m['rot']['dims'])
    scores = (torch.einsum('ihd,jhd->hij', q[:, :, :d], keys) + torch.einsum('ihr,jr->hij', turned, shared_key)) * m['scale']
    distance = positions[:, None] - positions[None, :]
    visible = (distance >= 0) & (distance < m['mask']['size'])
    p = torch.softmax(scores.masked_fill(~visible[None], -math.inf), dim=-1)
    if probabilities is not None:
        probabilities.append(p)
    gate = torch.sigmoid(h @ w[pre + 'g'].t())                                                              # [T, H]
    out = torch.einsum('hij,jhd->ihd', p, values) * gate[:, :, None]
    return out.reshape(t, heads * dv) @ w[pre + 'o'].t()


# ---------------------------------------------------------------------------------------------- feed-forwards
def dense(h, w, pre):
    return xielu(h @ w[pre + 'up'].t(), w[pre + 'act']) @ w[pre + 'down'].t()


def router_logits(h, w, pre):
    return h @ w[pre + 'router'].t() + w[pre + 'router.b']


def route(h, w, pre, r):
    """(chosen [T, top], weights [T, top]): the largest logits, and the softmax over those alone."""
    best = router_logits(h, w, pre).topk(r['top'], dim=-1)
    return best.indices, torch.softmax(best.values, dim=-1)


def route_margin(h, w, pre, r):
    """How far the last chosen logit lies above the first one left out, per token (inf if every expert is chosen)."""
    z = router_logits(h, w, pre).sort(dim=-1, descending=True).values
    if r['top'] == r['experts']:
        return torch.full((h.shape[0],), math.inf, dtype=h.dtype)
    return z[:, r['top'] - 1] - z[:, r['top']]


def moe(h, w, pre, f):
    chosen, weights = route(h, w, pre, f['router'])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for slot in range(chosen.shape[1]):
            e = f"{pre}e{int(chosen[t, slot])}."
            g, u = w[e + 'gate'] @ h[t], w[e + 'up'] @ h[t]
            out[t] += weights[t, slot] * (w[e + 'down'] @ (g * torch.sigmoid(g) * u))
    return out


# ---------------------------------------------------------------------------------------------- the model
def logits(tokens, weights, config, dtype=torch.float64, streams=None, margins=None, probabilities=None):
    """Logits [T, vocab] of one sequence.  ``streams``: a list that receives what goes on from every layer;
    ``margins``: a list that receives every routed feed-forward's ``route_margin``; ``probabilities``: a list that
    receives every layer's attention weights [H, T, T]."""
    w = {name: t.to(dtype) for name, t in weights.items()}
    eps = config['norm']['eps']
    positions = torch.arange(len(tokens))
    x = w['embed'][torch.tensor(tokens)] * config['embedding']['scale']
    results = [x]
    for index, layer in enumerate(config['layers']):
        pre = f'l{index}.'
        h = time_convolution(x, w[pre + 'canon1'])
        mixed = latent_attention(h, w, pre + 'mix.', layer['mixer'], eps, positions, probabilities)
        x = x + w[pre + 'ls1'] * layer_norm(mixed, w[pre + 'norm1'], w[pre + 'norm1.b'], eps)
        f = layer['mlp']
        if f is not None:
            if f['kind'] == 'moe' and margins is not None:
                margins.append(route_margin(x, w, pre + 'mlp.', f['router']))
            fed = dense(x, w, pre + 'mlp.') if f['kind'] == 'dense' else moe(x, w, pre + 'mlp.', f)
            x = x + w[pre + 'ls2'] * layer_norm(fed, w[pre + 'norm2'], w[pre + 'norm2.b'], eps)
        results.append(x)
        x = sum(w[pre + 'dwa'][j] * results[j] for j in range(index + 2))
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, w['final.norm'], w['final.norm.b'], eps) @ w['embed'].t()


def greedy(prompt, count, weights, config, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(logits(tokens, weights, config, dtype)[-1].argmax()))
    return tokens[len(prompt):]


# ---------------------------------------------------------------------------------------------- configurations
def dense_mlp(ff):
    return dict(kind='dense', ff=ff)


def moe_mlp(*, ff, experts, top):
    return dict(kind='moe', expert=dict(ff=ff), router=dict(experts=experts, top=top))


def layer(*, heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, window, base=10000.0, mlp=None):
    return dict(type='latent_attention', mlp=mlp,
                mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale,
                           rot=dict(base=base, dims=rot_dim), mask=dict(size=window)))


def make_config(layers, *, vocab, width, taps, scale=1.0, eps=1e-5):
    return dict(architecture='Zinesun', vocab=vocab, width=width, embedding=dict(scale=scale), canon=dict(taps=taps),
                layers=layers, norm=dict(eps=eps))


def random_weights(config, seed, spread=1.0):
    """Tensors under the checkpoint's names, rounded to bfloat16 values (a float32 and a bfloat16 engine then read the
    same numbers).  ``spread`` scales the matrices around 1 / sqrt(fan-in)."""
    g = torch.Generator().manual_seed(seed)
    width = config['width']

    def rounded(t):
        return t.to(torch.bfloat16).to(torch.float64)

    def matrix(rows, columns, gain=1.0):
        return rounded(torch.randn(rows, columns, generator=g) * (spread * gain / math.sqrt(columns)))

    def around(centre, size, noise):
        return rounded(centre + noise * torch.randn(size, generator=g))

    w = {'embed': matrix(config['vocab'], width, 1.0), 'final.norm': around(1.0, width, 0.1),
         'final.norm.b': around(0.0, width, 0.1)}
    for index, entry in enumerate(config['layers']):
        pre, m = f'l{index}.', entry['mixer']
        heads, d, r, dv, rank, q_rank = m['heads'], m['dim'], m['rot_dim'], m['vdim'], m['kv_rank'], m['q_rank']
        w[pre + 'canon1'] = rounded(0.4 * torch.randn(width, config['canon']['taps'], generator=g))
        w[pre + 'norm1'], w[pre + 'norm1.b'] = around(1.0, width, 0.1), around(0.0, width, 0.1)
        w[pre + 'ls1'] = around(0.6, width, 0.2)
        w[pre + 'dwa'] = around(1.0 / (index + 2), index + 2, 0.15)
        w[pre + 'mix.dq'], w[pre + 'mix.dq.norm'] = matrix(q_rank, width), around(1.0, q_rank, 0.1)
        w[pre + 'mix.uq'] = matrix(heads * (d + r), q_rank, 2.0)
        w[pre + 'mix.dkv'], w[pre + 'mix.dkv.norm'] = matrix(rank + r, width), around(1.0, rank, 0.1)
        w[pre + 'mix.uk'], w[pre + 'mix.uv'] = matrix(heads * d, rank, 2.0), matrix(heads * dv, rank)
        w[pre + 'mix.g'], w[pre + 'mix.o'] = matrix(heads, width, 2.0), matrix(width, heads * dv)
        f = entry['mlp']
        if f is None:
            continue
        w[pre + 'norm2'], w[pre + 'norm2.b'] = around(1.0, width, 0.1), around(0.0, width, 0.1)
        w[pre + 'ls2'] = around(0.6, width, 0.2)
        if f['kind'] == 'dense':
            w[pre + 'mlp.up'], w[pre + 'mlp.down'] = matrix(f['ff'], width, 1.5), matrix(width, f['ff'])
            w[pre + 'mlp.act'] = around(0.0, 2, 1.0)
        else:
            experts = f['router']['experts']
            w[pre + 'mlp.router'], w[pre + 'mlp.router.b'] = matrix(experts, width, 3.0), around(0.0, experts, 0.5)
            for e in range(experts):
                w[f'{pre}mlp.e{e}.gate'] = matrix(f['expert']['ff'], width, 1.5)
                w[f'{pre}mlp.e{e}.up'] = matrix(f['expert']['ff'], width, 1.5)
                w[f'{pre}mlp.e{e}.down'] = matrix(width, f['expert']['ff'])
    return w
