"""A plain, slow Dogozen in float64: one function per mechanism, whole sequences at once or token by token.

Nothing here is shared with the engine.  ``weights`` maps checkpoint names to float64 tensors; ``config`` is the
dict of config.json.  A sequence is run alone; ``state`` (a dict per layer) carries what decoding needs, so that the
same functions serve whole prompts and single tokens.
"""
import math

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    """RMS norm whose stored weight lies around zero."""
    return rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def scaled_frequencies(dims, base, scaling):
    """Rotary frequencies with the wavelength-dependent slow-down: short waves keep their frequency, long waves are
    slowed by ``factor``, and those between are blended."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = (scaling[k] for k in ('factor', 'low', 'high', 'original'))
            wavelength = 2 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def rotate(x, positions, freqs, dims):
    """x [T, heads, d]; the first ``dims`` elements in pairs (i, i + dims / 2)."""
    half = dims // 2
    a = positions.to(F)[:, None] * freqs[None, :]              # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def attend(q, k, v, q_pos, k_pos, scale, window=None, sink=None):
    """q [T, H, d], k [S, G, d], v [S, G, dv] -> [T, H * dv]; key j is visible to query i iff j <= i and, with a window,
    i - j < window; ``sink`` [H]: one more term exp(sink) in the softmax's denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[-1], dtype=F)
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale                      # [T, S]
        diff = q_pos[:, None] - k_pos[None, :]
        visible = diff >= 0
        if window is not None:
            visible &= diff < window
        s = s.masked_fill(~visible, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].expand_as(m))
        e = torch.exp(s - m)
        denom = e.sum(-1, keepdim=True)
        if sink is not None:
            denom = denom + torch.exp(sink[h] - m)
        out[:, h] = (e / denom) @ v[:, g]
    return out.reshape(T, -1)


def query_temperature(positions, coef, every):
    return 1.0 + coef * torch.log(torch.floor((positions.to(F) + 1) / every) + 1.0)


def attention_mixer(h, positions, w, p, m, eps, state, kv_state=None):
    """The 'attention' mixer.  ``state``: {'k', 'v'} of this layer (appended to); ``kv_state``: the cache of the layer
    named by kv_from (already holding this step's tokens), used instead of keys and values of its own."""
    H, G, d, dv = m['heads'], m['kv_heads'], m['dim'], m['vdim']
    T = h.shape[0]
    q = (h @ w[p + 'q'].T + w[p + 'q.b']).reshape(T, H, d)
    q = rms(q, eps)
    if m.get('q_temp') is not None:
        q = q * query_temperature(positions, m['q_temp']['coef'], m['q_temp']['every'])[:, None, None]
    if kv_state is None:
        k = (h @ w[p + 'k'].T + w[p + 'k.b']).reshape(T, G, d)
        k = rms(k, eps)
        v = (h @ w[p + 'v'].T + w[p + 'v.b']).reshape(T, G, dv)
        state['k'] = k if 'k' not in state else torch.cat([state['k'], k])
        state['v'] = v if 'v' not in state else torch.cat([state['v'], v])
        kv_state = state
    keys, values = kv_state['k'], kv_state['v']
    out = attend(q, keys, values, positions, torch.arange(keys.shape[0]), m['scale'])
    out = out * torch.sigmoid(h @ w[p + 'g'].T)
    return out @ w[p + 'o'].T


def window_attention(h, positions, w, p, m, state):
    """The left half of the 'parallel' mixer: rotated, windowed, with a sink."""
    H, G, d, dv = m['heads'], m['kv_heads'], m['dim'], m['vdim']
    T = h.shape[0]
    freqs = scaled_frequencies(m['rot']['dims'], m['rot']['base'], m['rot'].get('scaling'))
    q = rotate((h @ w[p + 'q'].T).reshape(T, H, d), positions, freqs, m['rot']['dims'])
    k = rotate((h @ w[p + 'k'].T).reshape(T, G, d), positions, freqs, m['rot']['dims'])
    v = (h @ w[p + 'v'].T).reshape(T, G, dv)
    state['k'] = k if 'k' not in state else torch.cat([state['k'], k])
    state['v'] = v if 'v' not in state else torch.cat([state['v'], v])
    keys, values = state['k'], state['v']
    out = attend(q, keys, values, positions, torch.arange(keys.shape[0]), m['scale'], window=m['mask']['size'],
                 sink=w[p + 'sink'])
    return out @ w[p + 'o'].T


def selective_scan(h, w, p, m, state):
    """The right half: a selective state-space scan, token by token.  ``state``: {'conv': the last taps - 1 inputs of
    the convolution [taps - 1, inner], 'S': [inner, n]}."""
    inner, n, taps, rank = m['inner'], m['state'], m['conv'], m['dt_rank']
    T = h.shape[0]
    xz = h @ w[p + 'in'].T
    x, z = xz[:, :inner], xz[:, inner:]
    past = state.get('conv', torch.zeros(taps - 1, inner, dtype=F))
    padded = torch.cat([past, x])
    conv = torch.zeros(T, inner, dtype=F)
    for j in range(taps):
        conv += padded[j:j + T] * w[p + 'conv'][:, j]
    if taps > 1:
        state['conv'] = padded[-(taps - 1):]
    u = silu(conv + w[p + 'conv.b'])
    low = u @ w[p + 'x'].T
    dt = softplus(low[:, :rank] @ w[p + 'dt'].T + w[p + 'dt.b'])          # [T, inner]
    B, C = low[:, rank:rank + n], low[:, rank + n:rank + 2 * n]
    A = -torch.exp(w[p + 'A_log'])                                          # [inner, n]
    S = state.get('S', torch.zeros(inner, n, dtype=F))
    y = torch.zeros(T, inner, dtype=F)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * u[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + w[p + 'D'] * u[t]
    state['S'] = S
    return (y * silu(z)) @ w[p + 'o'].T


def parallel_mixer(h, positions, w, p, m, state):
    left = window_attention(h, positions, w, p + 'left.', m['left'], state.setdefault('left', {}))
    right = selective_scan(h, w, p + 'right.', m['right'], state.setdefault('right', {}))
    return m['left_scale'] * left + m['right_scale'] * right


def gated(h, w, p):
    return (silu(h @ w[p + 'gate'].T) * (h @ w[p + 'up'].T)) @ w[p + 'down'].T


def route(h, w, p, f):
    """(chosen [T, top], weights [T, top], margin [T]): sigmoid scores, a group's score the sum of its two largest,
    the choice among the kept groups' experts, weights the chosen scores over their sum, times the router's scale.
    ``margin``: the smallest gap that decided anything (a group kept or an expert chosen) for each token."""
    r = f['router']
    E, top = r['experts'], r['top']
    groups = r.get('groups') or {'count': 1, 'keep': 1}
    count, keep = groups['count'], groups['keep']
    s = torch.sigmoid(h @ w[p + 'router'].T)                                # [T, E]
    T = s.shape[0]
    size = E // count
    by_group = s.reshape(T, count, size)
    group_score = by_group.topk(min(2, size), dim=-1).values.sum(-1)        # [T, count]
    order = group_score.sort(dim=-1, descending=True)
    kept = order.indices[:, :keep]
    margin = torch.full((T,), math.inf, dtype=F)
    if keep < count:
        margin = order.values[:, keep - 1] - order.values[:, keep]
    allowed = torch.zeros(T, count, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = s.masked_fill(~allowed[:, :, None].expand(T, count, size).reshape(T, E), -math.inf)
    best = masked.sort(dim=-1, descending=True)
    chosen = best.indices[:, :top]
    if top < keep * size:
        margin = torch.minimum(margin, best.values[:, top - 1] - best.values[:, top])
    picked = s.gather(1, chosen)
    weights = picked / (picked.sum(-1, keepdim=True) + 1e-20) * r['scale']
    return chosen, weights, margin


def routed(h, w, p, f, margins=None):
    chosen, weights, margin = route(h, w, p, f)
    if margins is not None:
        margins.append(margin)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weights[t]):
            out[t] += g * gated(h[t:t + 1], w, f'{p}e{e}.')[0]
    if f.get('shared') is not None:
        out = out + gated(h, w, p + 'shared.')
    return out


def feed_forward(h, w, p, f, margins=None):
    return gated(h, w, p) if f['kind'] == 'dense' else routed(h, w, p, f, margins)


def forward(config, w, tokens, start=0, states=None, collect=None, margins=None):
    """Logits [T, vocab] of ``tokens`` at positions start ..; ``states``: the list (one dict a layer) that earlier calls
    for the same sequence left, or None.  ``collect``: a list that receives the residual stream after every layer;
    ``margins``: a list that receives, per routed layer, every token's smallest gap between what its router chose and
    what it did not."""
    eps = config['norm']['eps']
    states = states if states is not None else [dict() for _ in config['layers']]
    x = w['embed'][torch.as_tensor(tokens)]
    positions = torch.arange(start, start + len(tokens))
    for i, layer in enumerate(config['layers']):
        p = f'l{i}.'
        h = norm(x, w[p + 'norm1'], eps)
        if layer['type'] == 'attention':
            source = layer['mixer'].get('kv_from')
            mixed = attention_mixer(h, positions, w, p + 'mix.', layer['mixer'], eps, states[i],
                                    kv_state=states[source] if source is not None else None)
        else:
            mixed = parallel_mixer(h, positions, w, p + 'mix.', layer['mixer'], states[i])
        x = x + norm(mixed, w[p + 'norm1b'], eps)
        if layer['mlp'] is not None:
            x = x + norm(feed_forward(norm(x, w[p + 'norm2'], eps), w, p + 'mlp.', layer['mlp'], margins), w[p + 'norm2b'], eps)
        if collect is not None:
            collect.append(x.clone())
    logits = norm(x, w['final.norm'], eps) @ w['embed'].T
    cap = config.get('logit_softcap')
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits, states


# ------------------------------------------------------------------------------------------------ making models
def attention_layer(*, heads, kv_heads, dim, vdim, scale, q_temp=None, kv_from=None, mlp=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if q_temp is not None:
        mixer['q_temp'] = dict(coef=q_temp[0], every=q_temp[1])
    if kv_from is not None:
        mixer['kv_from'] = kv_from
    return dict(type='attention', mixer=mixer, mlp=mlp)


def parallel_layer(*, heads, kv_heads, dim, vdim, scale, window, rot_dims, base=10000.0, scaling=None, inner, state, conv,
                   dt_rank, left_scale=1.0, right_scale=1.0, mlp=None):
    rot = dict(base=base, dims=rot_dims)
    if scaling is not None:
        rot['scaling'] = dict(zip(('factor', 'low', 'high', 'original'), scaling))
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot, mask=dict(size=window))
    right = dict(inner=inner, state=state, conv=conv, dt_rank=dt_rank)
    return dict(type='parallel', mixer=dict(left=left, right=right, left_scale=left_scale, right_scale=right_scale), mlp=mlp)


def dense_mlp(ff):
    return dict(kind='dense', ff=ff)


def moe_mlp(*, ff, experts, top, scale=1.0, count=1, keep=1, shared=None):
    out = dict(kind='moe', expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale,
                                                          groups=dict(count=count, keep=keep)))
    if shared is not None:
        out['shared'] = dict(ff=shared)
    return out


def make_config(layers, *, vocab, width, eps=1e-5, softcap=None):
    out = dict(architecture='Dogozen', vocab=vocab, width=width, layers=layers, norm=dict(eps=eps))
    if softcap is not None:
        out['logit_softcap'] = softcap
    return out


def random_weights(config, seed, spread=1.0):
    """float64 tensors whose values bfloat16 holds exactly, by checkpoint name."""
    g = torch.Generator().manual_seed(seed)
    width = config['width']
    w = {}

    def held(t):
        return t.to(torch.bfloat16).to(F)

    def matrix(name, rows, columns, gain=1.0):
        w[name] = held(torch.randn(rows, columns, generator=g, dtype=F) * (gain * spread / math.sqrt(columns)))

    def vector(name, size, std=0.1, mean=0.0):
        w[name] = held(mean + std * torch.randn(size, generator=g, dtype=F))

    def gated_tensors(p, ff):
        matrix(p + 'gate', ff, width)
        matrix(p + 'up', ff, width)
        matrix(p + 'down', width, ff)

    w['embed'] = held(torch.randn(config['vocab'], width, generator=g, dtype=F))
    vector('final.norm', width)
    for i, layer in enumerate(config['layers']):
        p, m = f'l{i}.', layer['mixer']
        for name in ('norm1', 'norm1b') + (('norm2', 'norm2b') if layer['mlp'] is not None else ()):
            vector(p + name, width)
        if layer['type'] == 'attention':
            H, G, d, dv = m['heads'], m['kv_heads'], m['dim'], m['vdim']
            matrix(p + 'mix.q', H * d, width)
            vector(p + 'mix.q.b', H * d, 0.3)
            if m.get('kv_from') is None:
                matrix(p + 'mix.k', G * d, width)
                vector(p + 'mix.k.b', G * d, 0.3)
                matrix(p + 'mix.v', G * dv, width)
                vector(p + 'mix.v.b', G * dv, 0.3)
            matrix(p + 'mix.g', H * dv, width, 2.0)
            matrix(p + 'mix.o', width, H * dv)
        else:
            a, r = m['left'], m['right']
            H, G, d, dv = a['heads'], a['kv_heads'], a['dim'], a['vdim']
            matrix(p + 'mix.left.q', H * d, width, 2.0)
            matrix(p + 'mix.left.k', G * d, width, 2.0)
            matrix(p + 'mix.left.v', G * dv, width)
            vector(p + 'mix.left.sink', H, 1.0)
            matrix(p + 'mix.left.o', width, H * dv)
            inner, n, taps, rank = r['inner'], r['state'], r['conv'], r['dt_rank']
            matrix(p + 'mix.right.in', 2 * inner, width)
            w[p + 'mix.right.conv'] = held(torch.randn(inner, taps, generator=g, dtype=F) * 0.5)
            vector(p + 'mix.right.conv.b', inner, 0.2)
            matrix(p + 'mix.right.x', rank + 2 * n, inner, 1.5)
            matrix(p + 'mix.right.dt', inner, rank)
            vector(p + 'mix.right.dt.b', inner, 1.0, -1.0)
            w[p + 'mix.right.A_log'] = held(torch.log(torch.rand(inner, n, generator=g, dtype=F) * 4.0 + 0.05))
            vector(p + 'mix.right.D', inner, 0.5, 1.0)
            matrix(p + 'mix.right.o', width, inner)
        f = layer['mlp']
        if f is None:
            continue
        if f['kind'] == 'dense':
            gated_tensors(p + 'mlp.', f['ff'])
            continue
        matrix(p + 'mlp.router', f['router']['experts'], width, 3.0)
        for e in range(f['router']['experts']):
            gated_tensors(f'{p}mlp.e{e}.', f['expert']['ff'])
        if f.get('shared') is not None:
            gated_tensors(p + 'mlp.shared.', f['shared']['ff'])
    return w


def logits(tokens, weights, config, margins=None):
    """Logits [T, vocab] of a whole sequence (``margins`` as in ``forward``)."""
    return forward(config, weights, tokens, margins=margins)[0]


def greedy(prompt, count, weights, config):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(logits(tokens, weights, config)[-1].argmax()))
    return tokens[len(prompt):]
