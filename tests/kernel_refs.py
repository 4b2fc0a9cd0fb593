"""Plain torch references of the HIP kernels, one per op of ``qil_amd.ops``, same signatures.

Two uses: GPU tests compare each kernel with its reference here; CPU tests
substitute these for the kernels (pytest monkeypatch) to exercise the cache
manager, the step function, the scheduler and trace replay without a GPU.  They
are test code: the engine never imports them.
"""
import torch


def _value(x):
    """A tensor, or the sum of float32 partial sums."""
    return x.sum() if hasattr(x, 'splits') else x


def _round(x, dtype):
    return x.to(dtype).to(torch.float32)


def embed(token_ids, table, scale=1.0):
    return table[token_ids.long()].to(torch.float32) * scale


def _norm(x, weight, eps, out_dtype):
    n = x * torch.rsqrt(x.square().mean(dim=-1, keepdim=True) + eps)
    return (_round(n, out_dtype) * weight).to(out_dtype)


def _delta(delta):
    """What a pending sub-layer output adds: itself, or (``PostNormed``) its RMS norm in float32, unrounded."""
    if hasattr(delta, 'value') and hasattr(delta, 'eps'):
        x = _value(delta.value).to(torch.float32)
        return x * torch.rsqrt(x.square().mean(dim=-1, keepdim=True) + delta.eps) * delta.weight
    return _value(delta).to(torch.float32)


def add_rmsnorm(stream, delta, weight, eps, out_dtype):
    if delta is not None:
        stream += _delta(delta)
    return _norm(stream, weight, eps, out_dtype)


def rows_rmsnorm(stream, delta, rows, weight, eps, out_dtype):
    x = stream[rows.long()]
    if delta is not None:
        x = x + _delta(delta)[rows.long()]
    return _norm(x, weight, eps, out_dtype)


def linear(x, weight, bias=None, out_dtype=None, partials=False):
    y = x.to(torch.float32) @ weight.to(torch.float32).t()
    if bias is not None:
        y = y + bias
    return y.to(out_dtype or x.dtype)


def _halves(gate_up, interleaved):
    """(gate, up) columns of [N, 2 I]: stacked, or in turns of 16 columns."""
    inner = gate_up.shape[1] // 2
    if not interleaved:
        return gate_up[:, :inner], gate_up[:, inner:]
    tiles = gate_up.reshape(gate_up.shape[0], inner // 16, 2, 16)
    return tiles[:, :, 0].reshape(-1, inner), tiles[:, :, 1].reshape(-1, inner)


def _gate(g, u, activation='silu', limit=0.0, alpha=1.0):
    if activation == 'clamped_swish':
        g, u = g.clamp(max=limit), u.clamp(min=-limit, max=limit)
        return g / (1 + torch.exp(-alpha * g)) * (u + 1)
    return g / (1 + torch.exp(-g)) * u


def gated_linear(x, weight, out_dtype=None, interleaved=False, lazy=False, activation='silu', limit=0.0, alpha=1.0):
    y = x.to(torch.float32) @ weight.to(torch.float32).t()
    g, u = _halves(y, interleaved)
    return _gate(g, u, activation, limit, alpha).to(out_dtype or x.dtype)


def silu_mul(gate_up, out_dtype=None, interleaved=False):
    gate_up = _value(gate_up)
    g, u = (t.to(torch.float32) for t in _halves(gate_up, interleaved))
    return (g / (1 + torch.exp(-g)) * u).to(out_dtype or gate_up.dtype)


def qk_norm_rope_store(qkv, *, heads, kv_heads, head_dim, q_weight, k_weight, eps, rotation, positions, slots,
                       k_cache, v_cache, page_size, dtype, norm_dim=None, rotate_first=False, extra_columns=0,
                       q_temperature=None, bias=None):
    qkv = _value(qkv)
    n, d = qkv.shape[0], head_dim
    x = qkv[:, :(heads + 2 * kv_heads) * d]
    if bias is not None:
        x = x.to(torch.float32) + bias
    x = x.reshape(n, heads + 2 * kv_heads, d)
    q, k, v = x[:, :heads].to(torch.float32), x[:, heads:heads + kv_heads].to(torch.float32), x[:, heads + kv_heads:]

    def normed(t, weight):
        if weight is None:
            return t
        return _round(t * torch.rsqrt(t.square().sum(dim=-1, keepdim=True) / (norm_dim or d) + eps), dtype) * weight

    def turned(t):
        if rotation is None:
            return t
        rot, half = rotation.rot_dim, rotation.rot_dim // 2
        if getattr(rotation, 'frequencies', None) is not None:
            angle = positions.to(torch.float32)[:, None] * rotation.frequencies[None, :]
            c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
        else:
            c = rotation.cos[positions.long()][:, None, :]
            s = rotation.sin[positions.long()][:, None, :]
        left, right = t[..., :half], t[..., half:rot]
        return torch.cat((left * c - right * s, left * s + right * c, t[..., rot:]), dim=-1)

    def shape(t, weight):
        return (normed(turned(t), weight) if rotate_first else turned(normed(t, weight))).to(dtype)

    if slots is not None:
        page, offset = slots.long() // page_size, slots.long() % page_size
        k_cache[page, :, offset] = shape(k, k_weight)
        v_cache[page, :, :, offset] = v.to(dtype)        # V is [pages, kv_heads, d, page_size]
    if q_temperature is not None:
        coef, every = q_temperature
        factor = 1.0 + coef * torch.log(torch.div(positions + 1, every, rounding_mode='floor').to(torch.float32) + 1.0)
        # the factor multiplies in float32, before the one rounding of the stored query
        plain = normed(turned(q), q_weight) if rotate_first else turned(normed(q, q_weight))
        return (plain * factor[:, None, None]).to(dtype).reshape(n, heads * d)
    return shape(q, q_weight).reshape(n, heads * d)


def paged_attention(q, *, heads, kv_heads, head_dim, k_cache, v_cache, page_size, block_tables, row_seq, positions,
                    cu_seqlens, seq_starts, single_rows, n_seqs, max_query, max_context, scale, window,
                    unmerged=False, tile_seqs=None, softcap=None, sinks=None, accumulate=torch.float32):
    n, d, g = q.shape[0], head_dim, heads // kv_heads
    qkv = q
    q = q.reshape(n, heads, d).to(accumulate)
    out = torch.empty((n, heads, d), dtype=accumulate, device=qkv.device)
    for row in range(n):
        ctx = int(positions[row]) + 1
        lo = max(0, ctx - window) if window else 0
        j = torch.arange(lo, ctx, device=qkv.device)
        pages = block_tables[int(row_seq[row])].long()[j // page_size]
        keys = k_cache[pages, :, j % page_size].to(accumulate)          # [ctx, kv_heads, d]
        values = v_cache[pages, :, :, j % page_size].to(accumulate)     # [ctx, kv_heads, d]
        keys = keys.repeat_interleave(g, dim=1)
        values = values.repeat_interleave(g, dim=1)
        scores = torch.einsum('hd,jhd->hj', q[row], keys) * scale
        if softcap:
            scores = softcap * torch.tanh(scores / softcap)
        if sinks is not None:                        # one more term in the divisor: no key, no value
            scores = torch.cat([scores, sinks.to(accumulate)[:, None]], dim=-1)
            out[row] = torch.einsum('hj,jhd->hd', torch.softmax(scores, dim=-1)[:, :-1], values)
            continue
        out[row] = torch.einsum('hj,jhd->hd', torch.softmax(scores, dim=-1), values)
    return out.reshape(n, heads * d).to(qkv.dtype)


def _uniform(seed, counter, vocab, device):
    i = torch.arange(vocab, dtype=torch.int64, device=device)
    offset = (((int(seed) & 0xFFFFFFFF) * 0x85EBCA77) + ((int(counter) & 0xFFFFFFFF) * 0xC2B2AE3D)) & 0xFFFFFFFF
    x = (i * 0x9E3779B1 + offset) & 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return ((x >> 8).to(torch.float32) + 0.5) * (1.0 / 16777216.0)


def sample_scores(logits, temperatures, seeds, counters):
    """The perturbed scores whose argmax is the draw (plain logits for temperature 0)."""
    rows = []
    for r in range(logits.shape[0]):
        t = float(temperatures[r])
        if t > 0:
            u = _uniform(int(seeds[r]), int(counters[r]), logits.shape[1], logits.device)
            rows.append(logits[r] / t - torch.log(-torch.log(u)))
        else:
            rows.append(logits[r])
    return torch.stack(rows)


def sample(logits, temperatures, seeds, counters, out=None):
    scores = sample_scores(logits, temperatures, seeds, counters)
    finite = torch.isfinite(logits).all(dim=-1).to(torch.int32)
    tokens = scores.argmax(dim=-1).to(torch.int32)
    if out is not None:
        out[0], out[1] = tokens, finite
        return out[0], out[1]
    return tokens, finite


def _any_norm(x, weight, eps, centre):
    if centre:
        x = x - x.mean(dim=-1, keepdim=True)
    return x / torch.sqrt(x.square().mean(dim=-1, keepdim=True) + eps) * weight


def add_norm(stream, delta, weight, eps, out_dtype, *, centre, delta_scale=1.0, bias=None):
    if delta is not None:
        stream += delta_scale * _value(delta).to(torch.float32)
    return (_any_norm(stream, weight, eps, centre) + (bias if bias is not None else 0.0)).to(out_dtype)


def rows_norm(stream, delta, rows, weight, eps, out_dtype, *, centre, delta_scale=1.0, bias=None):
    x = stream[rows.long()]
    if delta is not None:
        x = x + delta_scale * _value(delta)[rows.long()].to(torch.float32)
    return (_any_norm(x, weight, eps, centre) + (bias if bias is not None else 0.0)).to(out_dtype)


def plain_act(x, out_dtype, *, activation, params=None):
    z = _value(x).to(torch.float32)
    if activation == 'gelu_tanh':
        return (0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))).to(out_dtype)
    soft = torch.nn.functional.softplus(params)
    below = z.clamp(max=0.0)
    return torch.where(z > 0, soft[0] * z * z + 0.5 * z, (0.5 + soft[1]) * (torch.expm1(below) - below) + 0.5 * z).to(out_dtype)


def post_norm_scale_add(stream, value, *, weight, bias, channel_scale, eps, centre, out_dtype=None, history=None, depth=0,
                        mix=None):
    y = _value(value).to(torch.float32)
    if centre:
        y = y - y.mean(dim=-1, keepdim=True)
    z = y / torch.sqrt(y.square().mean(dim=-1, keepdim=True) + eps)
    if weight is not None:
        z = z * weight
    if bias is not None:
        z = z + bias
    if channel_scale is not None:
        z = z * channel_scale
    stream += z
    if depth:
        history[depth - 1] = stream
        stream.copy_((mix[:depth, None, None] * history[:depth]).sum(dim=0))
    return stream.to(out_dtype) if out_dtype is not None else None


def short_conv(x, weight, *, state, cu_seqlens, seq_starts, seq_slots, row_seq, n_seqs, out_dtype):
    taps, keep = weight.shape[0], weight.shape[0] - 1               # weight [taps, H]
    out = torch.empty_like(x)
    for s in range(n_seqs):
        first, last, start = int(cu_seqlens[s]), int(cu_seqlens[s + 1]), int(seq_starts[s])
        before = torch.zeros((keep, x.shape[1]), dtype=torch.float32)
        if keep and start > 0:
            before = state[int(seq_slots[s])].clone()
            before[:max(0, keep - start)] = 0.0                 # places before the sequence's start
        inputs = torch.cat([before, x[first:last]])
        rows = last - first
        out[first:last] = x[first:last] + sum(weight[j] * inputs[j:j + rows] for j in range(taps))
        if keep:
            state[int(seq_slots[s])] = inputs[-keep:]
    return out.to(out_dtype)


def gated_act(gate_up, out_dtype, *, activation, limit=0.0, alpha=1.0, interleaved=False):
    g, u = (t.to(torch.float32) for t in _halves(_value(gate_up), interleaved))
    return _gate(g, u, activation, limit, alpha).to(out_dtype)


def _turn(x, positions, frequencies):
    """x [N, ..., rot]: element i with i + rot / 2, angle position * frequencies[i]; float32."""
    half = x.shape[-1] // 2
    angle = positions.to(torch.float32)[:, None] * frequencies[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = angle.cos().reshape(shape), angle.sin().reshape(shape)
    u, v = x[..., :half], x[..., half:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin], dim=-1)


def latent_prepare(down, *, q_rank, rank, rot, q_weight, c_weight, eps, frequencies, positions, slots, latent, rope,
                   dtype, gates=0):
    x = _value(down).to(torch.float32)
    cq = _any_norm(x[:, :q_rank], q_weight, eps, False).to(dtype)
    if slots is not None:
        latent.view(-1, rank)[slots.long()] = _any_norm(x[:, q_rank:q_rank + rank], c_weight, eps, False).to(dtype)
        rope.view(-1, rot)[slots.long()] = _turn(x[:, q_rank + rank:q_rank + rank + rot], positions, frequencies).to(dtype)
    return (cq, torch.sigmoid(x[:, q_rank + rank + rot:])) if gates else cq


def head_product(x, weight, *, heads, out_dtype, out=None, out_columns=None):
    n, k, o = x.shape[0], weight.shape[1], weight.shape[2]
    result = torch.einsum('nhk,hko->nho', x.to(torch.float32).view(n, heads, -1)[:, :, :k], weight.to(torch.float32))
    if out is None:
        return result.reshape(n, heads * o).to(out_dtype)
    out.view(n, heads, out_columns)[:, :, :o] = result.to(out_dtype)
    return out


def latent_query(q, k_up, *, heads, dim, rot, rank, frequencies, positions):
    n = q.shape[0]
    q = q.to(torch.float32).view(n, heads, dim + rot)
    absorbed = torch.einsum('nhd,hdr->nhr', q[:, :, :dim], k_up.to(torch.float32))
    return torch.cat([absorbed, _turn(q[:, :, dim:], positions, frequencies)], dim=-1).reshape(n, heads * (rank + rot))


def latent_attention(q, *, latent, rope, page_size, block_tables, row_seq, positions, sink, scale, heads, rank, rot,
                     window=None, gate=None, **step):
    n = q.shape[0]
    q = q.view(n, heads, rank + rot)
    out = torch.zeros((n, heads, rank), dtype=torch.float32)
    flat_c, flat_r = latent.view(-1, rank).to(torch.float32), rope.view(-1, rot).to(torch.float32)
    for row in range(n):
        place = int(positions[row])
        keys = torch.arange(max(0, place - window + 1) if window else 0, place + 1)
        table = block_tables[int(row_seq[row])].long()
        slots = table[keys // page_size] * page_size + keys % page_size
        c, r = flat_c[slots], flat_r[slots]
        scores = (q[row, :, :rank] @ c.t() + q[row, :, rank:] @ r.t()) * scale                  # [heads, keys]
        if sink is not None:
            scores = torch.cat([scores, sink[:, None]], dim=1)
        p = torch.softmax(scores, dim=1)[:, :len(keys)]
        out[row] = p @ c
        if gate is not None:
            out[row] *= gate[row, :, None]
    return out.reshape(n, heads * rank)


def state_scan_slot(*, heads, dim, vdim, mode):
    tiles = -(-vdim // 16)
    return heads * dim * vdim + (heads * (dim + tiles + 1) if mode == 'mlstm' else 0)


def state_scan(proj, *, mode, heads, dim, vdim, q_offset, k_offset, v_offset, state, cu_seqlens, seq_starts, seq_slots,
               n_seqs, gates=None, gate_bias=None, cap=0.0, decay=None, frequencies=None, rot=0, q_scale=1.0, k_scale=1.0,
               max_query=None):
    """Token by token whatever ``max_query`` says.  -> (o, denominators): for 'mlstm' o is undivided and the denominators are returned beside it.  The state slot's
    layout is the kernel's: matrices, then a normaliser per head, then the maximum tiles + 1 times per head."""
    n, tiles = proj.shape[0], -(-vdim // 16)
    x = proj.to(torch.float32)
    q = x[:, q_offset:q_offset + heads * dim].reshape(n, heads, dim).clone()
    k = x[:, k_offset:k_offset + heads * dim].reshape(n, heads, dim).clone()
    v = x[:, v_offset:v_offset + heads * vdim].reshape(n, heads, vdim)
    out = torch.zeros((n, heads, vdim), dtype=torch.float32)
    below = torch.zeros((n, heads), dtype=torch.float32) if mode == 'mlstm' else None
    mats = heads * dim * vdim
    for s in range(n_seqs):
        lo, hi, start, slot = int(cu_seqlens[s]), int(cu_seqlens[s + 1]), int(seq_starts[s]), int(seq_slots[s])
        positions = torch.arange(start, start + hi - lo)
        qs, ks = q[lo:hi], k[lo:hi]
        if rot:
            qs = torch.cat([_turn(qs[..., :rot], positions, frequencies), qs[..., rot:]], dim=-1)
            ks = torch.cat([_turn(ks[..., :rot], positions, frequencies), ks[..., rot:]], dim=-1)
        qs, ks = qs * q_scale, ks * k_scale
        fresh = start == 0
        memory = torch.zeros(heads, dim, vdim) if fresh else state[slot, :mats].view(heads, dim, vdim).clone()
        if mode == 'mlstm':
            norms = state[slot, mats:mats + heads * dim].view(heads, dim)
            tops = state[slot, mats + heads * dim:].view(heads, tiles + 1)
            norm = torch.zeros(heads, dim) if fresh else norms.clone()
            top = torch.zeros(heads) if fresh else tops[:, 0].clone()
        for t in range(hi - lo):
            if mode == 'mlstm':
                pre = gates[lo + t] + gate_bias
                log_in = cap * torch.tanh(pre[:heads] / cap)
                log_keep = torch.nn.functional.logsigmoid(cap * torch.tanh(pre[heads:] / cap))
                now = torch.maximum(log_keep + top, log_in)
                a, b, top = torch.exp(log_keep + top - now), torch.exp(log_in - now), now
            elif mode == 'channel':                  # a decay per row of the memory: sigmoid(z)^(1 / tau)
                a = torch.exp(torch.nn.functional.logsigmoid(gates[lo + t].view(heads, dim)) / cap)[:, :, None]
                b = torch.ones(heads)
                memory = a * memory + ks[t][:, :, None] * v[lo + t][:, None, :]
                out[lo + t] = torch.einsum('hdv,hd->hv', memory, qs[t])
                continue
            else:
                a, b = decay, torch.ones(heads)
            memory = a[:, None, None] * memory + b[:, None, None] * ks[t][:, :, None] * v[lo + t][:, None, :]
            read = torch.einsum('hdv,hd->hv', memory, qs[t])
            if mode == 'mlstm':
                norm = a[:, None] * norm + b[:, None] * ks[t]
                below[lo + t] = torch.maximum((norm * qs[t]).sum(-1).abs(), torch.exp(-top)) + 1e-6
            out[lo + t] = read
        state[slot, :mats] = memory.reshape(-1)
        if mode == 'mlstm':
            norms[:] = norm
            tops[:] = top[:, None]
    return out.reshape(n, heads * vdim), below


def head_norm_gate(o, gate_source, *, gate_offset, heads, vdim, weight, eps, gate, out_dtype, denominators=None):
    n = o.shape[0]
    unit = o.view(n, heads, vdim)
    if denominators is not None:
        unit = unit / denominators[:, :, None]
    unit = (unit / torch.sqrt(unit.square().mean(dim=-1, keepdim=True) + eps)).reshape(n, heads * vdim)
    if weight is not None:
        unit = unit * weight
    g = gate_source[:, gate_offset:gate_offset + heads * vdim].to(torch.float32)
    return (unit * (torch.sigmoid(g) if gate == 'sigmoid' else g * torch.sigmoid(g))).to(out_dtype)


def moe_route(x, router, correction, *, groups, keep, top, renormalize=False, bias=None, score='softmax',
              group_score='max', weight_scale=1.0, renormalize_eps=0.0):
    logits = x.to(torch.float32) @ router.t() + (bias if bias is not None else 0.0)
    if score == 'sigmoid':
        scores = torch.sigmoid(logits)
        choice = scores + correction if correction is not None else scores.clone()
    else:
        scores = torch.softmax(logits, dim=-1)
        choice = scores + correction if correction is not None else logits.clone()
    n, outputs = scores.shape
    if groups > 1 and keep < groups:
        by_group = choice.view(n, groups, outputs // groups)
        if group_score == 'top2' and outputs // groups > 1:
            best = by_group.topk(2, dim=-1).values.sum(dim=-1)
        else:
            best = by_group.max(dim=-1).values
        kept = torch.zeros_like(best, dtype=torch.bool).scatter_(1, best.topk(keep, dim=-1).indices, True)
        choice = choice.masked_fill(~kept.repeat_interleave(outputs // groups, dim=1), float('-inf'))
    chosen = choice.topk(top, dim=-1).indices
    weights = scores.gather(1, chosen)
    if renormalize:
        weights = weights / (weights.sum(dim=-1, keepdim=True) + renormalize_eps)
    return chosen.to(torch.int32), weights * weight_scale


def moe_experts(x, chosen, weights, gate_up, down, *, activation, limit=0.0, alpha=1.0, lazy=False):
    """float32 [N, width]; the hidden activations pass through x's type as the kernel's do."""
    n, width = x.shape
    experts = gate_up.shape[0]
    xf = x.to(torch.float32)
    out = torch.zeros((n, width), dtype=torch.float32)
    for row in range(n):
        for slot in range(chosen.shape[1]):
            e = int(chosen[row, slot])
            if e >= experts:
                out[row] += weights[row, slot] * xf[row]
                continue
            g, u = gate_up[e, 0].to(torch.float32) @ xf[row], gate_up[e, 1].to(torch.float32) @ xf[row]
            hidden = _round(_gate(g, u, activation, limit, alpha), x.dtype)
            out[row] += weights[row, slot] * (down[e].to(torch.float32) @ hidden)
    return out


def scaled_sum(a, b, a_scale, b_scale):
    if hasattr(a, 'materialize'):
        a = a.materialize()
    return a_scale * _value(a).to(torch.float32) + b_scale * _value(b).to(torch.float32)


def sigmoid_gate(x, source, *, offset):
    gate = _value(source)[:, offset:offset + x.shape[1]].to(torch.float32)
    return (x.to(torch.float32) * torch.sigmoid(gate)).to(x.dtype)


def soft_cap(x, cap):
    return x.copy_(cap * torch.tanh(x / cap))


def check_selective_scan_geometry(*, inner, state, taps):
    pass


def channel_conv(x, weight, bias, *, columns, state, cu_seqlens, seq_starts, seq_slots, row_seq, n_seqs, activation,
                 out_dtype):
    x = _value(x)[:, :columns].to(torch.float32)
    taps, keep = weight.shape[0], weight.shape[0] - 1               # weight [taps, C]
    out = torch.empty_like(x)
    for s in range(n_seqs):
        first, last, start = int(cu_seqlens[s]), int(cu_seqlens[s + 1]), int(seq_starts[s])
        before = torch.zeros((keep, columns), dtype=torch.float32)
        if keep and start > 0:
            before = state[int(seq_slots[s])].clone()
            before[:max(0, keep - start)] = 0.0                 # places before the sequence's start
        inputs = torch.cat([before, x[first:last]])
        rows = last - first
        total = sum(weight[j] * inputs[j:j + rows] for j in range(taps))
        if bias is not None:
            total = total + bias
        out[first:last] = total * torch.sigmoid(total) if activation == 'silu' else total
        if keep:
            state[int(seq_slots[s])] = inputs[-keep:]
    return out.to(out_dtype)


def selective_scan(u, dt, bc, gate, *, dt_bias, a, d, state, gate_offset, cu_seqlens, seq_starts, seq_slots, n_seqs,
                   out_dtype, max_query=None):
    n, channels = u.shape
    states = a.shape[1]
    uf, dtf, bcf = u.to(torch.float32), _value(dt).to(torch.float32), _value(bc).to(torch.float32)
    z = _value(gate)[:, gate_offset:gate_offset + channels].to(torch.float32)
    step = torch.nn.functional.softplus(dtf + dt_bias, threshold=20.0)
    y = torch.empty((n, channels), dtype=torch.float32)
    for s in range(n_seqs):
        first, last = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        S = state[int(seq_slots[s])].clone() if int(seq_starts[s]) > 0 else torch.zeros((channels, states))
        for t in range(first, last):
            S = torch.exp(step[t][:, None] * a) * S + (step[t] * uf[t])[:, None] * bcf[t, :states][None, :]
            y[t] = S @ bcf[t, states:] + d * uf[t]
        state[int(seq_slots[s])] = S
    return (y * z * torch.sigmoid(z)).to(out_dtype)


ALL = dict(scaled_sum=scaled_sum, sigmoid_gate=sigmoid_gate, soft_cap=soft_cap, channel_conv=channel_conv,
           selective_scan=selective_scan, check_selective_scan_geometry=check_selective_scan_geometry,
           moe_route=moe_route, moe_experts=moe_experts, embed=embed, add_rmsnorm=add_rmsnorm, rows_rmsnorm=rows_rmsnorm, linear=linear, gated_linear=gated_linear, silu_mul=silu_mul,
           qk_norm_rope_store=qk_norm_rope_store, paged_attention=paged_attention, sample=sample,
           add_norm=add_norm, rows_norm=rows_norm, gated_act=gated_act, latent_prepare=latent_prepare, head_product=head_product,
           latent_query=latent_query, latent_attention=latent_attention, state_scan_slot=state_scan_slot, state_scan=state_scan,
           head_norm_gate=head_norm_gate, plain_act=plain_act, post_norm_scale_add=post_norm_scale_add, short_conv=short_conv)
