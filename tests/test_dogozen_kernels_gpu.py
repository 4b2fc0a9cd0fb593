"""The kernels the Dogozen design added or changed, each alone against its plain reference (``kernel_refs``) on the same
inputs: sinks in the attention kernels (rows alone, portions, keys in one piece and in parts, windows), the q/k kernel
with a query temperature, columns to skip and rows of queries only, the output gate, the weighted sum of two branches,
the logits' cap, the channel convolution with a bias and an activation and its state, the selective scan and its state,
and the router with sigmoid scores and groups judged by their two best."""
import pytest
import torch

import kernel_refs as refs
from qil_amd import ops
from test_kernels_gpu import build_cache

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def close(actual, expected, dtype, scale=1.0):
    tolerance = dict(atol=2e-5 * scale, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2 * scale, rtol=2e-2)
    torch.testing.assert_close(actual.float().cpu(), expected.float(), **tolerance)


def ints(values):
    return torch.tensor(values, dtype=torch.int32)


def partials(x, splits, g):
    """float32 partial sums [splits, ...] whose sum is x (or x itself, in its type, for splits == 0)."""
    if splits == 0:
        return x
    parts = torch.randn(splits, *x.shape, generator=g)
    parts[0] += x.float() - parts.sum(dim=0)
    return ops.Partials(parts)


def moved(x):
    return ops.Partials(x.tensor.cuda()) if isinstance(x, ops.Partials) else x.cuda()


class HostPartials:
    def __init__(self, p):
        self.tensor, self.splits, self.shape = p.tensor, p.splits, p.shape

    def sum(self):
        return self.tensor.sum(dim=0)


def host(x):
    return HostPartials(x) if isinstance(x, ops.Partials) else x


# ------------------------------------------------------------------------------------------------ sinks
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('lengths,chunks,page_size,d,heads,kv_heads,window', [
    ([70, 33, 5], [1, 1, 1], 16, 56, 6, 3, 37),                 # rows alone, a window
    ([1500, 40], [1, 1], 16, 64, 4, 2, None),                   # a long context: the keys in parts, merged
    ([2100], [1], 8, 128, 16, 8, 300),
    ([300, 2], [1, 1], 4, 24, 5, 1, 7),                         # sizes the matrix-core decode kernel does not take
    ([70, 70, 5, 33], [70, 2, 5, 17], 16, 56, 6, 3, 37),        # portions
    ([129, 64, 1000, 16], [129, 1, 3, 16], 16, 128, 8, 2, None),
    ([257, 100], [200, 31], 3, 40, 6, 2, 64),
    ([513], [513], 16, 64, 4, 2, 100),
    ([1200], [1200], 16, 128, 4, 2, 300),                       # the bfloat16 kernel for heads of 128, a long prompt
    ([1500, 900], [700, 900], 16, 128, 8, 8, None),
    ([1100], [1100], 16, 64, 4, 1, 512),
])
def test_attention_with_sinks(dtype, lengths, chunks, page_size, d, heads, kv_heads, window, monkeypatch):
    """One more term exp(sink) in every head's divisor, sinks from far below to far above the scores; with the keys in
    one piece and (forced, for the portions) in parts."""
    k_cache, v_cache, table, _ = build_cache(lengths, page_size, kv_heads, d, dtype)
    g = torch.Generator().manual_seed(d)
    starts = [n - c for n, c in zip(lengths, chunks)]
    positions = [p for s, c in zip(starts, chunks) for p in range(s, s + c)]
    row_seq = [i for i, c in enumerate(chunks) for _ in range(c)]
    cu = [0]
    for c in chunks:
        cu.append(cu[-1] + c)
    single = [cu[i] for i, c in enumerate(chunks) if c == 1]
    n = cu[-1]
    q = torch.randn(n, heads * d, generator=g).to(dtype)
    sinks = torch.linspace(-8.0, 8.0, heads)
    common = dict(heads=heads, kv_heads=kv_heads, head_dim=d, page_size=page_size, n_seqs=len(lengths),
                  max_query=max(chunks), max_context=max(lengths), scale=0.3, window=window)
    index = dict(block_tables=table.cpu(), row_seq=ints(row_seq), positions=ints(positions), cu_seqlens=ints(cu),
                 seq_starts=ints(starts), single_rows=ints(single) if max(chunks) > 1 else None)
    want = refs.paged_attention(q, k_cache=k_cache.cpu(), v_cache=v_cache.cpu(), sinks=sinks, accumulate=torch.float64,
                                **index, **common)
    without = refs.paged_attention(q, k_cache=k_cache.cpu(), v_cache=v_cache.cpu(), accumulate=torch.float64, **index, **common)
    assert (want.float() - without.float()).abs().max() > 0.05
    on_gpu = {k: None if v is None else v.cuda() for k, v in index.items()}
    for forced in (None, (64, 2)):
        if forced is not None and max(chunks) == 1:
            continue
        monkeypatch.setattr(ops, 'TILE_KEY_PARTS', forced)
        got = ops.paged_attention(q.cuda(), k_cache=k_cache, v_cache=v_cache, sinks=sinks.cuda(), **on_gpu, **common)
        assert torch.isfinite(got.float()).all()
        close(got, want, dtype, 0.3)


# ------------------------------------------------------------------------------------------------ the q/k kernel
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('heads,kv_heads,d,rot,extra,splits', [(4, 2, 64, 32, 256, 0), (6, 3, 56, 56, 0, 3), (3, 0, 24, 0, 72, 0),
                                                               (2, 0, 128, 0, 0, 2), (5, 5, 16, 0, 80, 1)])
def test_queries_with_a_temperature_and_columns_to_skip(dtype, heads, kv_heads, d, rot, extra, splits):
    if dtype == torch.float32 and splits == 0:
        splits = 1
    g = torch.Generator().manual_seed(heads * d)
    n, page_size, pages = 37, 8, 12
    positions = ints(sorted(torch.randint(0, 90, (n,), generator=g).tolist()))
    slots = torch.randperm(pages * page_size, generator=g)[:n].to(torch.int32)
    x = (torch.randn(n, (heads + 2 * kv_heads) * d + extra, generator=g)).to(dtype)
    qkv = partials(x, splits, g)
    ones = torch.ones(d)
    rotation = None
    if rot:
        from qil_amd.parts import RotaryFrequencies
        rotation = RotaryFrequencies(rot, 300.0, scaling=(4.0, 1.0, 4.0, 64)).rotation()
    caches = [torch.zeros(pages, max(kv_heads, 1), page_size, d).to(dtype), torch.zeros(pages, max(kv_heads, 1), d, page_size).to(dtype)]
    bias = torch.randn((heads + 2 * kv_heads) * d, generator=g)
    args = dict(heads=heads, kv_heads=kv_heads, head_dim=d, eps=1e-5, page_size=page_size, dtype=dtype, extra_columns=extra,
                q_temperature=(0.6, 7))
    kc, vc = caches[0].clone(), caches[1].clone()
    want = refs.qk_norm_rope_store(host(qkv), q_weight=ones, k_weight=ones, rotation=rotation, positions=positions,
                                   slots=slots if kv_heads else None, k_cache=kc, v_cache=vc, bias=bias, **args)
    gk, gv = caches[0].cuda(), caches[1].cuda()
    if rotation is not None:
        rotation = type(rotation)(None, None, rotation.rot_dim, rotation.frequencies.cuda())
    got = ops.qk_norm_rope_store(moved(qkv), q_weight=ones.cuda(), k_weight=ones.cuda(), rotation=rotation,
                                 positions=positions.cuda(), slots=slots.cuda() if kv_heads else None, k_cache=gk, v_cache=gv,
                                 bias=bias.cuda(), **args)
    close(got, want, dtype, 3.0)
    plain_args = dict(args, q_temperature=None)
    cold = refs.qk_norm_rope_store(host(qkv), q_weight=ones, k_weight=ones, rotation=None, positions=positions, slots=None,
                                   k_cache=kc, v_cache=vc, **plain_args)
    assert (want.float() - cold.float()).abs().max() > 0.3                 # the temperature is there
    if kv_heads:
        close(gk, kc, dtype)
        close(gv, vc, dtype)


# ------------------------------------------------------------------------------------------------ small steps
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('splits', [0, 1, 4])
def test_gate_sum_and_cap(dtype, splits):
    g = torch.Generator().manual_seed(splits)
    n, columns, width, offset = 19, 40, 136, 88
    x = torch.randn(n, columns, generator=g).to(dtype)
    source = partials((torch.randn(n, width, generator=g) * 3).to(dtype), splits, g)
    close(ops.sigmoid_gate(x.cuda(), moved(source), offset=offset), refs.sigmoid_gate(x, host(source), offset=offset), dtype)
    a = partials(torch.randn(n, width, generator=g).to(dtype), splits, g)
    b = partials(torch.randn(n, width, generator=g).to(dtype), 0 if splits == 4 else 2, g)
    got = ops.scaled_sum(moved(a), moved(b), 0.6, -1.5)
    assert got.dtype == torch.float32
    close(got, refs.scaled_sum(host(a), host(b), 0.6, -1.5), torch.float32, 4.0)
    logits = torch.randn(7, 301, generator=g) * 40
    close(ops.soft_cap(logits.clone().cuda(), 30.0), 30.0 * torch.tanh(logits / 30.0), torch.float32, 10.0)


# ------------------------------------------------------------------------------------------------ channel convolution
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('channels,taps,splits', [(20, 4, 0), (21, 1, 2), (7, 2, 1), (328, 4, 0), (300, 3, 3), (1028, 6, 0),
                                                  (64, 4, 2), (1024, 2, 0), (8, 5, 1)])
def test_channel_convolution_with_its_state(dtype, channels, taps, splits):
    """Steps over five slots: sequences that begin (whatever their slot held before, NaN here, is not read), that
    continue from a state shorter than taps - 1 inputs, that bring fewer rows than the state holds, and one long
    portion; a slot is given to a new sequence.  The input is the first columns of a wider product."""
    if dtype == torch.float32 and splits == 0:
        splits = 1
    g = torch.Generator().manual_seed(channels * 10 + taps)
    keep, width = taps - 1, 2 * channels + (3 if channels % 4 else 8)
    weight, bias = torch.randn(taps, channels, generator=g), torch.randn(channels, generator=g)
    state_c = torch.full((5, keep, channels), float('nan')) if keep else None
    state_g = state_c.clone().cuda() if keep else None
    steps = [([5, 1, 2], [0, 0, 0], [3, 0, 4]), ([1, 1, 70], [5, 1, 2], [3, 0, 4]), ([2, 1, 3, 1], [6, 2, 0, 72], [3, 0, 1, 4]),
             ([9, 2], [0, 8], [0, 3]), ([300, 1, 2, 9, 30], [10, 9, 0, 0, 0], [3, 0, 1, 2, 4])]
    for counts, starts, slots in steps:
        n = sum(counts)
        x = partials(torch.randn(n, width, generator=g).to(dtype), splits, g)
        cu = ints([0] + torch.tensor(counts).cumsum(0).tolist())
        row_seq = ints([s for s, c in enumerate(counts) for _ in range(c)])
        args = dict(cu_seqlens=cu, seq_starts=ints(starts), seq_slots=ints(slots), row_seq=row_seq)
        common = dict(columns=channels, n_seqs=len(counts), activation='silu', out_dtype=dtype)
        want = refs.channel_conv(host(x), weight, bias, state=state_c, **args, **common)
        got = ops.channel_conv(moved(x), weight.cuda(), bias.cuda(), state=state_g, **{k: v.cuda() for k, v in args.items()}, **common)
        assert torch.isfinite(got.float()).all()
        close(got, want, dtype, 4.0)
        if keep:
            used = sorted(slots)
            close(state_g[used], state_c[used], torch.float32, 1.0 if dtype == torch.float32 else 1e3)
            others = [s for s in range(5) if s not in used]
            assert torch.equal(state_g[others].cpu().isnan(), state_c[others].isnan())


# ------------------------------------------------------------------------------------------------ selective scan
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('channels,states,splits', [(20, 4, 0), (16, 16, 2), (33, 17, 1), (336, 20, 0), (7, 1, 3), (40, 70, 0),
                                                    (24, 130, 1)])
def test_selective_scan_with_its_state(dtype, channels, states, splits):
    """Steps over four slots: sequences that begin, continue, bring one row or many (up to 64 rows of every sequence
    the step walks each in one piece, beyond that in chunks of 64 tokens side by side, with sequences of one chunk and
    of a chunk's exact length among them); lanes past the last channel and past the last state, more states than the
    form with a thread a channel takes; inputs as tensors and as partial sums."""
    if dtype == torch.float32 and splits == 0:
        splits = 1
    g = torch.Generator().manual_seed(channels + states)
    a = -torch.exp(torch.randn(channels, states, generator=g))
    dt_bias, d = torch.randn(channels, generator=g) - 1.0, torch.randn(channels, generator=g)
    state_c = torch.full((4, channels, states), float('nan'))
    state_g = state_c.clone().cuda()
    gate_width, offset = 2 * channels + 5, channels + 2
    steps = [([5, 1], [0, 0], [3, 0]), ([1, 1, 70], [5, 1, 0], [3, 0, 2]), ([2, 130, 1], [6, 0, 70], [3, 1, 2]),
             ([1, 1, 1, 1], [8, 2, 71, 130], [3, 0, 2, 1]), ([9], [0], [0]), ([64, 64, 3], [9, 9, 72], [0, 3, 2]),
             ([65, 300, 128, 1], [73, 73, 75, 131], [0, 3, 2, 1])]
    for counts, starts, slots in steps:
        n = sum(counts)
        u = torch.randn(n, channels, generator=g).to(dtype)
        dt = partials(torch.randn(n, channels, generator=g).to(dtype), splits, g)
        bc = partials(torch.randn(n, 2 * states, generator=g).to(dtype), 0 if dtype == torch.bfloat16 else 1, g)
        gate = partials(torch.randn(n, gate_width, generator=g).to(dtype), splits, g)
        cu = ints([0] + torch.tensor(counts).cumsum(0).tolist())
        args = dict(cu_seqlens=cu, seq_starts=ints(starts), seq_slots=ints(slots))
        common = dict(gate_offset=offset, n_seqs=len(counts), out_dtype=dtype, max_query=max(counts))
        want = refs.selective_scan(u, host(dt), host(bc), host(gate), dt_bias=dt_bias, a=a, d=d, state=state_c, **args, **common)
        got = ops.selective_scan(u.cuda(), moved(dt), moved(bc), moved(gate), dt_bias=dt_bias.cuda(), a=a.cuda(), d=d.cuda(),
                                 state=state_g, **{k: v.cuda() for k, v in args.items()}, **common)
        assert torch.isfinite(got.float()).all()
        close(got, want, dtype, 8.0)
        used = sorted(slots)
        close(state_g[used], state_c[used], torch.float32, 4.0)
        others = [s for s in range(4) if s not in used]
        assert torch.equal(state_g[others].cpu().isnan(), state_c[others].isnan())


def test_a_scan_that_forgets_nothing_adds_up():
    """A = 0 (no decay), step size, B and C made one: the state is the running sum of the inputs and the output is
    states * that sum + D * u, through steps of any size."""
    channels, states = 5, 3
    a = torch.zeros(channels, states)
    dt_bias = torch.full((channels,), 0.5413248546129181)           # softplus(0.5413...) = 1
    d = torch.full((channels,), 2.0)
    state = torch.full((2, channels, states), float('nan')).cuda()
    inputs = torch.arange(1, 21, dtype=torch.float32)[:, None].repeat(1, channels)
    rows, at = [], 0
    for size in (1, 1, 2, 5, 1, 3, 7):
        u = inputs[at:at + size]
        got = ops.selective_scan(u.cuda(), torch.zeros(size, channels).cuda(), torch.ones(size, 2 * states).cuda(),
                                 torch.full((size, channels), 30.0).cuda(), dt_bias=dt_bias.cuda(), a=a.cuda(), d=d.cuda(),
                                 state=state, gate_offset=0, cu_seqlens=ints([0, size]).cuda(), seq_starts=ints([at]).cuda(),
                                 seq_slots=ints([1]).cuda(), n_seqs=1, max_query=size, out_dtype=torch.float32)
        rows.append(got.cpu())
        at += size
    got = torch.cat(rows)[:, 0]
    want = (states * inputs[:, 0].cumsum(0) + 2.0 * inputs[:, 0]) * 30.0          # silu(30) = 30 to float32
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-4)


# ------------------------------------------------------------------------------------------------ the router
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('outputs,groups,keep,top', [(14, 2, 1, 5), (6, 3, 2, 2), (20, 10, 1, 1), (9, 3, 3, 4), (5, 1, 1, 5),
                                                     (4, 4, 3, 2), (64, 8, 4, 8)])
def test_router_with_sigmoid_scores_and_groups_by_their_two_best(dtype, outputs, groups, keep, top):
    g = torch.Generator().manual_seed(outputs)
    n, width = 50, 36
    x = torch.randn(n, width, generator=g).to(dtype)
    router = torch.randn(outputs, width, generator=g) * 0.5
    args = dict(groups=groups, keep=keep, top=top, renormalize=True, score='sigmoid', group_score='top2', weight_scale=2.5,
                renormalize_eps=1e-20)
    want_chosen, want_weights = refs.moe_route(x, router, None, **args)
    chosen, weights = ops.moe_route(x.cuda(), router.cuda(), None, **args)
    # rows whose choice is a close call are left out (float32 sums in another order may decide otherwise)
    scores = torch.sigmoid(x.float() @ router.t())
    by_group = scores.view(n, groups, outputs // groups)
    group_score = by_group.topk(min(2, outputs // groups), dim=-1).values.sum(-1).sort(dim=-1, descending=True).values
    clear = torch.ones(n, dtype=torch.bool)
    if keep < groups:
        clear &= (group_score[:, keep - 1] - group_score[:, keep]) > 1e-4
    ordered = scores.sort(dim=-1, descending=True).values
    clear &= (ordered[:, :-1] - ordered[:, 1:]).min(dim=-1).values > 1e-5
    assert clear.sum() > n // 2
    assert torch.equal(chosen.cpu()[clear], want_chosen[clear])
    torch.testing.assert_close(weights.cpu()[clear], want_weights[clear], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(weights.cpu()[clear].sum(dim=-1), torch.full((int(clear.sum()),), 2.5), rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------------------------ decoding in one kernel
@pytest.mark.parametrize('lengths,page_size,d,heads,kv_heads,window,rot,splits,extra,biased,temperature,sunk,has_kv', [
    ([2100, 1, 700, 1290, 64, 2047, 300, 33], 16, 128, 16, 4, None, 0, 8, 16 * 128, True, (0.5, 64), False, True),
    ([1, 2, 31, 32, 33, 64, 65, 96], 8, 64, 6, 2, 20, 32, 3, 0, False, None, True, True),
    ([257, 512, 513], 32, 128, 8, 1, 100, 64, 1, 64, True, (1.5, 3), True, True),
    ([40, 1000, 3000], 16, 64, 16, 1, None, 0, 2, 16 * 64, True, (0.2, 100), False, False),
])
def test_decoding_with_queries_made_inside_is_the_two_kernels(lengths, page_size, d, heads, kv_heads, window, rot, splits, extra,
                                                              biased, temperature, sunk, has_kv):
    """The decode kernel that makes its queries, new key and new value itself, with what this design adds (the
    projection's bias, columns of another branch behind q, k and v, the query temperature, sinks, rows of queries
    only): bit for bit what the q/k kernel followed by the attention kernels leave, results and pages."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(d + heads)
    rows = len(lengths)
    stored = kv_heads if has_kv else 0
    k_cache, v_cache, table, _ = build_cache(lengths, page_size, kv_heads, d, dtype)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32).cuda()
    row_seq = torch.arange(rows, dtype=torch.int32).cuda()
    slots = (table[row_seq.long(), (positions // page_size).long()] * page_size + positions % page_size).to(torch.int32)
    qkv = ops.Partials((torch.randn(splits, rows, (heads + 2 * stored) * d + extra, generator=g) * 0.7).cuda())
    ones = torch.ones(d).cuda()
    bias = torch.randn((heads + 2 * stored) * d, generator=g).cuda() if biased else None
    sinks = torch.linspace(-3.0, 3.0, heads).cuda() if sunk else None
    rotation = None
    if rot:
        from qil_amd.parts import RotaryFrequencies
        rotation = RotaryFrequencies(rot, 1000.0, device='cuda', scaling=(4.0, 1.0, 4.0, 128)).rotation()
    sizes = dict(heads=heads, kv_heads=kv_heads, head_dim=d)
    assert ops.decode_attention_takes(qkv, page_size=page_size, rotation=rotation, dtype=dtype, **sizes)
    k_two, v_two = k_cache.clone(), v_cache.clone()
    q = ops.qk_norm_rope_store(qkv, q_weight=ones, k_weight=ones, eps=1e-6, rotation=rotation, positions=positions,
                               slots=slots if has_kv else None, k_cache=k_two, v_cache=v_two, page_size=page_size, dtype=dtype,
                               heads=heads, kv_heads=stored, head_dim=d, extra_columns=extra, q_temperature=temperature, bias=bias)
    want = ops.paged_attention(q, k_cache=k_two, v_cache=v_two, page_size=page_size, block_tables=table, row_seq=row_seq,
                               positions=positions, cu_seqlens=None, seq_starts=None, single_rows=None, n_seqs=rows,
                               max_query=1, max_context=max(lengths), scale=d ** -0.5, window=window, sinks=sinks, **sizes)
    k_one, v_one = k_cache.clone(), v_cache.clone()
    got = ops.decode_attention(qkv, q_weight=ones, k_weight=ones, eps=1e-6, rotation=rotation, positions=positions,
                               writes=has_kv, k_cache=k_one, v_cache=v_one, page_size=page_size, block_tables=table,
                               row_seq=row_seq, max_context=max(lengths), scale=d ** -0.5, window=window, has_kv=has_kv,
                               extra_columns=extra, bias=bias, q_temperature=temperature, sinks=sinks, **sizes)
    assert isinstance(got, torch.Tensor) and torch.isfinite(got.float()).all()
    torch.testing.assert_close(got, want, atol=0, rtol=0)
    same = lambda a, b: torch.equal(a.view(torch.int16), b.view(torch.int16))          # NaN-filled pages: compare the bits
    assert same(k_one, k_two) and same(v_one, v_two), 'the pages differ'
