"""The kernels the Zinesun design added or changed, each alone against its plain reference (``kernel_refs``) on the same
inputs: the short convolution with its state (widths the four-wide form takes and others, one to four taps, sequences
shorter than the state, slots that are used again), the activations without a gate branch, a normed sub-layer's output
joining the stream with a channel scale and an average over depth, and the latent attention with a window and a factor
per head (both kernels, windows at and around the kernel's steps of keys and the pages' borders)."""
import pytest
import torch

import kernel_refs as refs
from qil_amd import ops
from test_fubapel_kernels_gpu import paged

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def close(actual, expected, dtype, scale=1.0):
    tolerance = dict(atol=2e-5 * scale, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2 * scale, rtol=2e-2)
    torch.testing.assert_close(actual.float().cpu(), expected.float(), **tolerance)


def ints(values):
    return torch.tensor(values, dtype=torch.int32)


# ------------------------------------------------------------------------------------------------ short convolution
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('width', [20, 21, 7, 1028, 1300])
@pytest.mark.parametrize('taps', [1, 2, 3, 4, 6])
def test_short_convolution_with_its_state(dtype, width, taps):
    """Five steps over five slots: sequences that begin (whatever their slot held before, NaN here, is not read), that
    continue from a state shorter than taps - 1 inputs, that bring fewer rows than the state holds, and one long
    portion; a slot is given to a new sequence in the last step."""
    g = torch.Generator().manual_seed(width * 10 + taps)
    keep = taps - 1
    weight = torch.randn(taps, width, generator=g)
    state_c = torch.full((5, keep, width), float('nan')) if keep else None
    state_g = state_c.clone().cuda() if keep else None
    steps = [([5, 1, 2], [0, 0, 0], [3, 0, 4]),                  # (rows, positions before the step, slots)
             ([1, 1, 70], [5, 1, 2], [3, 0, 4]),
             ([2, 1, 3, 1], [6, 2, 0, 72], [3, 0, 1, 4]),
             ([9, 2], [0, 8], [0, 3]),                           # slot 0 begins anew
             ([1100, 1, 2, 9, 30], [10, 9, 0, 0, 0], [3, 0, 1, 2, 4])]       # enough rows for threads that walk several
    for counts, starts, slots in steps:
        n = sum(counts)
        x = torch.randn(n, width, generator=g)
        cu = ints([0] + torch.tensor(counts).cumsum(0).tolist())
        row_seq = ints([s for s, c in enumerate(counts) for _ in range(c)])
        args = dict(cu_seqlens=cu, seq_starts=ints(starts), seq_slots=ints(slots), row_seq=row_seq)
        want = refs.short_conv(x, weight, state=state_c, n_seqs=len(counts), out_dtype=dtype, **args)
        got = ops.short_conv(x.cuda(), weight.cuda(), state=state_g, n_seqs=len(counts), out_dtype=dtype,
                             **{k: v.cuda() for k, v in args.items()})
        assert torch.isfinite(got).all()
        close(got, want, dtype, 4.0)
        if keep:
            used = sorted(slots)
            close(state_g[used], state_c[used], torch.float32)
            others = [s for s in range(5) if s not in used]
            assert torch.equal(state_g[others].cpu().isnan(), state_c[others].isnan())       # nobody's slots are left alone


def test_each_tap_reads_the_input_that_many_steps_back():
    """One tap set to one and the others to nothing: the result is the input plus the input that many steps back, and
    nothing before the sequence's start, through steps of any size."""
    width, taps = 8, 4
    for tap in range(taps):
        weight = torch.zeros(taps, width)
        weight[tap] = 1.0
        back = taps - 1 - tap
        state = torch.full((2, taps - 1, width), float('nan')).cuda()
        inputs = torch.arange(1, 21, dtype=torch.float32)[:, None].repeat(1, width)
        rows, at = [], 0
        for size in (1, 1, 2, 5, 1, 3, 7):
            args = dict(cu_seqlens=ints([0, size]).cuda(), seq_starts=ints([at]).cuda(), seq_slots=ints([1]).cuda(),
                        row_seq=ints([0] * size).cuda())
            rows.append(ops.short_conv(inputs[at:at + size].cuda(), weight.cuda(), state=state, n_seqs=1,
                                       out_dtype=torch.float32, **args).cpu())
            at += size
        got = torch.cat(rows)[:, 0]
        want = inputs[:, 0] + torch.cat([torch.zeros(back), inputs[:20 - back, 0]])
        assert torch.equal(got, want), (tap, got, want)


# ------------------------------------------------------------------------------------------------ activations
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('activation', ['xielu', 'gelu_tanh'])
@pytest.mark.parametrize('shape', [(3, 40), (5, 37), (1, 4100), (9, 1)])
def test_activations_without_a_gate_branch(dtype, activation, shape):
    g = torch.Generator().manual_seed(shape[1])
    x = (torch.randn(shape, generator=g) * 4).to(dtype)
    x.view(-1)[:3] = torch.tensor([0.0, -30.0, 30.0]).to(dtype)[:x.numel()]
    for p, q in ((0.3, -0.7), (-2.0, 1.5)):
        params = torch.tensor([p, q]) if activation == 'xielu' else None
        got = ops.plain_act(x.cuda(), dtype, activation=activation, params=None if params is None else params.cuda())
        close(got, refs.plain_act(x, dtype, activation=activation, params=params), dtype, 40.0)
    parts = torch.randn((3,) + shape, generator=g)
    params = torch.tensor([0.1, 0.2]) if activation == 'xielu' else None
    got = ops.plain_act(ops.Partials(parts.cuda()), dtype, activation=activation, params=None if params is None else params.cuda())
    close(got, refs.plain_act(parts.sum(0), dtype, activation=activation, params=params), dtype, 10.0)


def test_xielu_by_hand():
    """softplus(p) z^2 + z / 2 above zero; (1 / 2 + softplus(q)) (exp(z) - 1 - z) + z / 2 below."""
    import math
    p, q = 0.4, -0.2
    z = [2.0, 0.5, 0.0, -0.5, -3.0]
    soft = lambda t: math.log1p(math.exp(t))
    want = [soft(p) * t * t + t / 2 if t > 0 else (0.5 + soft(q)) * (math.exp(t) - 1 - t) + t / 2 for t in z]
    got = ops.plain_act(torch.tensor([z]).cuda(), torch.float32, activation='xielu', params=torch.tensor([p, q]).cuda())
    torch.testing.assert_close(got.cpu()[0], torch.tensor(want), atol=1e-6, rtol=1e-6)


# ------------------------------------------------------------------------------------------------ the stream
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('width', [40, 37, 258, 1100, 4100])
@pytest.mark.parametrize('centre', [True, False])
def test_a_normed_output_joins_the_stream_with_a_channel_scale_and_an_average_over_depth(dtype, width, centre):
    g = torch.Generator().manual_seed(width)
    n = 6
    stream = torch.randn(n, width, generator=g) * 3 + 1.0
    weight, bias, channel = (torch.randn(width, generator=g) for _ in range(3))
    value = (torch.randn(n, width, generator=g) * 5 + 2.0).to(dtype)
    parts = torch.randn(3, n, width, generator=g) + 0.5
    history = torch.randn(5, n, width, generator=g)
    mix = torch.randn(4, generator=g)
    for v_gpu, v_cpu in ((value.cuda(), value), (ops.Partials(parts.cuda()), parts.sum(0))):
        for vectors in ((weight, bias, channel), (weight, None, None), (None, None, channel)):
            for depth in (0, 1, 4):
                w, b, c = vectors
                s_gpu, s_cpu, h_gpu, h_cpu = stream.clone().cuda(), stream.clone(), history.clone().cuda(), history.clone()
                args = dict(eps=1e-5, centre=centre, depth=depth)
                got = ops.post_norm_scale_add(s_gpu, v_gpu, weight=None if w is None else w.cuda(),
                                              bias=None if b is None else b.cuda(),
                                              channel_scale=None if c is None else c.cuda(), out_dtype=dtype,
                                              history=h_gpu if depth else None, mix=mix[:depth].cuda() if depth else None, **args)
                want = refs.post_norm_scale_add(s_cpu, v_cpu, weight=w, bias=b, channel_scale=c, out_dtype=dtype,
                                                history=h_cpu if depth else None, mix=mix[:depth] if depth else None, **args)
                close(got, want, dtype, 10.0)
                close(s_gpu, s_cpu, torch.float32, 10.0)                       # the stream holds the unrounded result
                close(h_gpu, h_cpu, torch.float32, 10.0)
                if depth:
                    assert torch.equal(h_gpu[depth:].cpu(), history[depth:])   # later entries are left alone
    s_gpu = stream.clone().cuda()
    assert ops.post_norm_scale_add(s_gpu, value.cuda(), weight=weight.cuda(), bias=bias.cuda(), channel_scale=None,
                                   eps=1e-5, centre=centre) is None
    y = value.float() - (value.float().mean(-1, keepdim=True) if centre else 0.0)
    close(s_gpu, stream + y / torch.sqrt(y.square().mean(-1, keepdim=True) + 1e-5) * weight + bias, torch.float32, 10.0)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('width', [40, 37, 1100])
def test_a_routed_sum_is_made_as_the_row_is_loaded(dtype, width):
    """A routed feed-forward's pairs in the place of the value: the weighted sum in slot order, an identity expert's
    pair being the token's own input; as the sum's own kernel followed by the plain form."""
    g = torch.Generator().manual_seed(width)
    n, top, experts = 7, 3, 5
    stream = torch.randn(n, width, generator=g)
    x = torch.randn(n, width, generator=g).to(dtype)
    pairs = torch.randn(n * top, width, generator=g) * 2
    chosen = torch.randint(0, experts + 2, (n, top), generator=g).to(torch.int32)       # two identity experts behind the five
    chosen[0] = torch.tensor([experts, 0, experts + 1])
    weights = torch.rand(n, top, generator=g)
    weight, bias, channel = (torch.randn(width, generator=g) for _ in range(3))
    history, mix = torch.randn(3, n, width, generator=g), torch.randn(3, generator=g)
    picked = torch.where((chosen >= experts)[:, :, None], x.float()[:, None, :].expand(n, top, width), pairs.view(n, top, width))
    summed = (weights[:, :, None] * picked).sum(dim=1)
    for depth in (0, 3):
        routed = ops.RoutedSum(x.cuda(), pairs.cuda(), chosen.cuda(), weights.cuda(), experts)
        s_gpu, s_two, s_cpu = stream.clone().cuda(), stream.clone().cuda(), stream.clone()
        h_gpu, h_two, h_cpu = history.clone().cuda(), history.clone().cuda(), history.clone()
        args = dict(weight=weight, bias=bias, channel_scale=channel)
        rest = dict(eps=1e-5, centre=True, out_dtype=dtype, depth=depth)
        on_gpu = {k: v.cuda() for k, v in args.items()}
        got = ops.post_norm_scale_add(s_gpu, routed, history=h_gpu if depth else None, mix=mix.cuda() if depth else None,
                                      **on_gpu, **rest)
        two = ops.post_norm_scale_add(s_two, ops.Partials(routed.materialize().unsqueeze(0)), history=h_two if depth else None,
                                      mix=mix.cuda() if depth else None, **on_gpu, **rest)
        want = refs.post_norm_scale_add(s_cpu, summed, history=h_cpu if depth else None, mix=mix if depth else None, **args, **rest)
        close(got, want, dtype, 10.0)
        close(s_gpu, s_cpu, torch.float32, 10.0)
        close(h_gpu, h_cpu, torch.float32, 10.0)
        close(got, two.cpu(), dtype)
        close(s_gpu, s_two.cpu(), torch.float32)
        close(h_gpu, h_two.cpu(), torch.float32)


# ------------------------------------------------------------------------------------------------ window and gate
WINDOWS = [1, 2, 7, 31, 32, 33, 64, 65, 96, 149, 150, 151, 1000]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(heads=5, rank=20, rot=6, page=4), dict(heads=3, rank=72, rot=32, page=16)])
def test_windowed_latent_attention_with_a_factor_per_head(dtype, sizes):
    """The general kernel: rows at many positions of one sequence, every window from one key to more than there are."""
    heads, rank, rot, page = sizes['heads'], sizes['rank'], sizes['rot'], sizes['page']
    g = torch.Generator().manual_seed(heads)
    n_tokens = 150
    order = torch.randperm(-(-n_tokens // page) + 2, generator=g).tolist()
    latent, rope, table, _, _ = paged(n_tokens, page, rank, rot, dtype, g, order)
    positions = ints([0, 1, page - 1, page, page + 1, 31, 32, 63, 64, 65, 95, 96, 97, 127, 128, 149])
    n = len(positions)
    q = torch.randn(n, heads * (rank + rot), generator=g) * 0.5
    gate = torch.rand(n, heads, generator=g)
    tables, row_seq = torch.stack([table, torch.zeros_like(table)]), torch.zeros(n, dtype=torch.int32)
    common = dict(page_size=page, scale=0.3, heads=heads, rank=rank, rot=rot, sink=None)
    for window in WINDOWS:
        for factor in (gate, None):
            want = refs.latent_attention(q, latent=latent, rope=rope, block_tables=tables, row_seq=row_seq,
                                         positions=positions, window=window, gate=factor, **common)
            got = ops.latent_attention(q.cuda(), latent=latent.cuda(), rope=rope.cuda(), block_tables=tables.cuda(),
                                       row_seq=row_seq.cuda(), positions=positions.cuda(), window=window,
                                       gate=None if factor is None else factor.cuda(), **common)
            assert torch.isfinite(got).all(), window
            close(got, want, torch.float32, 1.0 if dtype == torch.float32 else 50.0)


@pytest.mark.parametrize('sizes', [dict(heads=4, rank=128, rot=32, page=16), dict(heads=5, rank=32, rot=8, page=4),
                                   dict(heads=18, rank=64, rot=16, page=8)])
@pytest.mark.parametrize('step', ['portions', 'single rows', 'both'])
@pytest.mark.parametrize('key_parts', [None, (64, 1), (32, 3)])
def test_windowed_latent_attention_on_the_matrix_cores(sizes, step, key_parts, monkeypatch):
    """bfloat16 caches with the step's description, as the engine calls it: portions that start anywhere, single rows,
    the keys in one piece and in parts; windows inside one step of keys, at its edges, across pages and parts, and
    longer than any context."""
    heads, rank, rot, page = sizes['heads'], sizes['rank'], sizes['rot'], sizes['page']
    g = torch.Generator().manual_seed(rank + heads)
    lengths = {'portions': [(130, 41), (0, 67), (63, 2)], 'single rows': [(200, 1), (0, 1), (64, 1), (31, 1)],
               'both': [(95, 33), (17, 3), (150, 1), (0, 1)]}[step]                # (tokens cached before, rows of the step)
    most = max(a + b for a, b in lengths)
    pages_each = -(-most // page)
    order = torch.randperm(pages_each * len(lengths) + 2, generator=g)
    latent = torch.full((len(order), page, rank), float('nan')).to(torch.bfloat16)
    rope = torch.full((len(order), page, rot), float('nan')).to(torch.bfloat16)
    tables = order[:pages_each * len(lengths)].view(len(lengths), pages_each).to(torch.int32)
    positions, row_seq, cu = [], [], [0]
    for s, (cached, rows) in enumerate(lengths):
        keys = torch.arange(cached + rows)
        slots = tables[s].long()[keys // page] * page + keys % page
        latent.view(-1, rank)[slots] = torch.randn(len(keys), rank, generator=g).to(torch.bfloat16)
        rope.view(-1, rot)[slots] = torch.randn(len(keys), rot, generator=g).to(torch.bfloat16)
        positions += list(range(cached, cached + rows))
        row_seq += [s] * rows
        cu.append(cu[-1] + rows)
    n = len(positions)
    positions, row_seq, cu = ints(positions), ints(row_seq), ints(cu)
    starts = ints([a for a, _ in lengths])
    q = torch.randn(n, heads * (rank + rot), generator=g) * 0.4
    gate = torch.rand(n, heads, generator=g)
    monkeypatch.setattr(ops, 'LATENT_KEY_PARTS', key_parts)
    common = dict(page_size=page, scale=(rank + rot) ** -0.5 * 3, heads=heads, rank=rank, rot=rot, sink=None)
    for window in [1, 2, 16, 31, 32, 33, 63, 64, 65, 96, 130, 1000]:
        factor = gate if window % 2 == 0 else None
        want = refs.latent_attention(q, latent=latent, rope=rope, block_tables=tables, row_seq=row_seq, positions=positions,
                                     window=window, gate=factor, **common)
        got = ops.latent_attention(q.cuda(), latent=latent.cuda(), rope=rope.cuda(), block_tables=tables.cuda(),
                                   row_seq=row_seq.cuda(), positions=positions.cuda(), cu_seqlens=cu.cuda(),
                                   seq_starts=starts.cuda(), n_seqs=len(lengths), max_query=max(b for _, b in lengths),
                                   max_context=most, window=window, gate=None if factor is None else factor.cuda(), **common)
        assert torch.isfinite(got).all(), window
        torch.testing.assert_close(got.cpu(), want, atol=2e-2, rtol=2e-2, msg=lambda m: f'window {window}: {m}')


@pytest.mark.parametrize('dtype', DTYPES)
def test_the_key_at_the_window_s_far_edge_wins_and_the_one_beyond_is_not_seen(dtype):
    """A query that points at one key with a score far above all others: with the key just inside the window the
    result is that key's latent (times the head's factor), just outside it is not; for windows that end at page
    borders and the kernels' steps of keys, in rows of a portion and in single rows."""
    g = torch.Generator().manual_seed(3)
    heads, rank, rot, page, n_tokens = 4, 32, 8, 16, 400
    order = torch.randperm(-(-n_tokens // page), generator=g).tolist()
    latent, rope, table, c, r = paged(n_tokens, page, rank, rot, dtype, g, order)
    keys = torch.cat([c, r], dim=1).float()
    factor = torch.tensor([1.0, 0.5, 0.25, 2.0])
    for window in (1, 2, 16, 17, 32, 33, 64, 65, 97, 300):
        for position in (window - 1, window, 255, 256, 257, 399):
            if position - window + 1 < 0:
                continue
            inside, outside = position - window + 1, position - window
            targets = [inside] + ([outside] if outside >= 0 else [])
            q = torch.stack([(keys[t] * 60 / keys[t].square().sum()).repeat(heads) for t in targets])
            n = len(targets)
            base = dict(latent=latent.cuda(), rope=rope.cuda(), page_size=page, block_tables=table[None].cuda(),
                        row_seq=torch.zeros(n, dtype=torch.int32).cuda(), positions=ints([position] * n).cuda(), scale=1.0,
                        heads=heads, rank=rank, rot=rot, sink=None, window=window, gate=factor.expand(n, heads).contiguous().cuda())
            runs = [ops.latent_attention(q.cuda(), **base)]
            if dtype == torch.bfloat16:                                     # the matrix-core kernel: each row a sequence's only row
                single = dict(base, block_tables=table[None].expand(n, -1).contiguous().cuda(), row_seq=ints(list(range(n))).cuda())
                runs.append(ops.latent_attention(q.cuda(), cu_seqlens=ints(list(range(n + 1))).cuda(),
                                                 seq_starts=ints([position] * n).cuda(), n_seqs=n, max_query=1,
                                                 max_context=position + 1, **single))
            for got in runs:
                got = got.cpu().view(n, heads, rank)
                torch.testing.assert_close(got[0], factor[:, None] * c[inside].float(), atol=2e-2, rtol=2e-2,
                                           msg=lambda m: f'window {window}, position {position}: {m}')
                if outside >= 0:
                    assert (got[1] - factor[:, None] * c[outside].float()).abs().max() > 0.3, (window, position)
