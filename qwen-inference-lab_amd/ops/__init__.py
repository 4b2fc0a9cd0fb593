"""The kernels as Python functions over torch tensors on the GPU.

Each function checks what its kernel assumes (shapes, types, contiguity, sizes it
takes), then launches the hand-written HIP kernel on torch's current stream.
Nothing here computes on the host or through a library, with one exception:
bfloat16 matrix products with many rows and a bfloat16 result go to the GPU BLAS
library, where the reference uses one too (nn.Linear, qil/model.py:32-40).  An
op refuses sizes its kernel does not take with ``UnsupportedShape``; if the
kernel library cannot be built or loaded every op raises.

Tensors: ``T`` is the model's dtype (float32 or bfloat16).  The residual stream
is float32.  Index tensors are int32.
"""
import ctypes

import torch

from . import library

# Rows up to which every bfloat16 product runs on a weight-streaming kernel of this library (float32 results: always).
STREAM_GEMM_MAX_ROWS = 16
# ... and up to this many rows where K is a multiple of 128 (at least 384) and there is no bias: the kernel that
# passes A through LDS in stages.  Measured at 64 rows and 8B layer sizes against the GPU BLAS: 41 us against 47
# (gate/up), 24 against 37 (down), 15 against 17 (q/k/v), 11 against 15 (attention output).  Of 65 to 128 rows
# the library says which products it takes (those of few column tiles), and of 129 to 192 rows.
STREAM_GEMM_MOST_ROWS = 192
# Rows of the products that go to the 32 x 32 kernel with operands loaded straight into LDS; with the gate's epilogue
# it is ahead from 17 rows on, without it level with the staged kernel up to 32 rows.
MID_GEMM_FEWEST_ROWS, MID_GEMM_MOST_ROWS = 33, 256
MID_GATED_FEWEST_ROWS = 17
# Half the most keys a split of the row attention kernel gets (_rows_part scales the split with the work); tests set
# another value to force it.
ATTENTION_PART = 256
# Blocks the row attention kernel aims for.
ROWS_BLOCKS = 1024
# Blocks the matrix-core decode kernel aims for (256 CUs, 8 waves a block; measured best at 8 rows x 2048 keys).
DECODE_BLOCKS = 256
# Waves of a block of that kernel; each takes every DECODE_WAVES-th 32-key step of the block's keys.
DECODE_WAVES = 8
# Fewest keys of a block of that kernel (more, smaller parts cost more in the merge than they gain).
DECODE_MIN_PART = 256
# Most keys of a block.
DECODE_MAX_PART = 8192
# Rows up to which a decode step makes its queries, new keys and values inside the attention kernel: with few
# rows that saves a launch; with many the kernel is bound by memory and the blocks' start costs more than the
# launch (64 rows of 2048 keys: 111 us against 94 + 5; whole steps at 8B sizes: 24 and 32 rows gain 0.8 %
# with the fused kernel, 48 rows lose 2 %).
FUSED_DECODE_MOST_ROWS = 32
# Rows up to which the row kernel leaves its parts unmerged when the caller allows (the product after it merges them).
UNMERGED_ROWS_MOST = 16
# Launches of at most this many blocks (one a CU) let a wave load two of its steps at a time.
DECODE_PAIRS_BLOCKS = 256
# ... in the kernel that makes its queries itself only up to this head size (it needs the registers for them).
FUSED_PAIRS_MOST_DIM = 64


# A product of few rows may add its result into the residual stream itself (``add_to``), and the product after it may
# then make the RMSNorm of its operand itself (``Normed``): a norm kernel less per layer.  The adding kernel reads A
# once per 16 output columns and is a little slower than the kernel that leaves partial sums; measured on whole decode
# steps with the weights read once (nontemporal loads), the pair wins at every number of rows up to 16 (8B sizes:
# 1 row 3.43 -> 3.39 ms a step, 2 rows 3.51 -> 3.47, 4 rows 3.63 -> 3.61, 8 rows level, 12 rows 4.73 -> 4.66, 16 rows
# 5.08 -> 4.91; 0.6B sizes: 1 row 1.28 -> 1.23, 8 rows 1.56 -> 1.54).  (With plain loads it was level up to 8 rows of
# large products and stayed off there; ``ADD_GEMM_FEW_ROWS`` rows and ``ADD_GEMM_SMALL_PRODUCT`` weights are that rule.)
# A float32 product of up to 16 rows (the whole-line kernel's) may make its operand itself while it stages it: the
# merge of the attention's context parts (``Unmerged``) or the activation of the gated feed-forward before it
# (``Gated``).  That saves a kernel, and every block of 128 result columns repeats the work for its slice of K: it pays
# while rows x K x blocks of columns is small.  Measured on whole float32 decode steps (merge / activation alone):
# 0.6B sizes 4 rows -2.4 % / -2.3 %, 16 rows +0.4 / -0.7; 8B sizes 1 row -0.9 / -1.0, 4 rows -0.6 / -0.8, 8 rows
# +1.6 / +1.6; 32B sizes 1 row -1.2 / -1.9, 2 rows +2.0 / +0.4, 4 rows +4.2 / +0.1.
GATED_OPERAND_MOST_ROWS = 16
UNMERGED_OPERAND_MOST_WORK = 1 << 19
GATED_OPERAND_MOST_WORK = 1 << 21
NORMED_GEMM_MOST_ROWS = 16
ADD_GEMM_MOST_ROWS = 16
ADD_GEMM_FEW_ROWS = 0                 # up to this many rows only products of at most ...
ADD_GEMM_SMALL_PRODUCT = 8 << 20      # ... this many weights add into the stream themselves
# True: bfloat16 products of many rows run on this library's own kernels too (from 512 rows on blocks of 256 x 256,
# below that the 32 x 32 tile kernel, 1,024 rows at a time) wherever they take the sizes, and the GPU BLAS is left
# out.  Slower (a 2,048-token prompt at 8B sizes takes 30.5 ms against 27.4, one of 8,192 tokens 117 against 106), and
# the same bits from run to run, which the BLAS does not promise: its product of 2,112 rows at 32B layer sizes was
# seen to differ by a rounding between identical runs.
OWN_LARGE_PRODUCTS = False
WIDE_GEMM_FEWEST_ROWS = 512           # from here on the 256 x 256 block kernel, below the 32 x 32 tile kernel


class UnsupportedShape(ValueError):
    pass


class Partials:
    """A matrix product left as float32 partial sums [splits, N, O]; its value is their sum in split
    order, made by the kernel that consumes it (norm, rotary/store, SiLU gate)."""

    def __init__(self, tensor):
        self.tensor, self.splits, self.shape = tensor, tensor.shape[0], tuple(tensor.shape[1:])
        self.device = tensor.device

    def sum(self):
        return self.tensor.sum(dim=0)


class Unmerged:
    """Attention of single rows left as the float32 partial results of the context's parts (rows 0 .. N-1
    of the step, all alone in their sequences).  ``merge()`` gives the [N, heads * d] tensor; ``linear``
    takes it as it is and merges while it stages its operand."""

    def __init__(self, workspace, positions, out, *, heads, head_dim, window, part, parts):
        self.workspace, self.positions, self.out = workspace, positions, out
        self.heads, self.head_dim, self.window, self.part, self.parts = heads, head_dim, window, part, parts
        self.shape, self.dtype, self.device = tuple(out.shape), out.dtype, out.device

    def merge(self):
        _check(library.load().qil_attn_merge(_ptr(self.workspace), _ptr(self.positions), None, _ptr(self.out),
                                             self.shape[0], self.heads, self.head_dim, self.window, self.part,
                                             self.parts, _code(self.dtype), None, _stream()), 'attn_merge')
        return self.out


class Gated:
    """The activation of a gated feed-forward, silu(gate) * up, not computed yet: ``sums`` are the gate and up
    products' partial sums (``Partials`` [N, 2 I]).  ``linear`` makes the activation while it stages its operand
    when its kernel takes the sizes, which saves the activation kernel; ``materialize()`` runs that kernel."""

    def __init__(self, sums, interleaved, dtype):
        self.sums, self.interleaved, self.dtype = sums, bool(interleaved), dtype
        self.shape, self.device = (sums.shape[0], sums.shape[1] // 2), sums.device
        self.is_cuda = sums.tensor.is_cuda

    def materialize(self):
        return silu_mul(self.sums, self.dtype, interleaved=self.interleaved)


class Added:
    """What ``linear`` returns when it has added its result into ``add_to`` itself.  ``squares`` [pieces, N] float32:
    the rows' sums of squares of the stream as it is now, in pieces of 16 columns."""

    def __init__(self, squares):
        self.squares = squares


class Averaged(Added):
    """What a block hands on when the stream is complete and is a weighted average over the results of the blocks so
    far: ``history`` float32 [total, N, H] holds those results (entry 0: the embedding's output), the first ``count``
    of them are filled.  The next block of the kind appends its own."""

    def __init__(self, history, count):
        super().__init__(None)
        self.history, self.count = history, int(count)


class Normed:
    """The RMSNorm of the float32 residual stream, not computed yet.  ``added`` is what completed the stream
    (``Added``: nothing is pending for it, and its rows' sums of squares are there).  ``linear`` makes the norm
    while it stages its operand when its kernel takes the sizes, which saves the norm kernel;
    ``materialize()`` runs the norm kernel."""

    def __init__(self, stream, weight, eps, dtype, added):
        self.stream, self.weight, self.eps, self.dtype, self.squares = stream, weight, float(eps), dtype, added.squares
        self.shape, self.device = tuple(stream.shape), stream.device

    def materialize(self):
        return add_rmsnorm(self.stream, None, self.weight, self.eps, self.dtype)


class PostNormed:
    """A sub-layer output that joins the residual stream as its RMS norm: stream += value / rms(value) * weight.
    ``value``: tensor of the model's type, float32 tensor, or ``Partials``.  The norms that add a pending output
    (``add_rmsnorm``, ``rows_rmsnorm``) take it and make both norms in one kernel, in float32 throughout."""

    def __init__(self, value, weight, eps):
        self.value, self.weight, self.eps = value, weight, float(eps)
        self.shape, self.device = tuple(value.shape), value.device


class RoutedSum:
    """The result of a routed feed-forward before its weighted sum: ``pairs`` float32 [N * top, width] (every (token,
    slot) pair's expert output), ``weights`` and ``chosen`` [N, top], and the feed-forward's input ``x`` (what an
    identity expert, a chosen index from ``experts`` on, passes).  A norm that takes a ``PostNormed`` makes the sum
    while it loads the row; ``materialize()`` runs the sum's own kernel."""

    def __init__(self, x, pairs, chosen, weights, experts):
        self.x, self.pairs, self.chosen, self.weights, self.experts = x, pairs, chosen, weights, int(experts)
        self.shape, self.device, self.dtype = tuple(x.shape), x.device, x.dtype

    def materialize(self):
        n, width = self.shape
        out = torch.empty((n, width), dtype=torch.float32, device=self.device)
        _check(library.load().qil_moe_combine(_ptr(self.x), _code(self.dtype), _ptr(self.pairs), _ptr(self.chosen),
                                              _ptr(self.weights), _ptr(out), n, width, self.experts, self.chosen.shape[1],
                                              _stream()), 'moe_combine')
        return out


def _plain_delta(delta):
    """A pending sub-layer output as the norms' kernels take it: a routed sum is made first."""
    return Partials(delta.materialize().unsqueeze(0)) if isinstance(delta, RoutedSum) else delta


def _post_normed(stream, pending, rows, weight, eps, out_dtype, update):
    n, width = stream.shape
    value = pending.value
    _require(stream, 'stream', torch.float32)
    _require(weight, 'weight', torch.float32, (width,))
    _require(pending.weight, 'post-norm weight', torch.float32, (width,))
    if isinstance(value, RoutedSum) and value.dtype == out_dtype:
        top = value.chosen.shape[1]
        _require(value.x, 'routed input', out_dtype, (n, width))
        _require(value.pairs, 'routed pairs', torch.float32, (n * top, width))
        _require(value.chosen, 'chosen', torch.int32, (n, top))
        _require(value.weights, 'weights', torch.float32, (n, top))
        if rows is not None:
            _require(rows, 'rows', torch.int32)
        count = n if rows is None else rows.shape[0]
        out = torch.empty((count, width), dtype=out_dtype, device=stream.device)
        _check(library.load().qil_post_norm_add_norm_routed(
            _ptr(stream), _ptr(value.pairs), _ptr(value.weights), _ptr(value.chosen), _ptr(value.x), top, value.experts,
            _ptr(pending.weight), pending.eps, _ptr(rows), _ptr(weight), _ptr(out), count, width, float(eps), int(update),
            _code(out_dtype), _stream()), 'post_norm_add_norm_routed')
        return out
    value = _plain_delta(value)
    if isinstance(value, Partials):
        _require(value.tensor, 'delta', torch.float32, (value.splits, n, width))
        pointer, code, splits = value.tensor.data_ptr(), 0, value.splits
    else:
        _require(value, 'delta', None, (n, width))
        if value.dtype not in (torch.float32, out_dtype):
            raise ValueError(f'delta must be float32 or {out_dtype}')
        pointer, code, splits = value.data_ptr(), _code(value.dtype), 1
    if rows is not None:
        _require(rows, 'rows', torch.int32)
    count = n if rows is None else rows.shape[0]
    out = torch.empty((count, width), dtype=out_dtype, device=stream.device)
    _check(library.load().qil_post_norm_add_norm(_ptr(stream), pointer, code, splits, n, _ptr(pending.weight), pending.eps,
                                                 _ptr(rows), _ptr(weight), _ptr(out), count, width, float(eps),
                                                 int(update), _code(out_dtype), _stream()), 'post_norm_add_norm')
    return out


def _operand(value, name, model_dtype, shape):
    """(pointer, dtype code, splits) of a consumer's input: a tensor of the model's type or Partials."""
    if isinstance(value, Partials):
        _require(value.tensor, name, torch.float32, (value.splits, *shape))
        return value.tensor.data_ptr(), 0, value.splits
    _require(value, name, model_dtype, shape)
    return value.data_ptr(), _code(model_dtype), 1


_CODES = {torch.float32: 0, torch.bfloat16: 1}


def _code(dtype):
    try:
        return _CODES[dtype]
    except KeyError:
        raise UnsupportedShape(f'kernels exist for float32 and bfloat16, not {dtype}') from None


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def _stream():
    """The current stream's handle.  (torch's direct accessor where it has one: building a Stream object for
    every launch cost a quarter of a small model's step on the host.)"""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(tensor):
    return None if tensor is None else tensor.data_ptr()


def _check(status, name):
    if status:
        raise RuntimeError(f'{name}: HIP kernel launch failed (status {status})'
                           if status > 0 else f'{name}: size not taken by the kernel')


def _require(tensor, name, dtype=None, shape=None):
    if not tensor.is_cuda:
        raise RuntimeError(f'{name} is on {tensor.device}: the kernels run on the GPU only')
    if not tensor.is_contiguous():
        raise ValueError(f'{name} must be contiguous')
    if dtype is not None and tensor.dtype != dtype:
        raise ValueError(f'{name} must be {dtype}, is {tensor.dtype}')
    if shape is not None and tuple(tensor.shape) != tuple(shape):
        raise ValueError(f'{name} must have shape {tuple(shape)}, has {tuple(tensor.shape)}')


def check_attention_geometry(*, heads, kv_heads, head_dim, dtype):
    """Sizes the attention kernels take; called when an attention part is built."""
    _code(dtype)
    if heads < 1 or kv_heads < 1 or heads % kv_heads:
        raise UnsupportedShape(f'heads {heads} must be a positive multiple of kv_heads {kv_heads}')
    if head_dim % 8 or not 8 <= head_dim <= 256:
        raise UnsupportedShape(f'head_dim {head_dim}: the attention kernels take multiples of 8 from 8 to 256 (an '
                               'attention part pads other even sizes up to 256 with zeros)')


def _check_caches(k_cache, v_cache, dtype, kv_heads, page_size, head_dim):
    """K [pages, kv_heads, page_size, d]; V transposed within the page: [pages, kv_heads, d, page_size]."""
    _require(k_cache, 'k_cache', dtype)
    _require(v_cache, 'v_cache', dtype)
    if k_cache.ndim != 4 or tuple(k_cache.shape[1:]) != (kv_heads, page_size, head_dim):
        raise ValueError(f'k_cache must be [pages, {kv_heads}, {page_size}, {head_dim}]')
    if v_cache.ndim != 4 or tuple(v_cache.shape[1:]) != (kv_heads, head_dim, page_size) \
            or v_cache.shape[0] != k_cache.shape[0]:
        raise ValueError(f'v_cache must be [pages, {kv_heads}, {head_dim}, {page_size}]')


def embed(token_ids, table, scale=1.0):
    """int32 [N], T [V, H] -> float32 stream [N, H] = table[token] * scale."""
    library.check_device()                                 # every step begins here
    _require(token_ids, 'token_ids', torch.int32)
    _require(table, 'table')
    n, width = token_ids.shape[0], table.shape[1]
    stream = torch.empty((n, width), dtype=torch.float32, device=table.device)
    _check(library.load().qil_embed(_ptr(token_ids), _ptr(table), _ptr(stream), n, width, float(scale), _code(table.dtype),
                                    _stream()), 'embed')
    return stream


def add_rmsnorm(stream, delta, weight, eps, out_dtype):
    """stream += delta (in place, float32 sum; skipped if delta is None); returns norm(stream) as out_dtype.

    ``delta``: tensor of ``out_dtype`` [N, H], Partials, or a ``PostNormed`` (its norm is what is added)."""
    if isinstance(delta, PostNormed):
        return _post_normed(stream, delta, None, weight, eps, out_dtype, True)
    delta = _plain_delta(delta)
    n, width = stream.shape
    _require(stream, 'stream', torch.float32)
    _require(weight, 'weight', torch.float32, (width,))
    pointer, code, splits = (None, _code(out_dtype), 1) if delta is None else _operand(delta, 'delta', out_dtype, (n, width))
    out = torch.empty((n, width), dtype=out_dtype, device=stream.device)
    _check(library.load().qil_add_rmsnorm(_ptr(stream), pointer, code, splits, n, None, _ptr(weight), _ptr(out), n,
                                          width, float(eps), 1, _code(out_dtype), _stream()), 'add_rmsnorm')
    return out


def rows_rmsnorm(stream, delta, rows, weight, eps, out_dtype):
    """norm(stream[rows] + delta[rows]) as out_dtype [len(rows), H]; stream is left as it is."""
    if isinstance(delta, PostNormed):
        return _post_normed(stream, delta, rows, weight, eps, out_dtype, False)
    delta = _plain_delta(delta)
    n, width = stream.shape
    _require(stream, 'stream', torch.float32)
    _require(weight, 'weight', torch.float32, (width,))
    _require(rows, 'rows', torch.int32)
    pointer, code, splits = (None, _code(out_dtype), 1) if delta is None else _operand(delta, 'delta', out_dtype, (n, width))
    out = torch.empty((rows.shape[0], width), dtype=out_dtype, device=stream.device)
    _check(library.load().qil_add_rmsnorm(_ptr(stream), pointer, code, splits, n, _ptr(rows), _ptr(weight), _ptr(out),
                                          rows.shape[0], width, float(eps), 0, _code(out_dtype), _stream()),
           'rows_rmsnorm')
    return out


def linear(x, weight, bias=None, out_dtype=None, partials=False, add_to=None):
    """x [N, K] @ weight [O, K]^T (+ bias float32 [O]) -> [N, O] in out_dtype (default: x's).

    ``partials=True`` allows the result to come back as ``Partials`` (bfloat16 products with few
    rows: float32, K split over blocks) for a consumer that adds them; otherwise a tensor.
    ``x`` may be ``Unmerged`` attention results, or a ``Normed`` residual stream.
    ``add_to``: the float32 residual stream [N, O]; if the kernel for these sizes can add its result into it
    (every element complete before it is added), it does and an ``Added`` is returned instead of the result."""
    if isinstance(x, Gated):
        lib = library.load()
        n, k = x.shape
        o = weight.shape[0]
        splits = lib.qil_gemm_f32_splits(n, o, k)
        if partials and bias is None and out_dtype in (None, torch.float32) and x.dtype == torch.float32 and \
                weight.dtype == torch.float32 and n <= GATED_OPERAND_MOST_ROWS and \
                n * k * -(-o // 128) <= GATED_OPERAND_MOST_WORK and \
                lib.qil_gemm_f32_gated_takes(n, o, k, int(x.interleaved), splits):
            _require(x.sums.tensor, 'gate and up sums', torch.float32, (x.sums.splits, n, 2 * k))
            _require(weight, 'weight', torch.float32, (o, k))
            out = torch.empty((splits, n, o), dtype=torch.float32, device=x.device)
            _check(lib.qil_gemm_f32_gated(_ptr(x.sums.tensor), x.sums.splits, int(x.interleaved), _ptr(weight), _ptr(out),
                                          n, o, k, splits, _stream()), 'gemm_f32_gated')
            return Partials(out)
        x = x.materialize()
    if isinstance(x, Normed):
        lib = library.load()
        n, k = x.shape
        o = weight.shape[0]
        splits = lib.qil_gemm_bf16_splits(n, o, k)
        if partials and bias is None and out_dtype in (None, x.dtype) and x.dtype == torch.bfloat16 and \
                n <= NORMED_GEMM_MOST_ROWS and weight.dtype == x.dtype and lib.qil_gemm_bf16_normed_takes(n, o, k, splits):
            _require(x.stream, 'stream', torch.float32, (n, k))
            _require(x.weight, 'norm weight', torch.float32, (k,))
            _require(x.squares, 'squares', torch.float32, (x.squares.shape[0], n))
            _require(weight, 'weight', x.dtype, (o, k))
            out = torch.empty((splits, n, o), dtype=torch.float32, device=x.device)
            _check(lib.qil_gemm_bf16_normed(_ptr(x.stream), _ptr(x.weight), _ptr(x.squares), x.squares.shape[0], x.eps,
                                            _ptr(weight), _ptr(out), n, o, k, splits, _stream()), 'gemm_bf16_normed')
            return Partials(out)
        x = x.materialize()
    if add_to is not None and isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and bias is None and \
            out_dtype in (None, x.dtype) and x.shape[0] <= ADD_GEMM_MOST_ROWS:
        lib = library.load()
        n, k = x.shape
        o = weight.shape[0]
        if (n > ADD_GEMM_FEW_ROWS or o * k <= ADD_GEMM_SMALL_PRODUCT) and lib.qil_gemm_bf16_add_takes(n, o, k):
            _require(x, 'x')
            _require(weight, 'weight', x.dtype, (o, k))
            _require(add_to, 'add_to', torch.float32, (n, o))
            squares = torch.empty((o // 16, n), dtype=torch.float32, device=x.device)
            _check(lib.qil_gemm_bf16_add(_ptr(x), _ptr(weight), _ptr(add_to), _ptr(squares), n, o, k, 0, 0, _stream()),
                   'gemm_bf16_add')
            return Added(squares)
    if isinstance(x, Unmerged):
        lib = library.load()
        n, k = x.shape
        o = weight.shape[0]
        _require(weight, 'weight', x.dtype, (o, k))
        splits = lib.qil_gemm_bf16_splits(n, o, k)
        if partials and bias is None and out_dtype in (None, x.dtype) and x.dtype == torch.bfloat16 and \
                lib.qil_gemm_bf16_unmerged_takes(n, o, x.heads, x.head_dim, splits):
            out = torch.empty((splits, n, o), dtype=torch.float32, device=x.device)
            _check(lib.qil_gemm_bf16_unmerged(_ptr(x.workspace), _ptr(x.positions), _ptr(weight), _ptr(out), n, o,
                                              x.heads, x.head_dim, x.window, x.part, x.parts, splits, _stream()),
                   'gemm_bf16_unmerged')
            return Partials(out)
        if partials and bias is None and out_dtype in (None, x.dtype) and x.dtype == torch.float32:
            splits = lib.qil_gemm_f32_splits(n, o, k)
            if n * k * -(-o // 128) <= UNMERGED_OPERAND_MOST_WORK and \
                    lib.qil_gemm_f32_unmerged_takes(n, o, x.heads, x.head_dim, splits):
                out = torch.empty((splits, n, o), dtype=torch.float32, device=x.device)
                _check(lib.qil_gemm_f32_unmerged(_ptr(x.workspace), _ptr(x.positions), _ptr(weight), _ptr(out), n, o,
                                                 x.heads, x.head_dim, x.window, x.part, x.parts, splits, _stream()),
                       'gemm_f32_unmerged')
                return Partials(out)
        x = x.merge()
    _require(x, 'x')
    _require(weight, 'weight', x.dtype)
    n, k = x.shape
    o = weight.shape[0]
    if weight.shape[1] != k:
        raise ValueError(f'linear: x has {k} columns, weight {weight.shape[1]}')
    if bias is not None:
        _require(bias, 'bias', torch.float32, (o,))
    out_dtype = out_dtype or x.dtype
    lib = library.load()
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise UnsupportedShape('a float32 product has a float32 result')
        splits = lib.qil_gemm_f32_splits(n, o, k) if partials and bias is None else 1
        out = torch.empty((splits, n, o), dtype=torch.float32, device=x.device)
        _check(lib.qil_gemm_f32(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), n, o, k, splits, _stream()), 'gemm_f32')
        return Partials(out) if splits > 1 else out[0]
    _code(x.dtype)
    # (beyond 256 rows: in blocks of rows, for the products that the library is slow at; the kernel's file says which)
    if bias is None and out_dtype == x.dtype and (MID_GEMM_FEWEST_ROWS <= n <= MID_GEMM_MOST_ROWS or
                                                   (n > MID_GEMM_MOST_ROWS and lib.qil_gemm_bf16_mid_rows_takes(n, o, k))):
        splits = lib.qil_gemm_bf16_mid_splits(n, o, k)
        if splits == 1 or (splits > 1 and partials):
            out = torch.empty((splits, n, o), dtype=torch.float32 if splits > 1 else x.dtype, device=x.device)
            _check(lib.qil_gemm_bf16_mid(_ptr(x), _ptr(weight), _ptr(out), n, o, k, _code(out.dtype), splits, _stream()),
                   'gemm_bf16_mid')
            return Partials(out) if splits > 1 else out[0]
    streams = n <= STREAM_GEMM_MOST_ROWS and bool(lib.qil_gemm_bf16_streams(n, o, k, bias is not None))
    if streams and partials and bias is None and out_dtype == x.dtype:
        splits = lib.qil_gemm_bf16_splits(n, o, k)
        if splits > 1 or n <= STREAM_GEMM_MAX_ROWS:
            out = torch.empty((splits, n, o), dtype=torch.float32, device=x.device)
            _check(lib.qil_gemm_bf16(_ptr(x), _ptr(weight), None, _ptr(out), n, o, k, 0, splits, 0, 0, _stream()),
                   'gemm_bf16')
            return Partials(out)
    if out_dtype == torch.float32 or streams:
        out = torch.empty((n, o), dtype=out_dtype, device=x.device)
        _check(lib.qil_gemm_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), n, o, k, _code(out_dtype), 1, 0, 0,
                                 _stream()), 'gemm_bf16')
        return out
    if OWN_LARGE_PRODUCTS and out_dtype == x.dtype and n >= WIDE_GEMM_FEWEST_ROWS and lib.qil_gemm_bf16_wide_takes(n, o, k, 1):
        out = torch.empty((n, o), dtype=x.dtype, device=x.device)
        _check(lib.qil_gemm_bf16_wide(_ptr(x), _ptr(weight), _ptr(out), n, o, k, _code(out.dtype), 1, _stream()),
               'gemm_bf16_wide')
    elif OWN_LARGE_PRODUCTS and out_dtype == x.dtype and lib.qil_gemm_bf16_mid_splits(min(n, 1024), o, k) > 0:
        out = torch.empty((n, o), dtype=x.dtype, device=x.device)
        for at in range(0, n, 1024):                    # the kernel takes up to 1,024 rows, in blocks of 256
            rows = min(1024, n - at)
            _check(lib.qil_gemm_bf16_mid(x[at:at + rows].data_ptr(), _ptr(weight), out[at:at + rows].data_ptr(), rows, o, k,
                                         _code(out.dtype), 1, _stream()), 'gemm_bf16_mid')
    else:
        out = torch.mm(x, weight.t())                  # GPU BLAS, float32 accumulation
    if bias is not None:
        _check(lib.qil_add_bias(_ptr(out), _ptr(bias), n, o, _code(out.dtype), _stream()), 'add_bias')
    return out


def interleave_gate_up(gate, up):
    """The [2 I, K] matrix that ``gated_linear(..., interleaved=True)`` takes: gate and up rows in turns of 16
    (gate rows 0-15, up rows 0-15, gate rows 16-31, ...).  A pure re-layout; I must be a multiple of 16."""
    inner, k = gate.shape
    if up.shape != gate.shape or inner % 16:
        raise ValueError('interleave_gate_up: two [I, K] matrices with I a multiple of 16')
    return torch.stack((gate.view(inner // 16, 16, k), up.view(inner // 16, 16, k)), dim=1).reshape(2 * inner, k).contiguous()


def gated_linear(x, weight, out_dtype=None, interleaved=False, lazy=False, activation='silu', limit=0.0, alpha=1.0):
    """act(x @ gate^T, x @ up^T) -> [N, I] (``activation``: a name of ``GATE_FUNCTIONS``; silu(gate) * up unless said), with ``weight`` the [2 I, K] matrix of both: the gate rows stacked
    before the up rows, or (``interleaved``) both in turns of 16 rows, which the kernels read faster.

    One kernel when a fused kernel takes the sizes (bfloat16; up to 16 rows, or up to 256 rows of an interleaved
    matrix large enough to fill the chip, or from 512 rows on under ``OWN_LARGE_PRODUCTS``); otherwise the product
    followed by ``silu_mul``.  Both add in float32.
    ``lazy``: a few float32 rows may come back as ``Gated`` (the product's partial sums) for ``linear`` to finish."""
    if isinstance(x, Normed):
        x = x.materialize()
    _require(x, 'x')
    _require(weight, 'weight', x.dtype)
    n, k = x.shape
    both = weight.shape[0]
    if weight.shape[1] != k or both % 2 or (interleaved and both % 32):
        raise ValueError(f'gated_linear: x {tuple(x.shape)}, weight {tuple(weight.shape)}')
    out_dtype = out_dtype or x.dtype
    lib = library.load()
    if activation != 'silu':                       # the product, then the activation kernel
        return gated_act(linear(x, weight, None, partials=True), out_dtype, activation=activation, limit=limit, alpha=alpha,
                         interleaved=interleaved)
    # 17 to 256 rows of an interleaved matrix: the 32 x 32 tile kernel where it takes the sizes (measured against the
    # staged 16 x 16 kernel with the same epilogue at 17 to 64 rows: 37 to 38 us against 38 to 43 at Qwen3-8B sizes,
    # 73 to 85 against 87 to 102 at 14B sizes)
    if x.dtype == torch.bfloat16 and interleaved and MID_GATED_FEWEST_ROWS <= n <= MID_GEMM_MOST_ROWS and \
            lib.qil_gemm_bf16_mid_gated_takes(n, both // 2, k):
        out = torch.empty((n, both // 2), dtype=out_dtype, device=x.device)
        _check(lib.qil_gemm_bf16_mid_gated(_ptr(x), _ptr(weight), _ptr(out), n, both // 2, k, _code(out_dtype), _stream()),
               'gemm_bf16_mid_gated')
        return out
    if x.dtype == torch.bfloat16 and n and lib.qil_gemm_bf16_gated_takes(n, both // 2, k, int(interleaved)):
        out = torch.empty((n, both // 2), dtype=out_dtype, device=x.device)
        _check(lib.qil_gemm_bf16_gated(_ptr(x), _ptr(weight), _ptr(out), n, both // 2, k, _code(out_dtype), 0, 0,
                                       int(interleaved), _stream()), 'gemm_bf16_gated')
        return out
    if OWN_LARGE_PRODUCTS and x.dtype == torch.bfloat16 and interleaved and n >= WIDE_GEMM_FEWEST_ROWS and \
            lib.qil_gemm_bf16_wide_gated_takes(n, both // 2, k):
        out = torch.empty((n, both // 2), dtype=out_dtype, device=x.device)
        _check(lib.qil_gemm_bf16_wide_gated(_ptr(x), _ptr(weight), _ptr(out), n, both // 2, k, _code(out_dtype), _stream()),
               'gemm_bf16_wide_gated')
        return out
    sums = linear(x, weight, None, partials=True)
    if lazy and x.dtype == torch.float32 and out_dtype == torch.float32 and n <= GATED_OPERAND_MOST_ROWS:
        return Gated(sums if isinstance(sums, Partials) else Partials(sums[None]), interleaved, out_dtype)
    return silu_mul(sums, out_dtype, interleaved=interleaved)


def silu_mul(gate_up, out_dtype=None, interleaved=False):
    """[N, 2 I] (tensor of the model's type or Partials) -> silu(gate) * up, [N, I].  The gate columns come first, or
    (``interleaved``) gate and up columns come in turns of 16."""
    n, both = gate_up.shape
    if both % 2 or (interleaved and both % 32):
        raise ValueError('silu_mul: needs an even number of columns (a multiple of 32 when they are interleaved)')
    out_dtype = out_dtype or (gate_up.dtype if not isinstance(gate_up, Partials) else None)
    if out_dtype is None:
        raise ValueError('silu_mul of Partials needs out_dtype')
    pointer, code, splits = _operand(gate_up, 'gate_up', out_dtype, (n, both))
    out = torch.empty((n, both // 2), dtype=out_dtype, device=gate_up.device)
    _check(library.load().qil_silu_mul(pointer, code, splits, _ptr(out), n, both // 2, _code(out_dtype), int(interleaved),
                                       _stream()), 'silu_mul')
    return out


def _rotation_arguments(rotation, head_dim):
    """(cos or frequencies, sin or None, rotated width) of a ``Rotation`` for the kernels: tables [positions, rot / 2],
    or (``rotation.frequencies``) the rot / 2 float32 frequencies alone, from which the kernels make the angles."""
    if rotation is None:
        return None, None, 0
    rot = rotation.rot_dim
    if getattr(rotation, 'frequencies', None) is not None:
        _require(rotation.frequencies, 'frequencies', torch.float32, (rot // 2,))
        cos, sin = rotation.frequencies, None
    else:
        cos, sin = rotation.cos, rotation.sin
        _require(cos, 'cos', torch.float32)
        _require(sin, 'sin', torch.float32, cos.shape)
        if cos.shape[1] * 2 != rot:
            raise ValueError('rotation tables do not fit rot_dim')
    if rot > head_dim or rot % 2:
        raise ValueError('rotation does not fit the head')
    return cos, sin, rot


def qk_norm_rope_store(qkv, *, heads, kv_heads, head_dim, q_weight, k_weight, eps, rotation, positions, slots,
                       k_cache, v_cache, page_size, dtype, norm_dim=None, rotate_first=False, extra_columns=0,
                       q_temperature=None, bias=None):
    """Per-head RMSNorm of q and k (if weights are given), rotation by position (if given).  ``norm_dim``: the
    number of elements the norm's mean runs over when the heads are padded with zeros (default: head_dim).
    ``rotate_first``: the rotation comes before the norm.  A rotation that carries ``frequencies`` is applied from
    position * frequency, made in the kernel.

    ``extra_columns``: so many more columns follow the v heads in every row of ``qkv`` (another branch of a stacked
    product); they are skipped.  ``kv_heads`` 0: the rows hold queries only.  ``q_temperature`` (coef, every): the
    query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1) last, in float32.  ``bias``
    float32 [(heads + 2 kv_heads) d]: the projection's bias, added here (the product before then has none and may
    stay partial sums).

    ``qkv`` [N, (heads + 2 kv_heads) d + extra_columns]: tensor of type ``dtype`` or Partials.  Returns q as ``dtype``
    [N, heads * d]; k and v go into the caches at ``slots`` (None: not stored)."""
    n = qkv.shape[0]
    pointer, code, splits = _operand(qkv, 'qkv', dtype, (n, (heads + 2 * kv_heads) * head_dim + extra_columns))
    coef, every = q_temperature if q_temperature is not None else (0.0, 0)
    if bias is not None:
        _require(bias, 'bias', torch.float32, ((heads + 2 * kv_heads) * head_dim,))
    _require(positions, 'positions', torch.int32, (n,))
    for w, name in ((q_weight, 'q_weight'), (k_weight, 'k_weight')):
        if w is not None:
            _require(w, name, torch.float32, (head_dim,))
    if (q_weight is None) != (k_weight is None):
        raise ValueError('q and k norms come together')
    cos, sin, rot = _rotation_arguments(rotation, head_dim)
    if slots is not None:
        _require(slots, 'slots', torch.int32, (n,))
        _check_caches(k_cache, v_cache, dtype, kv_heads, page_size, head_dim)
    q = torch.empty((n, heads * head_dim), dtype=dtype, device=qkv.device)
    _check(library.load().qil_qk_norm_rope_store(
        pointer, code, splits, _ptr(q), _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin), _ptr(positions),
        _ptr(slots), _ptr(k_cache), _ptr(v_cache), n, heads, kv_heads, head_dim, rot, page_size, float(eps),
        int(norm_dim or 0), int(bool(rotate_first)), int(extra_columns), float(coef), int(every), _ptr(bias), _code(dtype),
        _stream()),
        'qk_norm_rope_store')
    return q


def _rows_part(rows, kv_heads, max_context):
    """Keys a part of the row kernel: about ROWS_BLOCKS blocks in all, parts of 64 to ATTENTION_PART * 2 keys
    (measured in float32 at 2,048 keys of 8 kv heads: 1 row 28 us with parts of 64 to 256 against 67 with 512;
    8 rows 45 us with 128 against 54 with 256 and 62 with 64; 64 rows level from 256 on; 8 rows of 8,192 keys best
    at 256 and 512)."""
    if ATTENTION_PART != 256:                          # a test or tuning run has set it
        return ATTENTION_PART
    wanted = max_context * rows * kv_heads / ROWS_BLOCKS
    part = 64
    while part < 2 * ATTENTION_PART and part * 1.41 < wanted:      # the nearest of 64, 128, 256, 512
        part *= 2
    return part


def _decode_parts(rows, kv_heads, max_context):
    """(keys a part, parts) of the matrix-core decode kernel: the context is split until the chip has enough blocks.

    With more blocks than CUs the blocks run in rounds, and a last round that is mostly empty costs a whole one (33
    rows of 8 kv heads are 264 blocks: 75 us against 52 for 32 rows of 2,048 keys).  Then the context is cut so that
    the rounds fill: the fewest parts of 1,024 keys or more that fill their rounds to 90 %, else of 512 or more to
    80 % (33 rows: 4 parts, 69 us; at 8,192 keys 7 parts, about 197 against 276; 65 rows 2 parts, 112 against 116)."""
    blocks = rows * kv_heads
    if blocks > DECODE_BLOCKS:
        fill = lambda count: count / (-(-count // DECODE_BLOCKS) * DECODE_BLOCKS)
        if fill(blocks) < 0.72:
            for fewest_keys, enough in ((1024, 0.9), (512, 0.8)):
                for parts in range(2, 33):
                    part = -(-(-(-max_context // parts)) // 64) * 64
                    if part < fewest_keys:
                        break
                    if part > DECODE_MAX_PART:
                        continue
                    actual = -(-max_context // part)
                    if fill(blocks * actual) >= enough:
                        return part, actual
    wanted = max(1, DECODE_BLOCKS // blocks)
    part = min(DECODE_MAX_PART, max(DECODE_MIN_PART, -(-(-(-max_context // wanted)) // 64) * 64))
    return part, max(1, -(-max_context // part))


def decode_attention_takes(qkv, *, heads, kv_heads, head_dim, page_size, rotation, dtype):
    """Whether ``decode_attention`` takes the step: a float32 ``Partials`` q/k/v product, bfloat16 caches, sizes of
    the fused kernel."""
    rot = rotation.rot_dim if rotation is not None else 0
    return isinstance(qkv, Partials) and qkv.shape[0] <= FUSED_DECODE_MOST_ROWS and dtype == torch.bfloat16 and \
        bool(library.load().qil_attn_decode_fused_takes(heads, kv_heads, head_dim, page_size, rot))


def decode_attention(qkv, *, heads, kv_heads, head_dim, q_weight, k_weight, eps, rotation, positions, writes, k_cache,
                     v_cache, page_size, block_tables, row_seq, max_context, scale, window, unmerged=False,
                     rotate_first=False, softcap=None, has_kv=True, extra_columns=0, bias=None, q_temperature=None, sinks=None):
    """``qk_norm_rope_store`` and ``paged_attention`` in one kernel for a step whose rows are all alone in their
    sequences: queries, the new key and the new value are made from the partial sums ``qkv`` inside the
    attention kernel (bit for bit what the two kernels make), the new key and value are written into the
    pages (``writes``) and used from registers.  ``rotate_first`` and ``softcap`` as in ``qk_norm_rope_store`` and
    ``paged_attention``.  ``has_kv=False`` (with ``writes`` False): the rows of ``qkv`` hold queries only;
    ``extra_columns``, ``bias``, ``q_temperature`` as in ``qk_norm_rope_store``, ``sinks`` as in ``paged_attention``
    (a step with sinks comes back merged).  Returns what ``paged_attention`` returns."""
    n = qkv.shape[0]
    dtype = torch.bfloat16
    stored = kv_heads if has_kv else 0
    if writes and not has_kv:
        raise ValueError('decode_attention: a step that writes keys and values needs them in qkv')
    _require(qkv.tensor, 'qkv', torch.float32, (qkv.splits, n, (heads + 2 * stored) * head_dim + extra_columns))
    if bias is not None:
        _require(bias, 'bias', torch.float32, ((heads + 2 * stored) * head_dim,))
    if sinks is not None:
        _require(sinks, 'sinks', torch.float32, (heads,))
        unmerged = False
    coef, every = q_temperature if q_temperature is not None else (0.0, 0)
    _require(block_tables, 'block_tables', torch.int32)
    _require(row_seq, 'row_seq', torch.int32, (n,))
    _require(positions, 'positions', torch.int32, (n,))
    _check_caches(k_cache, v_cache, dtype, kv_heads, page_size, head_dim)
    if block_tables.ndim != 2 or block_tables.shape[1] * page_size < max_context:
        raise ValueError('block_tables are too narrow for the longest context')
    for w, name in ((q_weight, 'q_weight'), (k_weight, 'k_weight')):
        if w is not None:
            _require(w, name, torch.float32, (head_dim,))
    cos, sin, rot = _rotation_arguments(rotation, head_dim)
    lib = library.load()
    out = torch.empty((n, heads * head_dim), dtype=dtype, device=k_cache.device)
    window_arg = int(window or 0)
    part, parts = _decode_parts(n, kv_heads, max_context)
    nbytes = lib.qil_attn_rows_workspace(n, heads, head_dim, parts)
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=out.device) if nbytes else None
    _check(lib.qil_attn_decode_fused(_ptr(qkv.tensor), qkv.splits, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos),
                                     _ptr(sin), rot, int(bool(writes)), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                     block_tables.shape[1], _ptr(row_seq), _ptr(positions), _ptr(workspace), _ptr(out),
                                     n, heads, kv_heads, head_dim, page_size, window_arg, float(scale), part, parts,
                                     DECODE_WAVES, int(n * kv_heads * parts <= DECODE_PAIRS_BLOCKS and head_dim <= FUSED_PAIRS_MOST_DIM),
                                     int(bool(rotate_first)), float(softcap or 0.0), int(bool(has_kv)), int(extra_columns),
                                     _ptr(bias), float(coef), int(every), _ptr(sinks), _stream()), 'attn_decode_fused')
    if parts > 1:
        if sinks is not None:                           # the merge adds the sinks' term
            _check(lib.qil_attn_merge(_ptr(workspace), _ptr(positions), None, _ptr(out), n, heads, head_dim, window_arg,
                                      part, parts, _code(dtype), _ptr(sinks), _stream()), 'attn_merge')
            return out
        result = Unmerged(workspace, positions, out, heads=heads, head_dim=head_dim, window=window_arg, part=part,
                          parts=parts)
        return result if unmerged else result.merge()
    return out


TILE_KEY_PARTS = None   # tests: (keys per part, parts) forces the tile kernel's key split where it takes the sizes


def tile_key_parts(lib, dtype, n_seqs, max_query, heads, kv_heads, head_dim, page_size, table_stride, max_context,
                   general=False):
    """(keys per part, parts) for the matrix-core tile kernels; parts == 1: the keys in one piece.  ``general``: the
    step runs on the general tile kernel whatever its sizes."""
    part = ctypes.c_int(0)
    if general or dtype != torch.bfloat16 or not (head_dim in (64, 128) and
                                       lib.qil_attn_tile_bf16_takes(head_dim, page_size, table_stride)):
        parts = lib.qil_attn_tile_key_parts(n_seqs, max_query, heads, kv_heads, head_dim, max_context, _code(dtype),
                                            ctypes.byref(part))
        if TILE_KEY_PARTS is not None:
            part = ctypes.c_int(TILE_KEY_PARTS[0])
            parts = max(TILE_KEY_PARTS[1], -(-max_context // part.value))
        return part.value, parts
    parts = lib.qil_attn_tile_parts(n_seqs, max_query, heads, kv_heads, head_dim, page_size, table_stride, max_context,
                                    ctypes.byref(part))
    if TILE_KEY_PARTS is not None and head_dim in (64, 128) and lib.qil_attn_tile_bf16_takes(head_dim, page_size,
                                                                                              table_stride):
        part = ctypes.c_int(TILE_KEY_PARTS[0])
        parts = max(TILE_KEY_PARTS[1], -(-max_context // part.value))
    return part.value, parts


def paged_attention(q, *, heads, kv_heads, head_dim, k_cache, v_cache, page_size, block_tables, row_seq, positions,
                    cu_seqlens, seq_starts, single_rows, n_seqs, max_query, max_context, scale, window,
                    unmerged=False, tile_seqs=None, softcap=None, sinks=None):
    """Attention of every row of the step over its request's cached keys.

    ``q`` [N, heads * head_dim] (head h at columns [h d, (h + 1) d)).  Row n belongs to sequence ``row_seq[n]`` (a row of ``block_tables``) and sees keys j with
    j <= positions[n] and, with a window, j > positions[n] - window.  -> T [N, heads * head_dim].

    Sequences with two or more rows (``cu_seqlens``, ``seq_starts``) go to the matrix-core tile
    kernel; rows alone in their sequence (``single_rows``: their indices, or None when every row is
    alone, i.e. ``max_query == 1``) go to the split-context row kernel.  With ``unmerged`` the result may
    come back as ``Unmerged`` (every row alone, context in several parts) for ``linear`` to merge.
    ``tile_seqs``: the caller has put the sequences of two or more rows first and there are this many; the tile
    kernel then gets blocks for these only (None: for every sequence; those of one row leave at once).
    ``softcap`` c: scores are scaled, then capped softly, c * tanh(score / c), before the softmax.  The kernels
    specialised for bfloat16 heads of 64 and 128 have no cap; capped steps run on the general tile kernel.
    ``sinks`` float32 [heads]: exp(sinks[h]) joins the divisor of head h's softmax once (no key, no value, not
    scaled).  It enters where a row's result is normalised: in the kernel when the keys are in one piece, in the merge
    of the parts otherwise.  The general tile kernel, the bfloat16 prompt kernel for heads of 128, the matrix-core
    decode kernel and the row kernel take it; steps with sinks run on those and come back merged.
    """
    cap = float(softcap or 0.0)
    if sinks is not None:
        _require(sinks, 'sinks', torch.float32, (heads,))
        unmerged = False
    if cap < 0:
        raise ValueError('softcap must be positive')
    n = q.shape[0]
    qkv = q
    check_attention_geometry(heads=heads, kv_heads=kv_heads, head_dim=head_dim, dtype=qkv.dtype)
    _require(q, 'q', None, (n, heads * head_dim))
    _require(block_tables, 'block_tables', torch.int32)
    _require(row_seq, 'row_seq', torch.int32, (n,))
    _require(positions, 'positions', torch.int32, (n,))
    _check_caches(k_cache, v_cache, qkv.dtype, kv_heads, page_size, head_dim)
    if block_tables.ndim != 2 or block_tables.shape[1] * page_size < max_context:
        raise ValueError('block_tables are too narrow for the longest context')
    lib = library.load()
    out = torch.empty((n, heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    if max_query > 1:
        _require(cu_seqlens, 'cu_seqlens', torch.int32, (n_seqs + 1,))
        _require(seq_starts, 'seq_starts', torch.int32, (n_seqs,))
        if block_tables.shape[0] != n_seqs:
            raise ValueError('one block table row per sequence')
        if single_rows is None:
            raise ValueError('single_rows must list the rows that are alone when some sequence has several')
        _require(single_rows, 'single_rows', torch.int32)
        # sequences of one row leave their blocks at once: only the others count for how full the chip is
        several = max(1, n_seqs - single_rows.shape[0])
        if tile_seqs is not None:
            if tile_seqs != n_seqs - single_rows.shape[0]:
                raise ValueError('tile_seqs must count the sequences of two or more rows')
            n_seqs = tile_seqs
        part, parts = tile_key_parts(lib, qkv.dtype, several, max_query, heads, kv_heads,
                                     head_dim, page_size, block_tables.shape[1], max_context, general=cap > 0)
        if parts > 1:
            # few row tiles deep in a long context: the keys in parts, one block each, merged afterwards (over all
            # rows of the step: what the merge leaves in rows that are alone is overwritten below)
            # (with the sequences of several rows first, their rows are the step's first and the only ones merged)
            merged = n if tile_seqs is None else n - single_rows.shape[0]
            workspace = torch.empty(lib.qil_attn_rows_workspace(merged, heads, head_dim, parts) // 4, dtype=torch.float32,
                                    device=qkv.device)
            if cap == 0 and qkv.dtype == torch.bfloat16 and head_dim in (64, 128) and \
                    lib.qil_attn_tile_bf16_takes(head_dim, page_size, block_tables.shape[1]):
                _check(lib.qil_attn_tile_bf16_parts(_ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache),
                                                    _ptr(block_tables), block_tables.shape[1], _ptr(cu_seqlens),
                                                    _ptr(seq_starts), _ptr(workspace), merged, n_seqs, max_query, heads,
                                                    kv_heads, head_dim, page_size, int(window or 0), float(scale), part,
                                                    parts, _stream()), 'attn_tile_parts')
            else:
                _check(lib.qil_attn_tile_in_parts(_ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache),
                                                  _ptr(block_tables), block_tables.shape[1], _ptr(cu_seqlens),
                                                  _ptr(seq_starts), _ptr(workspace), merged, n_seqs, max_query, heads,
                                                  kv_heads, head_dim, page_size, int(window or 0), float(scale), cap,
                                                  part, parts, _code(qkv.dtype), _stream()), 'attn_tile_in_parts')
            _check(lib.qil_attn_merge(_ptr(workspace), _ptr(positions), None, _ptr(out), merged, heads, head_dim,
                                      int(window or 0), part, parts, _code(qkv.dtype), _ptr(sinks), _stream()), 'attn_merge')
        else:
            _check(lib.qil_attn_tile(_ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                     block_tables.shape[1], _ptr(cu_seqlens), _ptr(seq_starts), _ptr(out), n_seqs,
                                     max_query, heads, kv_heads, head_dim, page_size, int(window or 0), float(scale),
                                     cap, _code(qkv.dtype), _ptr(sinks), _stream()), 'attn_tile')
        rows = single_rows.shape[0]
    else:
        single_rows, rows = None, n
    if rows:
        window_arg = int(window or 0)
        if qkv.dtype == torch.bfloat16 and lib.qil_attn_decode_takes(heads, kv_heads, head_dim, page_size):
            # matrix-core kernel; split the context until the chip has about four blocks per CU
            part, parts = _decode_parts(rows, kv_heads, max_context)
            nbytes = lib.qil_attn_rows_workspace(rows, heads, head_dim, parts)
            workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=qkv.device) if nbytes else None
            _check(lib.qil_attn_decode(_ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                       block_tables.shape[1], _ptr(row_seq), _ptr(positions), _ptr(single_rows),
                                       _ptr(workspace), _ptr(out), rows, heads, kv_heads, head_dim, page_size,
                                       window_arg, float(scale), part, parts, DECODE_WAVES,
                                       int(rows * kv_heads * parts <= DECODE_PAIRS_BLOCKS and head_dim <= 128), cap,
                                       _ptr(sinks), _stream()), 'attn_decode')
            if unmerged and parts > 1 and single_rows is None:
                return Unmerged(workspace, positions, out, heads=heads, head_dim=head_dim, window=window_arg,
                                part=part, parts=parts)
            _check(lib.qil_attn_merge(_ptr(workspace), _ptr(positions), _ptr(single_rows), _ptr(out), rows, heads,
                                      head_dim, window_arg, part, parts, _code(qkv.dtype), _ptr(sinks), _stream()), 'attn_merge')
        else:
            part = _rows_part(rows, kv_heads, max_context)
            parts = max(1, -(-max_context // part))
            nbytes = lib.qil_attn_rows_workspace(rows, heads, head_dim, parts)
            workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=qkv.device) if nbytes else None
            if unmerged and parts > 1 and single_rows is None and rows <= UNMERGED_ROWS_MOST:
                _check(lib.qil_attn_rows_unmerged(_ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache),
                                                  _ptr(block_tables), block_tables.shape[1], _ptr(row_seq),
                                                  _ptr(positions), _ptr(workspace), rows, heads, kv_heads, head_dim,
                                                  page_size, window_arg, float(scale), cap, part, parts, _code(qkv.dtype),
                                                  _stream()), 'attn_rows_unmerged')
                return Unmerged(workspace, positions, out, heads=heads, head_dim=head_dim, window=window_arg,
                                part=part, parts=parts)
            _check(lib.qil_attn_rows(_ptr(qkv), qkv.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                     block_tables.shape[1], _ptr(row_seq), _ptr(positions), _ptr(single_rows),
                                     _ptr(workspace), _ptr(out), rows, heads, kv_heads, head_dim, page_size,
                                     window_arg, float(scale), cap, part, parts, _code(qkv.dtype), _ptr(sinks), _stream()),
                   'attn_rows')
    return out


def sample(logits, temperatures, seeds, counters, out=None):
    """float32 [M, V] -> (int32 tokens [M], int32 finite flags [M]).

    temperature 0: greedy, lowest index on ties; > 0: seeded Gumbel-max draw from softmax(logits / T)
    keyed by (seed, counter).  ``out``: an int32 [2, M] tensor to hold tokens and flags (its rows are returned)."""
    m, vocab = logits.shape
    _require(logits, 'logits', torch.float32)
    _require(temperatures, 'temperatures', torch.float32, (m,))
    _require(seeds, 'seeds', torch.int32, (m,))
    _require(counters, 'counters', torch.int32, (m,))
    lib = library.load()
    if out is None:
        out = torch.empty((2, m), dtype=torch.int32, device=logits.device)
    _require(out, 'out', torch.int32, (2, m))
    tokens, finite = out[0], out[1]
    workspace = torch.empty(lib.qil_sample_workspace(m, vocab) // 4, dtype=torch.int32, device=logits.device)
    _check(lib.qil_sample(_ptr(logits), _ptr(temperatures), _ptr(seeds), _ptr(counters), _ptr(tokens), _ptr(finite),
                          _ptr(workspace), m, vocab, _stream()), 'sample')
    return tokens, finite


# ---------------------------------------------------------------------------------------------------------------
# Norms with a scaled residual add; gate functions by name
def add_norm(stream, delta, weight, eps, out_dtype, *, centre, delta_scale=1.0, bias=None):
    """stream += delta_scale * delta (in place, float32; skipped if delta is None); returns the norm of the sum as
    out_dtype: layer norm (``centre``: the mean is removed, the variance is that of the centred row) or RMS norm,
    times ``weight``, plus ``bias`` (float32 [H]) if given, rounded once.  ``delta``: tensor of ``out_dtype`` [N, H]
    or Partials."""
    delta = _plain_delta(delta)
    n, width = stream.shape
    _require(stream, 'stream', torch.float32)
    _require(weight, 'weight', torch.float32, (width,))
    if bias is not None:
        _require(bias, 'bias', torch.float32, (width,))
    pointer, code, splits = (None, _code(out_dtype), 1) if delta is None else _operand(delta, 'delta', out_dtype, (n, width))
    out = torch.empty((n, width), dtype=out_dtype, device=stream.device)
    _check(library.load().qil_add_norm(_ptr(stream), pointer, code, splits, n, float(delta_scale), None, _ptr(weight),
                                       _ptr(bias), _ptr(out), n, width, float(eps), 1, int(bool(centre)), _code(out_dtype),
                                       _stream()), 'add_norm')
    return out


def rows_norm(stream, delta, rows, weight, eps, out_dtype, *, centre, delta_scale=1.0, bias=None):
    """``add_norm`` of the selected rows only, [len(rows), H]; stream is left as it is."""
    delta = _plain_delta(delta)
    n, width = stream.shape
    _require(stream, 'stream', torch.float32)
    _require(weight, 'weight', torch.float32, (width,))
    if bias is not None:
        _require(bias, 'bias', torch.float32, (width,))
    _require(rows, 'rows', torch.int32)
    pointer, code, splits = (None, _code(out_dtype), 1) if delta is None else _operand(delta, 'delta', out_dtype, (n, width))
    out = torch.empty((rows.shape[0], width), dtype=out_dtype, device=stream.device)
    _check(library.load().qil_add_norm(_ptr(stream), pointer, code, splits, n, float(delta_scale), _ptr(rows), _ptr(weight),
                                       _ptr(bias), _ptr(out), rows.shape[0], width, float(eps), 0, int(bool(centre)),
                                       _code(out_dtype), _stream()), 'rows_norm')
    return out


# Gate functions of gated feed-forwards: name -> code of the kernels.  'silu': silu(g) * u.  'clamped_swish' (with a
# limit L and a slope a): g' = min(g, L), u' = clamp(u, -L, L), g' * sigmoid(a g') * (u' + 1).
GATE_FUNCTIONS = {'silu': 0, 'clamped_swish': 1}


def gated_act(gate_up, out_dtype, *, activation, limit=0.0, alpha=1.0, interleaved=False):
    """[N, 2 I] (tensor of the model's type or Partials) -> act(gate, up), [N, I], for any gate function of
    ``GATE_FUNCTIONS``.  The gate columns come first, or (``interleaved``) gate and up columns come in turns of 16."""
    n, both = gate_up.shape
    if both % 2 or (interleaved and both % 32):
        raise ValueError('gated_act: needs an even number of columns (a multiple of 32 when they are interleaved)')
    pointer, code, splits = _operand(gate_up, 'gate_up', out_dtype, (n, both))
    out = torch.empty((n, both // 2), dtype=out_dtype, device=gate_up.device)
    _check(library.load().qil_gated_act(pointer, code, splits, _ptr(out), n, both // 2, _code(out_dtype), int(interleaved),
                                        GATE_FUNCTIONS[activation], float(limit), float(alpha), _stream()), 'gated_act')
    return out


# Activations of feed-forwards without a gate branch: name -> code of the kernel.  'xielu' (two stored numbers p, q):
# z > 0: softplus(p) z^2 + z / 2, else (1 / 2 + softplus(q)) (exp(z) - 1 - z) + z / 2.  'gelu_tanh': the tanh form of gelu.
PLAIN_ACTIVATIONS = {'xielu': 0, 'gelu_tanh': 1}


def plain_act(x, out_dtype, *, activation, params=None):
    """[N, I] (tensor of the model's type or Partials) -> act(x) [N, I] of ``out_dtype``, for an activation of
    ``PLAIN_ACTIVATIONS``; ``params`` float32 [2]: the two stored numbers of 'xielu'.  float32 arithmetic, one rounding."""
    n, inner = x.shape
    pointer, code, splits = _operand(x, 'x', out_dtype, (n, inner))
    if activation == 'xielu':
        _require(params, 'params', torch.float32, (2,))
    out = torch.empty((n, inner), dtype=out_dtype, device=x.device)
    _check(library.load().qil_plain_act(pointer, code, splits, _ptr(out), n, inner, _code(out_dtype),
                                        PLAIN_ACTIVATIONS[activation], _ptr(params), _stream()), 'plain_act')
    return out


def post_norm_scale_add(stream, value, *, weight, bias, channel_scale, eps, centre, out_dtype=None, history=None, depth=0,
                        mix=None):
    """A sub-layer's output joins the float32 residual stream as its norm: stream += channel_scale * (norm(value) *
    weight + bias), in place and in float32 (``centre``: layer norm, else RMS norm; ``weight``, ``bias``,
    ``channel_scale`` float32 [H] or None).  ``value``: a tensor of the model's type or float32, ``Partials`` or a
    ``RoutedSum``.  With ``history`` (float32 [>= depth, N, H]) the sum X is stored as entry ``depth - 1`` and the
    stream becomes sum_(j < depth) mix[j] * history[j], ``mix`` float32 [depth].  With ``out_dtype`` the new stream
    comes back rounded to that type (what the next sub-layer's products read), else None."""
    n, width = stream.shape
    _require(stream, 'stream', torch.float32)
    routed = value if isinstance(value, RoutedSum) else None
    if routed is not None:                              # the weighted sum is made as the kernel loads the row
        top = routed.chosen.shape[1]
        _require(routed.x, 'routed input', None, (n, width))
        _require(routed.pairs, 'routed pairs', torch.float32, (n * top, width))
        _require(routed.chosen, 'chosen', torch.int32, (n, top))
        _require(routed.weights, 'weights', torch.float32, (n, top))
    elif isinstance(value, Partials):
        _require(value.tensor, 'value', torch.float32, (value.splits, n, width))
        pointer, code, splits = value.tensor.data_ptr(), 0, value.splits
    else:
        _require(value, 'value', None, (n, width))
        pointer, code, splits = value.data_ptr(), _code(value.dtype), 1
    for name, vector in (('weight', weight), ('bias', bias), ('channel_scale', channel_scale)):
        if vector is not None:
            _require(vector, name, torch.float32, (width,))
    if depth:
        _require(history, 'history', torch.float32)
        _require(mix, 'mix', torch.float32, (depth,))
        if history.ndim != 3 or history.shape[0] < depth or tuple(history.shape[1:]) != (n, width):
            raise ValueError(f'post_norm_scale_add: history must be [>= {depth}, {n}, {width}]')
    out = torch.empty((n, width), dtype=out_dtype, device=stream.device) if out_dtype is not None else None
    tail = (_ptr(weight), _ptr(bias), _ptr(channel_scale), float(eps), int(bool(centre)), _ptr(out),
            _code(out_dtype) if out_dtype is not None else 0, _ptr(history) if depth else None, int(depth),
            _ptr(mix) if depth else None, n, width, _stream())
    if routed is not None:
        _check(library.load().qil_post_norm_scale_add_routed(_ptr(stream), _ptr(routed.pairs), _ptr(routed.weights),
                                                             _ptr(routed.chosen), _ptr(routed.x), _code(routed.x.dtype), top,
                                                             routed.experts, *tail), 'post_norm_scale_add_routed')
    else:
        _check(library.load().qil_post_norm_scale_add(_ptr(stream), pointer, code, splits, *tail), 'post_norm_scale_add')
    return out


def short_conv(x, weight, *, state, cu_seqlens, seq_starts, seq_slots, row_seq, n_seqs, out_dtype):
    """x + conv(x): a causal convolution over time on every channel, conv(x)_t = sum_j weight[j] * x_(t - taps + 1 + j),
    over the rows of every sequence of the step and the taps - 1 inputs before them, which are the sequence's
    state (``state`` float32 [slots, taps - 1, H]: read unless the sequence starts at position 0, and left holding
    the sequence's last taps - 1 inputs).  ``x`` float32 [N, H] (the residual stream), ``weight`` float32 [taps, H]
    (a tap's factors for all channels side by side).  -> [N, H] of ``out_dtype``; float32 arithmetic, one rounding."""
    n, width = x.shape
    _require(x, 'x', torch.float32)
    taps = weight.shape[0]
    _require(weight, 'weight', torch.float32, (taps, width))
    if taps > 1:
        _require(state, 'state', torch.float32)
        if state.ndim != 3 or tuple(state.shape[1:]) != (taps - 1, width):
            raise ValueError(f'short_conv: state must be [slots, {taps - 1}, {width}]')
    _require(cu_seqlens, 'cu_seqlens', torch.int32, (n_seqs + 1,))
    _require(seq_starts, 'seq_starts', torch.int32, (n_seqs,))
    _require(seq_slots, 'seq_slots', torch.int32, (n_seqs,))
    _require(row_seq, 'row_seq', torch.int32, (n,))
    out = torch.empty((n, width), dtype=out_dtype, device=x.device)
    _check(library.load().qil_short_conv(_ptr(x), _ptr(weight), _ptr(state) if taps > 1 else None, _ptr(cu_seqlens),
                                         _ptr(seq_starts), _ptr(seq_slots), _ptr(row_seq), _ptr(out), _code(out_dtype), n,
                                         width, taps, _stream()), 'short_conv')
    return out


# ---------------------------------------------------------------------------------------------------------------
# Attention over a cached latent
def latent_prepare(down, *, q_rank, rank, rot, q_weight, c_weight, eps, frequencies, positions, slots, latent, rope,
                   dtype, gates=0):
    """From the stacked down products ``down`` [N, q_rank + rank + rot (+ gates)] (tensor of ``dtype`` or Partials):
    the RMS-normed query latent [N, q_rank] (returned); the RMS-normed key/value latent and the rotated shared key
    part go into the caches ``latent`` [.., rank] / ``rope`` [.., rot] at ``slots`` (None: nothing is stored).  With
    ``gates`` more columns the result is (query latent, float32 [N, gates] of their sigmoids)."""
    n = down.shape[0]
    pointer, code, splits = _operand(down, 'down', dtype, (n, q_rank + rank + rot + gates))
    _require(q_weight, 'q_weight', torch.float32, (q_rank,))
    _require(c_weight, 'c_weight', torch.float32, (rank,))
    _require(frequencies, 'frequencies', torch.float32, (rot // 2,))
    _require(positions, 'positions', torch.int32, (n,))
    if slots is not None:
        _require(slots, 'slots', torch.int32, (n,))
        _require(latent, 'latent', dtype)
        _require(rope, 'rope', dtype)
        if latent.shape[-1] != rank or rope.shape[-1] != rot or latent.shape[:-1] != rope.shape[:-1]:
            raise ValueError('latent_prepare: caches must be [.., rank] and [.., rot] over the same slots')
    out = torch.empty((n, q_rank), dtype=dtype, device=down.device)
    gate = torch.empty((n, gates), dtype=torch.float32, device=down.device) if gates else None
    _check(library.load().qil_latent_prepare(pointer, code, splits, _ptr(q_weight), _ptr(c_weight), _ptr(frequencies),
                                             _ptr(positions), _ptr(slots), _ptr(out), _ptr(latent), _ptr(rope), _ptr(gate),
                                             n, q_rank, rank, rot, gates, float(eps), _code(dtype), _stream()),
           'latent_prepare')
    return (out, gate) if gates else out


HEAD_PRODUCT_BLAS_ROWS = 256     # rows from which a bfloat16 product per head goes to the GPU BLAS in one batch


def head_product(x, weight, *, heads, out_dtype, out=None, out_columns=None):
    """A product per head: x [N, heads * X] (head h's K inputs lead its X columns), weight [heads, K, O] (for every k
    its O outputs side by side) -> [N, heads * O] of ``out_dtype``, or into the leading O of every head's
    ``out_columns`` columns of ``out``.  Own kernels for few rows (k split in a block) and in float32; bfloat16 weights
    with ``HEAD_PRODUCT_BLAS_ROWS`` rows or more take one batched product of the GPU BLAS, float32 inputs rounded to
    bfloat16 first."""
    n = x.shape[0]
    _require(x, 'x')
    _require(weight, 'weight')
    if weight.ndim != 3 or weight.shape[0] != heads or x.shape[1] % heads or x.shape[1] // heads < weight.shape[1]:
        raise ValueError(f'head_product: x {tuple(x.shape)}, weight {tuple(weight.shape)}, {heads} heads')
    k, o = weight.shape[1], weight.shape[2]
    if out is None:
        out_columns = o
        out = torch.empty((n, heads * o), dtype=out_dtype, device=x.device)
    _require(out, 'out', out_dtype, (n, heads * out_columns))
    if n >= HEAD_PRODUCT_BLAS_ROWS and weight.dtype == torch.bfloat16:
        # many rows: one batched matrix-core product of the GPU BLAS (bfloat16 operands, float32 sums), a batch per head
        inputs = x.view(n, heads, x.shape[1] // heads)[:, :, :k]
        if inputs.dtype != torch.bfloat16:
            inputs = inputs.to(torch.bfloat16)
        product = torch.bmm(inputs.transpose(0, 1), weight)                    # [heads, N, O]
        out.view(n, heads, out_columns)[:, :, :o].copy_(product.transpose(0, 1))
        return out
    _check(library.load().qil_head_product(_ptr(x), _code(x.dtype), x.shape[1], x.shape[1] // heads, _ptr(weight),
                                           _code(weight.dtype), _ptr(out), _code(out_dtype), heads * out_columns,
                                           out_columns, n, heads, k, o, _stream()), 'head_product')
    return out


def latent_query(q, k_up, *, heads, dim, rot, rank, frequencies, positions):
    """Queries in the latent's space.  ``q`` [N, heads * (dim + rot)] (a head's unrotated part first), ``k_up``
    [heads, dim, rank] (the key expansion, a head's rows, as stored) -> float32 [N, heads, rank + rot]:
    k_up_h^T q_h, then the head's rotated part turned by the row's position."""
    n = q.shape[0]
    _require(q, 'q', None, (n, heads * (dim + rot)))
    _require(k_up, 'k_up', q.dtype, (heads, dim, rank))
    _require(frequencies, 'frequencies', torch.float32, (rot // 2,))
    _require(positions, 'positions', torch.int32, (n,))
    out = torch.empty((n, heads * (rank + rot)), dtype=torch.float32, device=q.device)
    head_product(q, k_up, heads=heads, out_dtype=torch.float32, out=out, out_columns=rank + rot)
    _check(library.load().qil_rotate_tail(_ptr(q), _code(q.dtype), heads * (dim + rot), dim + rot, dim, _ptr(frequencies),
                                          _ptr(positions), _ptr(out), heads * (rank + rot), rank + rot, rank, n, heads,
                                          rot, _stream()), 'rotate_tail')
    return out


# False: bfloat16 caches go to the general kernel too (tests and tuning runs).
LATENT_MATRIX_CORES = True
LATENT_KEY_PARTS = None     # tests: (keys a part, parts) forces the matrix-core kernel's split of the keys


def latent_attention(q, *, latent, rope, page_size, block_tables, row_seq, positions, sink, scale, heads, rank, rot,
                     cu_seqlens=None, seq_starts=None, n_seqs=None, max_query=None, max_context=None, window=None,
                     gate=None):
    """Every row's attention over its request's cached latents: ``q`` float32 [N, heads * (rank + rot)] as
    ``latent_query`` makes it; caches [pages, page_size, rank] and [pages, page_size, rot]; row n sees keys
    j <= positions[n] of sequence row_seq[n] (a row of ``block_tables``).  ``sink`` float32 [heads] or None: a logit
    per head that counts once in the softmax's denominator and has no value.  ``window`` w: the row at position p sees
    the keys j with 0 <= p - j < w only.  ``gate`` float32 [N, heads]: a factor on every head's result.
    -> float32 [N, heads * rank], the weighted sums of the latents.

    With the step's description (``cu_seqlens``, ``seq_starts``, ``n_seqs``, ``max_query``, ``max_context``; rows packed
    sequence after sequence) bfloat16 caches of sizes it takes go to the matrix-core kernel, which serves several rows
    and all heads from one staged tile of keys and cuts the keys into parts when the step has few rows."""
    n = q.shape[0]
    _require(q, 'q', torch.float32, (n, heads * (rank + rot)))
    _require(latent, 'latent')
    _require(rope, 'rope', latent.dtype)
    if tuple(latent.shape[1:]) != (page_size, rank) or tuple(rope.shape[1:]) != (page_size, rot) or \
            latent.shape[0] != rope.shape[0]:
        raise ValueError('latent_attention: caches must be [pages, page_size, rank] and [pages, page_size, rot]')
    _require(block_tables, 'block_tables', torch.int32)
    _require(row_seq, 'row_seq', torch.int32, (n,))
    _require(positions, 'positions', torch.int32, (n,))
    if sink is not None:
        _require(sink, 'sink', torch.float32, (heads,))
    if gate is not None:
        _require(gate, 'gate', torch.float32, (n, heads))
    if window is not None and (type(window) is not int or window < 1):
        raise ValueError('latent_attention: a window is a positive integer')
    window = window or 0
    lib = library.load()
    if not lib.qil_latent_attention_takes(heads, rank, rot):
        raise UnsupportedShape(f'latent attention: {heads} heads, rank {rank}, {rot} rotated elements')
    out = torch.empty((n, heads * rank), dtype=torch.float32, device=q.device)
    if LATENT_MATRIX_CORES and latent.dtype == torch.bfloat16 and cu_seqlens is not None and \
            lib.qil_latent_mfma_takes(heads, rank, rot):
        _require(cu_seqlens, 'cu_seqlens', torch.int32, (n_seqs + 1,))
        _require(seq_starts, 'seq_starts', torch.int32, (n_seqs,))
        if block_tables.shape[0] != n_seqs or block_tables.shape[1] * page_size < max_context:
            raise ValueError('one block table row per sequence, wide enough for the longest context')
        single = int(max_query == 1)
        plan = [ctypes.c_int(0) for _ in range(4)]
        lib.qil_latent_mfma_plan(n, n_seqs, single, heads, max_context, window, *[ctypes.byref(v) for v in plan])
        rt, hb, part, parts = (v.value for v in plan)
        if LATENT_KEY_PARTS is not None:
            part, parts = LATENT_KEY_PARTS[0], max(LATENT_KEY_PARTS[1], -(-max_context // LATENT_KEY_PARTS[0]))
        nbytes = lib.qil_latent_mfma_workspace(n, heads, rank, parts)
        workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=q.device) if nbytes else None
        _check(lib.qil_latent_mfma(_ptr(q), _ptr(latent), _ptr(rope), _ptr(block_tables), block_tables.shape[1],
                                   _ptr(cu_seqlens), _ptr(seq_starts), _ptr(positions), _ptr(sink), _ptr(gate), _ptr(out),
                                   _ptr(workspace), n, n_seqs, single, heads, rank, rot, page_size, float(scale), window,
                                   rt, hb, part, parts, _stream()), 'latent_mfma')
        return out
    _check(lib.qil_latent_attention(_ptr(q), _ptr(latent), _ptr(rope), _ptr(block_tables), block_tables.shape[1],
                                    _ptr(row_seq), _ptr(positions), _ptr(sink), _ptr(gate), _ptr(out), n, heads, rank, rot,
                                    page_size, float(scale), window, _code(latent.dtype), _stream()), 'latent_attention')
    return out


# ---------------------------------------------------------------------------------------------------------------
# Recurrences with a matrix state
SCAN_MODES = {'decay': 0, 'mlstm': 1, 'channel': 2}
SCAN_BLOCKS_FROM = 32           # rows of one sequence from which a step's recurrence runs in blocks side by side


def state_scan_slot(*, heads, dim, vdim, mode):
    """float32 elements of one request's state for ``state_scan``: the heads' [dim, vdim] matrices, and for 'mlstm' a
    normaliser [dim] per head and the running maximum once per head and block of the kernel (one per 16 state columns
    and one for the normaliser's)."""
    tiles = -(-vdim // 16)
    return heads * dim * vdim + (heads * (dim + tiles + 1) if SCAN_MODES[mode] == SCAN_MODES['mlstm'] else 0)


def state_scan(proj, *, mode, heads, dim, vdim, q_offset, k_offset, v_offset, state, cu_seqlens, seq_starts, seq_slots,
               n_seqs, gates=None, gate_bias=None, cap=0.0, decay=None, frequencies=None, rot=0, q_scale=1.0, k_scale=1.0,
               max_query=None):
    """S_t = a_t S_(t-1) + b_t k_t v_t^T, o_t = S_t^T q_t per head over every sequence's rows of the step, from the
    sequence's state slot (empty where the sequence starts at position 0) and back into it.

    ``proj`` [N, P]: a row holds the heads' queries from column ``q_offset``, keys from ``k_offset`` (heads * dim each)
    and values from ``v_offset`` (heads * vdim).  Mode 'decay': a_t = decay[h], b_t = 1.  Mode 'mlstm': exponential
    gates from ``gates`` float32 [N, 2 heads] (+ ``gate_bias`` [2 heads]; input gates first) soft-capped at ``cap``,
    with a running maximum and a normaliser.  Mode 'channel': every row i of a head's S keeps a_t[i] =
    sigmoid(z)^(1 / tau) of itself, with z = ``gates`` float32 [N, heads * dim] and tau = ``cap``; b_t = 1.
    Queries and keys are rotated by position on their leading ``rot``
    elements (``frequencies`` [rot / 2]) and then scaled.  ``max_query``: the most rows of one sequence, if the caller
    knows it; from ``SCAN_BLOCKS_FROM`` rows on the step is worked in blocks of 64 tokens side by side (the sums of the
    blocks, their carry from block to block, the outputs), below that token by token.
    -> (float32 [N, heads * vdim], denominators): 'decay' gives o_t and None; 'mlstm' gives S_t^T q_t undivided and
    float32 [N, heads] with max(|n_t . q_t|, exp(-m_t)) + 1e-6, which ``head_norm_gate`` divides by."""
    n = proj.shape[0]
    _require(proj, 'proj')
    code = _code(proj.dtype)
    lib = library.load()
    if not lib.qil_state_scan_takes(dim, vdim, rot):
        raise UnsupportedShape(f'state_scan: dim {dim} (up to 256), vdim {vdim}, {rot} rotated elements')
    width = proj.shape[1]
    if min(q_offset, k_offset, v_offset) < 0 or max(q_offset, k_offset) + heads * dim > width or v_offset + heads * vdim > width:
        raise ValueError('state_scan: offsets do not fit the rows')
    slot = state_scan_slot(heads=heads, dim=dim, vdim=vdim, mode=mode)
    if slot != lib.qil_state_scan_slot(heads, dim, vdim, SCAN_MODES[mode]):
        raise RuntimeError('state_scan: the kernel library lays a state slot out differently')
    _require(state, 'state', torch.float32)
    if state.ndim != 2 or state.shape[1] != slot:
        raise ValueError(f'state_scan: state must be [slots, {slot}]')
    _require(cu_seqlens, 'cu_seqlens', torch.int32, (n_seqs + 1,))
    _require(seq_starts, 'seq_starts', torch.int32, (n_seqs,))
    _require(seq_slots, 'seq_slots', torch.int32, (n_seqs,))
    if mode == 'mlstm':
        _require(gates, 'gates', torch.float32, (n, 2 * heads))
        _require(gate_bias, 'gate_bias', torch.float32, (2 * heads,))
    elif mode == 'channel':
        _require(gates, 'gates', torch.float32, (n, heads * dim))
        if not cap > 0:
            raise ValueError("state_scan: mode 'channel' needs a positive tau in the place of the cap")
    else:
        _require(decay, 'decay', torch.float32, (heads,))
    if rot:
        _require(frequencies, 'frequencies', torch.float32, (rot // 2,))
    out = torch.empty((n, heads * vdim), dtype=torch.float32, device=proj.device)
    below = torch.empty((n, heads), dtype=torch.float32, device=proj.device) if mode == 'mlstm' else None
    if max_query is not None and max_query >= SCAN_BLOCKS_FROM:
        floats = lib.qil_state_scan_chunked_workspace(n, n_seqs, heads, dim, vdim, SCAN_MODES[mode])
        workspace = torch.empty(floats, dtype=torch.float32, device=proj.device)
        _check(lib.qil_state_scan_chunked(_ptr(proj), code, width, q_offset, k_offset, v_offset, _ptr(gates),
                                          _ptr(gate_bias), float(cap), _ptr(decay), _ptr(frequencies) if rot else None,
                                          rot, float(q_scale), float(k_scale), _ptr(state), slot, _ptr(cu_seqlens),
                                          _ptr(seq_starts), _ptr(seq_slots), _ptr(out), _ptr(below), _ptr(workspace), n,
                                          n_seqs, int(max_query), heads, dim, vdim, SCAN_MODES[mode], _stream()),
               'state_scan_chunked')
        return out, below
    _check(lib.qil_state_scan(_ptr(proj), code, width, q_offset, k_offset, v_offset, _ptr(gates), _ptr(gate_bias),
                              float(cap), _ptr(decay), _ptr(frequencies) if rot else None, rot, float(q_scale),
                              float(k_scale), _ptr(state), _ptr(cu_seqlens), _ptr(seq_starts), _ptr(seq_slots), _ptr(out),
                              _ptr(below), n_seqs, heads, dim, vdim, SCAN_MODES[mode], _stream()), 'state_scan')
    return out, below


def head_norm_gate(o, gate_source, *, gate_offset, heads, vdim, weight, eps, gate, out_dtype, denominators=None):
    """Per head: o / sqrt(mean(o^2) + eps) (* weight) * act(g), ``o`` float32 [N, heads * vdim] (first divided, head by
    head, by ``denominators`` float32 [N, heads] if given), g the heads * vdim columns of ``gate_source`` from
    ``gate_offset``; ``gate``: 'sigmoid' or 'silu'.  -> [N, heads * vdim] out_dtype."""
    n = o.shape[0]
    if denominators is not None:
        _require(denominators, 'denominators', torch.float32, (n, heads))
    _require(o, 'o', torch.float32, (n, heads * vdim))
    _require(gate_source, 'gate_source', out_dtype)
    if gate_source.shape[0] != n or gate_offset + heads * vdim > gate_source.shape[1]:
        raise ValueError('head_norm_gate: the gate columns do not fit')
    if weight is not None:
        _require(weight, 'weight', torch.float32, (heads * vdim,))
    out = torch.empty((n, heads * vdim), dtype=out_dtype, device=o.device)
    _check(library.load().qil_head_norm_gate(_ptr(o), _ptr(denominators), _ptr(gate_source), gate_source.shape[1], gate_offset, _ptr(weight),
                                             _ptr(out), n, heads, vdim, float(eps), {'sigmoid': 0, 'silu': 1}[gate],
                                             _code(out_dtype), _stream()), 'head_norm_gate')
    return out


# ---------------------------------------------------------------------------------------------------------------
# Routed feed-forward
ROUTER_SCORES = {'softmax': 0, 'sigmoid': 1}
ROUTER_GROUP_SCORES = {'max': 0, 'top2': 1}


def moe_route(x, router, correction, *, groups, keep, top, renormalize=False, bias=None, score='softmax',
              group_score='max', weight_scale=1.0, renormalize_eps=0.0):
    """x [N, width] (model type), router float32 [outputs, width], correction float32 [outputs] or None ->
    (chosen int32 [N, top], weights float32 [N, top]): softmax scores over all outputs in float32; the choice goes
    by score + correction among the outputs of the ``keep`` best of ``groups`` equal groups of neighbours (a group's
    score: its best choice score); the weights are the chosen outputs' scores (divided by their sum if asked, which
    makes them the softmax over the chosen logits alone).  ``bias`` float32 [outputs]: added to the logits.
    ``score='sigmoid'``: scores are sigmoid(logit) and the choice goes by the score (+ correction);
    ``group_score='top2'``: a group's score is the sum of its two largest choice scores; with ``renormalize`` the
    divisor is the chosen scores' sum + ``renormalize_eps``; ``weight_scale`` multiplies the weights last."""
    n, width = x.shape
    _require(x, 'x')
    outputs = router.shape[0]
    _require(router, 'router', torch.float32, (outputs, width))
    if correction is not None:
        _require(correction, 'correction', torch.float32, (outputs,))
    if bias is not None:
        _require(bias, 'bias', torch.float32, (outputs,))
    lib = library.load()
    if not lib.qil_moe_takes(width, outputs, 0, groups, keep, top):
        raise UnsupportedShape(f'moe_route: {outputs} outputs in {groups} groups ({keep} kept), top {top}, width {width}')
    chosen = torch.empty((n, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=x.device)
    logits = torch.empty((n, outputs), dtype=torch.float32, device=x.device)
    _check(lib.qil_moe_route(_ptr(x), _code(x.dtype), _ptr(router), _ptr(bias), _ptr(correction), _ptr(logits), _ptr(chosen),
                             _ptr(weights), n, width, outputs, groups, keep, top, int(bool(renormalize)),
                             ROUTER_SCORES[score], ROUTER_GROUP_SCORES[group_score], float(weight_scale),
                             float(renormalize_eps), _stream()), 'moe_route')
    return chosen, weights


def moe_experts(x, chosen, weights, gate_up, down, *, activation, limit=0.0, alpha=1.0, lazy=False):
    """The weighted sum of the chosen experts' outputs, float32 [N, width]; with ``lazy`` a ``RoutedSum`` (the pairs'
    rows, for a norm that makes the sum while it loads them).  ``gate_up`` [experts, 2, ff, width] (an
    expert's gate rows, then its up rows), ``down`` [experts, width, ff], both of x's type; an expert computes
    down(act(gate x, up x)) with ``activation`` of ``GATE_FUNCTIONS``.  A chosen index from ``experts`` on is an
    identity expert: its output is x itself.  The pairs (token, chosen expert) are grouped by expert on the device;
    the host sees no routing result, so a step may be captured into a graph."""
    n, width = x.shape
    top = chosen.shape[1]
    _require(x, 'x')
    _require(chosen, 'chosen', torch.int32, (n, top))
    _require(weights, 'weights', torch.float32, (n, top))
    experts, ff = gate_up.shape[0], gate_up.shape[2]
    _require(gate_up, 'gate_up', x.dtype, (experts, 2, ff, width))
    _require(down, 'down', x.dtype, (experts, width, ff))
    lib = library.load()
    pairs = n * top
    tile_rows = lib.qil_moe_tile_rows(pairs, experts)
    max_tiles = lib.qil_moe_max_tiles(pairs, experts, tile_rows)
    scratch = torch.empty(3 * max_tiles + pairs, dtype=torch.int32, device=x.device)
    hidden = torch.empty((pairs, ff), dtype=x.dtype, device=x.device)
    y = torch.empty((pairs, width), dtype=torch.float32, device=x.device)
    out = None if lazy else torch.empty((n, width), dtype=torch.float32, device=x.device)
    _check(lib.qil_moe_experts(_ptr(x), _code(x.dtype), _ptr(chosen), _ptr(weights), _ptr(gate_up), _ptr(down),
                               _ptr(scratch), scratch[3 * max_tiles:].data_ptr(), _ptr(hidden), _ptr(y), _ptr(out), n, width,
                               ff, experts, top, tile_rows, max_tiles, GATE_FUNCTIONS[activation], float(limit),
                               float(alpha), _stream()), 'moe_experts')
    return RoutedSum(x, y, chosen, weights, experts) if lazy else out


# ---------------------------------------------------------------------------------------------------------------
# Small float32 steps between products, and the selective state-space mixer's two kernels
def _any_operand(value, name, shape):
    """(pointer, dtype code, splits) of an input that is a bfloat16 or float32 tensor or Partials."""
    if isinstance(value, Partials):
        _require(value.tensor, name, torch.float32, (value.splits, *shape))
        return value.tensor.data_ptr(), 0, value.splits
    _require(value, name, None, shape)
    return value.data_ptr(), _code(value.dtype), 1


def scaled_sum(a, b, a_scale, b_scale):
    """a_scale * a + b_scale * b as float32 [N, H]; ``a`` and ``b`` are tensors (float32 or bfloat16) or Partials."""
    n, width = a.shape
    if tuple(b.shape) != (n, width):
        raise ValueError(f'scaled_sum: {tuple(a.shape)} and {tuple(b.shape)}')
    a = _plain_delta(a)
    pa, ca, sa = _any_operand(a, 'a', (n, width))
    pb, cb, sb = _any_operand(b, 'b', (n, width))
    out = torch.empty((n, width), dtype=torch.float32, device=a.device)
    _check(library.load().qil_scaled_sum(pa, ca, sa, pb, cb, sb, float(a_scale), float(b_scale), _ptr(out), n, width,
                                         _stream()), 'scaled_sum')
    return out


def sigmoid_gate(x, source, *, offset):
    """x * sigmoid(source[:, offset : offset + C]) for x [N, C] of the model's type; ``source`` [N, W] is a tensor of
    that type or Partials (the stacked product whose last columns are the gate's logits).  The sigmoid and the
    product are float32; one rounding."""
    n, columns = x.shape
    _require(x, 'x')
    width = source.shape[1]
    if source.shape[0] != n or offset < 0 or offset + columns > width:
        raise ValueError('sigmoid_gate: the gate columns do not lie inside the source')
    pointer, code, splits = _any_operand(source, 'source', (n, width))
    out = torch.empty_like(x)
    _check(library.load().qil_sigmoid_gate(_ptr(x), pointer, code, splits, width, int(offset), _ptr(out), n, columns,
                                           _code(x.dtype), _stream()), 'sigmoid_gate')
    return out


def soft_cap(x, cap):
    """cap * tanh(x / cap) of a float32 tensor, in place; returns it."""
    _require(x, 'x', torch.float32)
    _check(library.load().qil_soft_cap(_ptr(x), float(cap), x.numel(), _stream()), 'soft_cap')
    return x


def check_selective_scan_geometry(*, inner, state, taps):
    """Sizes the selective scan's kernels take; called when the part is built."""
    if not (inner >= 1 and 1 <= state <= 256 and 1 <= taps <= 64):
        raise UnsupportedShape(f'selective scan: inner {inner}, state {state} (at most 256), {taps} taps (at most 64)')


CONV_ACTIVATIONS = {None: 0, 'silu': 1}


def channel_conv(x, weight, bias, *, columns, state, cu_seqlens, seq_starts, seq_slots, row_seq, n_seqs, activation,
                 out_dtype):
    """act(bias + causal convolution over time) on the first ``columns`` columns of ``x`` [N, W] (tensor of the
    model's type or Partials): out[t, c] = act(bias[c] + sum_j weight[j, c] * x[t - taps + 1 + j, c]) over the rows of
    every sequence of the step and the taps - 1 inputs before them, which are the sequence's state (``state`` float32
    [slots, taps - 1, columns]: read unless the sequence starts at position 0, and left holding the sequence's last
    taps - 1 inputs).  ``weight`` float32 [taps, columns], ``bias`` float32 [columns] or None.  -> [N, columns] of
    ``out_dtype``; float32 arithmetic, one rounding."""
    n, width = x.shape
    taps = weight.shape[0]
    _require(weight, 'weight', torch.float32, (taps, columns))
    if bias is not None:
        _require(bias, 'bias', torch.float32, (columns,))
    if taps > 1:
        _require(state, 'state', torch.float32)
        if state.ndim != 3 or tuple(state.shape[1:]) != (taps - 1, columns):
            raise ValueError(f'channel_conv: state must be [slots, {taps - 1}, {columns}]')
    _require(cu_seqlens, 'cu_seqlens', torch.int32, (n_seqs + 1,))
    _require(seq_starts, 'seq_starts', torch.int32, (n_seqs,))
    _require(seq_slots, 'seq_slots', torch.int32, (n_seqs,))
    _require(row_seq, 'row_seq', torch.int32, (n,))
    pointer, code, splits = _any_operand(x, 'x', (n, width))
    out = torch.empty((n, columns), dtype=out_dtype, device=weight.device)
    _check(library.load().qil_channel_conv(pointer, code, splits, width, _ptr(weight), _ptr(bias),
                                           _ptr(state) if taps > 1 else None, _ptr(cu_seqlens), _ptr(seq_starts),
                                           _ptr(seq_slots), _ptr(row_seq), _ptr(out), _code(out_dtype), n, columns, taps,
                                           CONV_ACTIVATIONS[activation], _stream()), 'channel_conv')
    return out


def selective_scan(u, dt, bc, gate, *, dt_bias, a, d, state, gate_offset, cu_seqlens, seq_starts, seq_slots, n_seqs,
                   max_query, out_dtype):
    """The selective scan over every sequence of the step, its rows in order:

        step = softplus(dt[t, c] + dt_bias[c]);   S[c, n] <- exp(step * a[c, n]) * S[c, n] + step * u[t, c] * B[t, n]
        y[t, c] = (sum_n S[c, n] * C[t, n] + d[c] * u[t, c]) * silu(z[t, c])

    ``u`` [N, C] of the model's type; ``dt`` [N, C], ``bc`` [N, 2 n] (B then C) and ``gate`` [N, W] (z from column
    ``gate_offset`` on) are tensors of that type or Partials; ``dt_bias``, ``d`` float32 [C], ``a`` float32 [C, n];
    ``state`` float32 [slots, C, n]: read unless the sequence starts at position 0, and left holding S after the
    sequence's last row.  Everything from the step size on is float32.  -> [N, C] of ``out_dtype``.
    ``max_query``: the most rows of one sequence.  Up to 32 states a thread takes a channel with its states in
    registers; sequences of more than 64 rows are then cut into chunks of 64 tokens that run side by side (every chunk
    from zero, a carry over the chunks, every chunk again from its true state).  The forms differ by rounding only."""
    n, channels = u.shape
    states = a.shape[1]
    _require(u, 'u', out_dtype)
    _require(a, 'a', torch.float32, (channels, states))
    _require(dt_bias, 'dt_bias', torch.float32, (channels,))
    _require(d, 'd', torch.float32, (channels,))
    _require(state, 'state', torch.float32)
    if state.ndim != 3 or tuple(state.shape[1:]) != (channels, states):
        raise ValueError(f'selective_scan: state must be [slots, {channels}, {states}]')
    _require(cu_seqlens, 'cu_seqlens', torch.int32, (n_seqs + 1,))
    _require(seq_starts, 'seq_starts', torch.int32, (n_seqs,))
    _require(seq_slots, 'seq_slots', torch.int32, (n_seqs,))
    gate_columns = gate.shape[1]
    if gate_offset < 0 or gate_offset + channels > gate_columns:
        raise ValueError('selective_scan: the gate columns do not lie inside their source')
    p_dt, c_dt, s_dt = _any_operand(dt, 'dt', (n, channels))
    p_bc, c_bc, s_bc = _any_operand(bc, 'bc', (n, 2 * states))
    p_g, c_g, s_g = _any_operand(gate, 'gate', (n, gate_columns))
    lib = library.load()
    if not lib.qil_selective_scan_takes(channels, states, 1):
        raise UnsupportedShape(f'selective_scan: {channels} channels of {states} states')
    y = torch.empty((n, channels), dtype=out_dtype, device=u.device)
    nbytes = lib.qil_selective_scan_workspace(n_seqs, int(max_query), channels, states)
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device=u.device) if nbytes else None
    _check(lib.qil_selective_scan(_ptr(u), p_dt, c_dt, s_dt, _ptr(dt_bias), _ptr(a), p_bc, c_bc, s_bc, _ptr(d), p_g, c_g,
                                  s_g, gate_columns, int(gate_offset), _ptr(state), _ptr(cu_seqlens), _ptr(seq_starts),
                                  _ptr(seq_slots), _ptr(y), _code(out_dtype), n, n_seqs, channels, states, int(max_query),
                                  _ptr(workspace), _stream()), 'selective_scan')
    return y
