"""The HIP kernels as functions on torch tensors.

Every function checks on the host that its operands have the element types, shapes and layout
the kernel and its grid assume, and raises otherwise: a kernel is never launched on operands it
would read or write out of bounds. Tensors only carry memory; no torch operator computes
anything here. Kernels run on torch's current stream."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .library import check, library

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
EPILOGUES = {None: 0, "none": 0, "gelu_new": 1, "gelu": 2}


class OperandError(ValueError):
    pass


def _require(condition: bool, message: str) -> None:
    if not condition:
        raise OperandError(message)


def _code(dtype: torch.dtype) -> int:
    if not (dtype in _DTYPE_CODE):
        raise OperandError(f"no kernel for element type {dtype}")
    return _DTYPE_CODE[dtype]


def _device_tensor(t: torch.Tensor, name: str, dtype=None, dim=None) -> None:
    if not (isinstance(t, torch.Tensor)):
        raise OperandError(f"{name} is not a tensor")
    if not (t.is_cuda):
        raise OperandError(f"{name} is not on the GPU: there is no CPU path")
    if dtype is not None:
        if not (t.dtype == dtype):
            raise OperandError(f"{name} must be {dtype}, not {t.dtype}")
    if dim is not None:
        if not (t.dim() == dim):
            raise OperandError(f"{name} must have {dim} dimensions, not {t.dim()}")
    if not (t.is_contiguous()):
        raise OperandError(f"{name} must be contiguous")


def _ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()  # ctypes turns the integer into the pointer argument


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The raw handle of torch's current stream (also the capturing one inside a graph capture)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def embed(tokens, positions, wte, wpe, out=None, token_sources=None, token_slots=None):
    """out[t] = wte[tokens[t]] + wpe[positions[t]] in float32 (``wpe`` None: the token row alone). A
    negative token gives a zero row.
    With ``token_sources`` and ``token_slots`` the token of a row whose source is not negative is
    token_slots[source]; it is also written into ``tokens``."""
    _device_tensor(tokens, "tokens", torch.int32, 1)
    _device_tensor(positions, "positions", torch.int32, 1)
    _device_tensor(wte, "wte", dim=2)
    n, width = tokens.shape[0], wte.shape[1]
    _require(positions.shape[0] == n, "tokens and positions differ in length")
    if wpe is not None:
        _device_tensor(wpe, "wpe", wte.dtype, 2)
        _require(wpe.shape[1] == width, "wte and wpe differ in width")
    if token_sources is not None:
        _device_tensor(token_sources, "token_sources", torch.int32, 1)
        _device_tensor(token_slots, "token_slots", torch.int32, 1)
        _require(token_sources.shape[0] >= n, "fewer sources than tokens")
    if out is None:
        out = torch.empty((n, width), dtype=torch.float32, device=tokens.device)
    _device_tensor(out, "out", torch.float32, 2)
    _require(tuple(out.shape) == (n, width), "out has the wrong shape")
    check(library().mllm_embed(_ptr(tokens), _ptr(positions), _ptr(token_sources), _ptr(token_slots if token_sources is not None else None),
                               _ptr(wte), _ptr(wpe), _ptr(out), n, width, _code(wte.dtype), _stream()))
    return out


def layernorm(x, gamma, beta, eps, out_dtype=torch.float32, row_index=None, out=None, with_sums=False, packed_out=False):
    """Row LayerNorm of float32 rows, plain or pending (PendingRows: the sums are taken on the way
    in); ``row_index`` (int32) picks the input row of each output row. ``with_sums``: returns
    (normalised rows, the rows with their sums taken) - what the residual stream goes on with.
    ``packed_out``: the normalised rows come as PackedRows, for a product of few rows."""
    if with_sums:
        _require(row_index is None, "the rows with their sums taken are not gathered")
        if not isinstance(x, PendingRows) or x.base.shape[1] % 4 or (x.partials is None and x.bias is None):
            x = settle(x)
            return layernorm(x, gamma, beta, eps, out_dtype=out_dtype, out=out, packed_out=packed_out), x
    pending = isinstance(x, PendingRows)
    if pending and x.base.shape[1] % 4:
        x, pending = settle(x), False
    if pending:
        base, partials, bias, n_partials = _pending(x)
    else:
        _device_tensor(x, "x", torch.float32, 2)
        base = x
    width = base.shape[1]
    _device_tensor(gamma, "gamma", torch.float32, 1)
    _device_tensor(beta, "beta", torch.float32, 1)
    _require(gamma.shape[0] == width and beta.shape[0] == width, "gamma/beta do not match the row width")
    n = base.shape[0]
    if row_index is not None:
        _device_tensor(row_index, "row_index", torch.int32, 1)
        n = row_index.shape[0]
    if packed_out:
        _require(out is None, "packed rows are allocated here")
        result = empty_packed_rows(n, width, out_dtype, base.device)
        out = result.data
    else:
        if out is None:
            out = torch.empty((n, width), dtype=out_dtype, device=base.device)
        _device_tensor(out, "out", out_dtype, 2)
        _require(tuple(out.shape) == (n, width), "out has the wrong shape")
        result = out
    if pending:
        summed = torch.empty_like(base) if with_sums else None
        check(library().mllm_pending_layernorm(_ptr(base), _ptr(partials), _ptr(bias), n_partials, base.shape[0], _ptr(row_index), _ptr(gamma),
                                               _ptr(beta), _ptr(out), _ptr(summed), n, width, float(eps), _code(out_dtype), int(packed_out), _stream()))
        if with_sums:
            return result, summed
    else:
        check(library().mllm_layernorm(_ptr(base), _ptr(row_index), _ptr(gamma), _ptr(beta), _ptr(out), n, width, float(eps), _code(out_dtype),
                                       int(packed_out), _stream()))
    return result


def add(a, b, out=None):
    """a (float32) + b (float32 or bfloat16) in float32."""
    _device_tensor(a, "a", torch.float32)
    _device_tensor(b, "b")
    _require(a.shape == b.shape, "a and b differ in shape")
    if out is None:
        out = torch.empty_like(a)
    _device_tensor(out, "out", torch.float32)
    _require(out.shape == a.shape, "out has the wrong shape")
    check(library().mllm_add(_ptr(a), _ptr(b), _ptr(out), a.numel(), _code(b.dtype), _stream()))
    return out


class PackedMatrix:
    """A weight matrix [rows (out), cols (in)] in the packed layout of the matrix kernels: chunks
    of 16 rows x 64 bytes, each chunk's 16-byte pieces in the order the lanes of a wave take them
    as matrix-core operands, zeros beyond the matrix. ``data`` is the flat device tensor."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device


# Rows from which on activations are worth passing in the packed layout between the kernels of a
# layer (measured on MI355X: from 17 rows the products of few rows gain up to a half; below, nothing
# in bfloat16, and the 32-bit path loses 7 %).
PACKED_ROWS_FROM = 17


class PackedRows(PackedMatrix):
    """Rows of activations [rows, cols] in the same packed layout, as a kernel left them for a
    product of few rows to read (what lies beyond the rows and columns is not defined, and the
    product does not use it)."""


def empty_packed_rows(rows: int, cols: int, dtype, device) -> PackedRows:
    per_piece = 16 // (4 if dtype == torch.float32 else 2)
    chunks = -(-rows // 16) * -(-cols // (4 * per_piece))
    return PackedRows(torch.empty(chunks * 64 * per_piece, dtype=dtype, device=device), rows, cols)


def takes_packed_rows(rows: int, weight, dtype) -> bool:
    """Whether ``linear`` / ``linear_qkv_cache`` of so many rows with this weight reads (and can
    write) rows in the packed layout: where the product takes the kernel for few rows."""
    _, _, n, k = _matrix(weight, "weight", dtype)
    return bool(library().mllm_gemm_takes_packed_rows(int(rows), n, k, _code(dtype)))


def _rows(x, name):
    """(pointer, packed flag, rows, cols, dtype, device) of activations given plain or packed."""
    if isinstance(x, PackedRows):
        return _ptr(x.data), 1, x.rows, x.cols, x.data.dtype, x.data.device
    _device_tensor(x, name, dim=2)
    return _ptr(x), 0, x.shape[0], x.shape[1], x.dtype, x.device


def pack_matrix(src, dtype=None, transpose=False) -> PackedMatrix:
    """A float32/bfloat16 matrix [out, in] (or, with ``transpose``, stored [in, out]) in the packed
    layout, in element type ``dtype`` (default: its own). Load-time work on weights."""
    _device_tensor(src, "src", dim=2)
    dtype = src.dtype if dtype is None else dtype
    rows, cols = (src.shape[1], src.shape[0]) if transpose else src.shape
    _require(rows > 0 and cols > 0, "an empty matrix cannot be packed")
    lib = library()
    data = torch.empty((lib.mllm_packed_elements(rows, cols, _code(dtype)),), dtype=dtype, device=src.device)
    check(lib.mllm_pack_matrix(_ptr(src), _ptr(data), rows, cols, _code(src.dtype), _code(dtype), int(bool(transpose)), _stream()))
    return PackedMatrix(data, rows, cols)


def _matrix(weight, name, dtype):
    """(pointer, packed flag, rows, cols) of a weight given row-major or packed."""
    if isinstance(weight, PackedMatrix):
        _device_tensor(weight.data, name, dtype, 1)
        return _ptr(weight.data), 1, weight.rows, weight.cols
    _device_tensor(weight, name, dtype, 2)
    return _ptr(weight), 0, weight.shape[0], weight.shape[1]


def linear(x, weight, bias=None, activation=None, residual=None, out_dtype=None, out=None, packed_out=False):
    """act(x @ weight.T + bias) (+ residual). ``weight`` is [out, in], a row-major tensor or a
    PackedMatrix; sums are float32. x may be PackedRows, and with ``packed_out`` the result is,
    where ``takes_packed_rows`` says so.

    x and weight share their element type (float32: true 32-bit MFMA; bfloat16: bf16 MFMA);
    bias and residual are float32; a residual makes the output float32."""
    x_ptr, x_packed, m, k, x_dtype, device = _rows(x, "x")
    w_ptr, w_packed, n, w_cols = _matrix(weight, "weight", x_dtype)
    if not (w_cols == k):
        raise OperandError(f"x has {k} columns but weight has {w_cols}")
    if not (activation in EPILOGUES):
        raise OperandError(f"unknown activation {activation!r}")
    if bias is not None:
        _device_tensor(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == n, "bias does not match weight")
    if out_dtype is None:
        out_dtype = torch.float32 if residual is not None else x_dtype
    if residual is not None:
        _device_tensor(residual, "residual", torch.float32, 2)
        _require(tuple(residual.shape) == (m, n), "residual has the wrong shape")
        _require(out_dtype == torch.float32, "a residual sum is float32")
    _require(x_dtype != torch.float32 or out_dtype == torch.float32, "float32 inputs give float32 outputs")
    if packed_out:
        _require(out is None and residual is None, "packed rows are allocated here, and hold no residual sum")
        result = empty_packed_rows(m, n, out_dtype, device)
        out = result.data
    else:
        if out is None:
            out = torch.empty((m, n), dtype=out_dtype, device=device)
        _device_tensor(out, "out", out_dtype, 2)
        _require(tuple(out.shape) == (m, n), "out has the wrong shape")
        result = out
    check(library().mllm_gemm(x_ptr, w_ptr, w_packed, _ptr(bias), _ptr(residual), _ptr(out), m, n, k, _code(x_dtype), _code(out_dtype),
                              EPILOGUES[activation], x_packed, int(packed_out), _stream()))
    return result


def split_blocks(weight, dtype, rows: int = 1) -> int:
    """Into how many partial products along K ``linear_split`` should cut the product of ``rows``
    rows with this weight (1: better left whole): more than one where few rows and few output
    columns meet a long K. The same for all row counts up to 64, and for all that need the same
    number of 128-row tiles."""
    _, _, n, k = _matrix(weight, "weight", dtype)
    return int(library().mllm_gemm_split_blocks(int(rows), n, k, _code(dtype)))


def linear_split(x, weight, k_blocks: int):
    """x @ weight.T as ``k_blocks`` partial products over consecutive parts of K: float32
    [k_blocks, rows, out]; their sum is the product. The blocks of a product with few output
    columns each read whole rows of x; cut along K they read a part, and many more run. x may be
    PackedRows (up to 64 rows)."""
    x_ptr, x_packed, m, k, x_dtype, device = _rows(x, "x")
    w_ptr, w_packed, n, w_cols = _matrix(weight, "weight", x_dtype)
    if not (w_cols == k):
        raise OperandError(f"x has {k} columns but weight has {w_cols}")
    partials = torch.empty((k_blocks, m, n), dtype=torch.float32, device=device)
    check(library().mllm_gemm_split(x_ptr, w_ptr, w_packed, _ptr(partials), m, n, k, _code(x_dtype), int(k_blocks), x_packed, _stream()))
    return partials


def convert(src, dtype, transpose=False, out=None):
    """A 1-D or 2-D float32/bfloat16 tensor in another element type (or the same: a copy), a 2-D one
    transposed on request (contiguous result, written into ``out`` if one is given). Load-time work on weights."""
    _device_tensor(src, "src")
    _require(src.dim() in (1, 2), "convert takes vectors and matrices")
    rows, cols = (1, src.shape[0]) if src.dim() == 1 else src.shape
    _require(not transpose or src.dim() == 2, "only a matrix can be transposed")
    shape = src.shape if not transpose else (cols, rows)
    if out is None:
        out = torch.empty(tuple(shape), dtype=dtype, device=src.device)
    _device_tensor(out, "out", dtype)
    _require(tuple(out.shape) == tuple(shape), "out has the wrong shape")
    check(library().mllm_convert(_ptr(src), _ptr(out), rows, cols, _code(src.dtype), _code(dtype), int(bool(transpose)), _stream()))
    return out


def _check_pages(k_pages, v_pages, n_kv_heads, head_size):
    _device_tensor(k_pages, "k_pages", dim=4)
    _device_tensor(v_pages, "v_pages", k_pages.dtype, 4)
    _require(k_pages.shape == v_pages.shape, "key and value pages differ in shape")
    _require(k_pages.shape[1] == n_kv_heads and k_pages.shape[3] == head_size, "pages do not match the heads")
    return k_pages.shape[0], k_pages.shape[2]


def cache_write(k_src, v_src, k_pages, v_pages, slots, n_kv_heads, head_size):
    """Copies the key and value columns of each row into cache slot slots[row] (negative: skip).

    k_src / v_src are 2-D views [rows, n_kv_heads*head_size] whose rows may be strided (slices
    of a fused projection); pages are [num_pages, n_kv_heads, page_size, head_size]."""
    num_pages, page_size = _check_pages(k_pages, v_pages, n_kv_heads, head_size)
    width = n_kv_heads * head_size
    for t, name in ((k_src, "k_src"), (v_src, "v_src")):
        if not (t.is_cuda and t.dim() == 2 and t.dtype == k_pages.dtype):
            raise OperandError(f"{name} must be a 2-D GPU tensor of the pages' type")
        if not (t.shape[1] == width and t.stride(1) == 1):
            raise OperandError(f"{name} must have {width} contiguous columns")
    _require(k_src.shape[0] == v_src.shape[0] and k_src.stride(0) == v_src.stride(0), "k_src and v_src differ in rows or stride")
    _device_tensor(slots, "slots", torch.int32, 1)
    n = k_src.shape[0]
    _require(slots.shape[0] >= n, "fewer slots than rows")
    check(library().mllm_cache_write(_ptr(k_src), _ptr(v_src), k_src.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(slots), n, n_kv_heads, head_size, page_size, _code(k_pages.dtype), _stream()))


def linear_qkv_cache(x, weight, bias, k_pages, v_pages, slots, n_heads, n_kv_heads, head_size):
    """The fused q/k/v projection: returns q [rows, n_heads*head_size] and writes the key and value
    columns straight into the cache pages at slots[row] (negative: skip). x may be PackedRows where
    ``takes_packed_rows`` says so."""
    x_ptr, x_packed, m, k, x_dtype, device = _rows(x, "x")
    w_ptr, w_packed, w_rows, w_cols = _matrix(weight, "weight", x_dtype)
    num_pages, page_size = _check_pages(k_pages, v_pages, n_kv_heads, head_size)
    _require(k_pages.dtype == x_dtype, "pages and x differ in element type")
    q_width, kv_width = n_heads * head_size, n_kv_heads * head_size
    _require((w_rows, w_cols) == (q_width + 2 * kv_width, k), "weight does not match the heads or x")
    _require(k % (16 // (4 if x_dtype == torch.float32 else 2)) == 0, "the input width is not a multiple of a 16-byte piece")
    if bias is not None:
        _device_tensor(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == w_rows, "bias does not match weight")
    _device_tensor(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] >= m, "fewer slots than rows")
    q = torch.empty((m, q_width), dtype=x_dtype, device=device)
    check(library().mllm_gemm_qkv_cache(x_ptr, w_ptr, w_packed, _ptr(bias), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(slots), m, k, q_width,
                                        kv_width, n_kv_heads, head_size, page_size, _code(x_dtype), x_packed, _stream()))
    return q


_units: dict = {}


def _compute_units(device) -> int:
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _units:
        _units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _units[index]


DECODE_MAX_Q_LEN = 8        # portions up to this many tokens take the split-key kernel
DECODE_TARGET_WAVES = 4096  # the most waves a launch should have: 16 to each of 256 compute units are resident at once (measured: a
                            # second round of blocks costs more than longer shares of the keys per wave)
DECODE_MIN_SPLIT = 64       # keys a wave should at least have
DECODE_MAX_SPLITS = 16      # waves per block
DECODE_MAX_PARTS = 64       # runs a token's keys are cut into at most, a block each, where (token, head) pairs are few
# What such a run should at least hold. Measured on MI355X with heads of 64: up to some 32 pairs (a single token) runs
# of 512 keys pay (12 pairs, 3,000 keys: 15.3 -> 12.4 us in bfloat16, 23.2 -> 15.1 in 32-bit; 32 pairs with heads of
# 128, 8,000 keys: 76.8 -> 33.5 us); around 100 pairs only runs of 4 KiB a head dimension do, which is 1,024 keys in
# 32-bit (3,900 keys: 53.7 -> 42.3 us) and 2,048 in bfloat16 (where two runs of 1,000 cost 2 us more than one of 2,000).
DECODE_MIN_PART_FEW = 512
DECODE_MIN_PART_BYTES = 4096


_arrival_counters: dict = {}
_outgrown_counters: list = []


def _arrivals(k_pages, rows: int, n_heads: int):
    """Counters, zero between launches, for the decode attention's blocks that share a (row, head): one set for each
    cache tensor (a layer of an engine), which serves one step at a time; the parts of a step that run side by side take
    different rows of it. Never given back: a captured step keeps launching with the address it was captured with."""
    key = (k_pages.device.index, k_pages.data_ptr())
    counters = _arrival_counters.get(key)
    if counters is None or counters.shape[0] < rows * n_heads:
        if torch.cuda.is_current_stream_capturing():
            # memory taken inside a capture belongs to the captured graph: this launch alone gets it (and the fill
            # that zeroes it is replayed with the launch)
            return torch.zeros(rows * n_heads, dtype=torch.int32, device=k_pages.device)
        if counters is not None:
            _outgrown_counters.append(counters)
        counters = _arrival_counters[key] = torch.zeros(max(rows * n_heads, 1024), dtype=torch.int32, device=k_pages.device)
    return counters


def paged_attention(q, k_pages, v_pages, token_request, positions, block_tables, n_heads, n_kv_heads, head_size, scale, window=0, max_q_len=None, max_len=None, q_starts=None, context_lens=None, out=None,
                    short_rows=None, short_requests=None, packed_out=False, first_row=0):
    """Causal attention of each row of q over its request's cached keys (max(0, p-window+1)..p).

    q is a 2-D view [rows, n_heads*head_size] (rows may be strided); token_request[row] is the
    row of block_tables that holds the request's pages (negative: padding row, output zero).
    ``max_q_len`` (the longest portion in the batch) picks the kernel; ``max_len`` (the longest
    sequence after this step) only sets how many waves share a token's keys. ``q_starts``
    ([requests + 1], first row of each request's portion; its rows are contiguous) and
    ``context_lens`` ([requests], keys stored before this step) let long portions take the
    matrix-core kernel, which walks tiles of one request's queries. ``short_rows`` and
    ``short_requests``: the first so many rows are the portions of the first so many requests and
    none of them is longer than DECODE_MAX_Q_LEN, while the rest are longer portions; a batch of
    both kinds then runs as two launches, each kind in its own kernel (a single decoded token with
    a long context would otherwise walk all its keys in one wave of the kernel for portions).
    ``packed_out``: where the kernel for decoding and short portions runs, the rows come as
    PackedRows (for the output product of few rows that reads them next); elsewhere as ever.
    ``first_row``: where the rows are a part of a step's batch whose other parts may run at the same time on other
    streams, the place of the first of them in the whole batch (kernels that keep counters per row keep them apart by it)."""
    _check_pages(k_pages, v_pages, n_kv_heads, head_size)
    page_size = k_pages.shape[2]
    width = n_heads * head_size
    _require(q.is_cuda and q.dim() == 2 and q.dtype == k_pages.dtype, "q must be a 2-D GPU tensor of the pages' type")
    if not (q.shape[1] == width and q.stride(1) == 1):
        raise OperandError(f"q must have {width} contiguous columns")
    n = q.shape[0]
    _device_tensor(token_request, "token_request", torch.int32, 1)
    _device_tensor(positions, "positions", torch.int32, 1)
    _device_tensor(block_tables, "block_tables", torch.int32, 2)
    _require(token_request.shape[0] >= n and positions.shape[0] >= n, "fewer positions than rows")
    if out is None:
        out = torch.empty((n, width), dtype=q.dtype, device=q.device)
    _device_tensor(out, "out", q.dtype, 2)
    _require(tuple(out.shape) == (n, width), "out has the wrong shape")
    lib = library()
    if n == 0:
        return out
    rows_aligned = q.data_ptr() % 16 == 0 and (q.stride(0) * q.element_size()) % 16 == 0  # 16-byte loads of q
    if (short_rows is not None and short_requests is not None and 0 < short_rows < n and max_q_len is not None
            and max_q_len > DECODE_MAX_Q_LEN and q_starts is not None and context_lens is not None and rows_aligned
            and lib.mllm_attention_decode_supported(head_size, page_size, _code(q.dtype))
            and lib.mllm_attention_prefill_supported(head_size, page_size)):
        _require(0 < short_requests < context_lens.shape[0], "short_requests does not cut the batch in two")
        common = dict(n_heads=n_heads, n_kv_heads=n_kv_heads, head_size=head_size, scale=scale, window=window, max_len=max_len, first_row=first_row)
        paged_attention(q[:short_rows], k_pages, v_pages, token_request, positions, block_tables, max_q_len=DECODE_MAX_Q_LEN,
                        q_starts=q_starts[: short_requests + 1], context_lens=context_lens[:short_requests],
                        out=out[:short_rows], **common)
        # the longer portions: their requests' entries of q_starts still count rows from the top of q
        paged_attention(q, k_pages, v_pages, token_request, positions, block_tables[short_requests:], max_q_len=max_q_len,
                        q_starts=q_starts[short_requests:], context_lens=context_lens[short_requests:], out=out, **common)
        return out
    if (max_q_len is not None and max_q_len <= DECODE_MAX_Q_LEN and rows_aligned
            and lib.mllm_attention_decode_supported(head_size, page_size, _code(q.dtype))):
        # decoding and short portions: a block per (token, head) whose waves share the keys; as many
        # waves per block as keep the launch within what is resident at once, never more than one
        # per 64 keys of reach
        reach = block_tables.shape[1] * page_size if max_len is None else max(1, min(max_len, block_tables.shape[1] * page_size))
        if window:
            reach = min(reach, int(window))
        # few tokens with many keys: a token's keys in several runs, a block each, so that the blocks are about as many
        # as the chip has compute units, and a second small kernel that puts the runs together
        n_parts, units = 1, _compute_units(q.device)
        min_part = DECODE_MIN_PART_FEW if 8 * n * n_heads <= units else DECODE_MIN_PART_BYTES // q.element_size()
        while n_parts < DECODE_MAX_PARTS and 2 * n * n_heads * n_parts <= units and 2 * n_parts * min_part <= reach:
            n_parts *= 2
        part_reach = -(-reach // n_parts)
        n_splits = 1
        while n_splits < DECODE_MAX_SPLITS and 2 * n * n_heads * n_parts * n_splits <= DECODE_TARGET_WAVES and n_splits * DECODE_MIN_SPLIT < part_reach:
            n_splits *= 2
        result = out
        if packed_out:
            result = empty_packed_rows(n, width, q.dtype, q.device)
            out = result.data
        parts = arrivals = None
        if n_parts > 1:
            parts = torch.empty((n, n_heads, n_parts, head_size + 2), dtype=torch.float32, device=q.device)
            arrivals = _arrivals(k_pages, int(first_row) + n, n_heads)[int(first_row) * n_heads :]
        check(lib.mllm_attention_decode(_ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), width if packed_out else out.stride(0),
                                        _ptr(token_request), _ptr(positions), _ptr(block_tables), block_tables.shape[1], n, n_heads, n_kv_heads,
                                        head_size, page_size, int(window), float(scale), n_splits, _code(q.dtype), int(packed_out),
                                        n_parts, _ptr(parts), _ptr(arrivals), _stream()))
        return result
    if (max_q_len is not None and max_q_len > DECODE_MAX_Q_LEN and q_starts is not None and context_lens is not None
            and rows_aligned and lib.mllm_attention_prefill_supported(head_size, page_size)):
        _device_tensor(q_starts, "q_starts", torch.int32, 1)
        _device_tensor(context_lens, "context_lens", torch.int32, 1)
        n_requests = context_lens.shape[0]
        _require(q_starts.shape[0] == n_requests + 1, "q_starts must have one entry more than context_lens")
        _require(block_tables.shape[0] >= n_requests, "fewer block tables than requests")
        check(lib.mllm_attention_prefill(_ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_starts), _ptr(context_lens), _ptr(block_tables), block_tables.shape[1], n_requests, int(max_q_len), int(max_len or 0), n_heads, n_kv_heads, head_size, page_size, int(window), float(scale), _code(q.dtype), _stream()))
        return out
    check(lib.mllm_attention(_ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(token_request), _ptr(positions), _ptr(block_tables), block_tables.shape[1], n, n_heads, n_kv_heads, head_size, page_size, int(window), float(scale), _code(q.dtype), _stream()))
    return out


def sample(logits, temperatures=None, top_ps=None, seeds=None, steps=None, out=None, token_slots=None, slot_of_row=None):
    """One token per row of float32 logits. Without temperatures (or where one is 0): argmax by
    numpy's rules. Else a draw from softmax(logits/temperature) within the top_p nucleus; the
    random numbers are a function of (seeds[row], steps[row], token index) alone. With
    ``token_slots`` and ``slot_of_row`` the token of row r is also stored in
    token_slots[slot_of_row[r]] (negative: not stored)."""
    _device_tensor(logits, "logits", torch.float32, 2)
    n, vocab = logits.shape
    for t, name, dtype in ((temperatures, "temperatures", torch.float32), (top_ps, "top_ps", torch.float32), (seeds, "seeds", torch.int64), (steps, "steps", torch.int32)):
        if t is not None:
            _device_tensor(t, name, dtype, 1)
            if not (t.shape[0] >= n):
                raise OperandError(f"{name} has fewer entries than rows")
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _device_tensor(out, "out", torch.int32, 1)
    _require(out.shape[0] >= n, "out is too short")
    if token_slots is not None:
        _device_tensor(token_slots, "token_slots", torch.int32, 1)
        _device_tensor(slot_of_row, "slot_of_row", torch.int32, 1)
        _require(slot_of_row.shape[0] >= n, "slot_of_row has fewer entries than rows")
    check(library().mllm_sample(_ptr(logits), n, vocab, _ptr(temperatures), _ptr(top_ps), _ptr(seeds), _ptr(steps), _ptr(out), _ptr(token_slots), _ptr(slot_of_row if token_slots is not None else None), _stream()))
    return out


def best_per_row(rows: int, weight, dtype) -> int:
    """How many (value, column) pairs a row ``linear_best`` leaves for so many rows with this weight; 0 where it has no
    kernel for the sizes."""
    _, _, n, k = _matrix(weight, "weight", dtype)
    return int(library().mllm_gemm_best_per_row(int(rows), n, k, _code(dtype)))


def linear_best(x, weight, bias=None):
    """x @ weight.T (+ bias) without writing the sums: (values float32 [rows, c], indices int32 [rows, c]), for every row
    the best (sum, column) of c disjoint sets of columns that together are all columns. The best pair of a row by
    numpy's argmax rules (``choose``) is the row's argmax. For the head of a step that decodes greedily."""
    _device_tensor(x, "x", dim=2)
    m, k = x.shape
    w_ptr, w_packed, n, w_cols = _matrix(weight, "weight", x.dtype)
    if not (w_cols == k):
        raise OperandError(f"x has {k} columns but weight has {w_cols}")
    if bias is not None:
        _device_tensor(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == n, "bias does not match weight")
    per_row = int(library().mllm_gemm_best_per_row(m, n, k, _code(x.dtype)))
    _require(per_row > 0, f"no kernel leaves the best columns of a product with K = {k}")
    values = torch.empty((m, per_row), dtype=torch.float32, device=x.device)
    indices = torch.empty((m, per_row), dtype=torch.int32, device=x.device)
    check(library().mllm_gemm_best(_ptr(x), w_ptr, w_packed, _ptr(bias), _ptr(values), _ptr(indices), per_row, m, n, k, _code(x.dtype), _stream()))
    return values, indices


@dataclass
class StepAdvance:
    """What ``choose`` moves on by one token for every live row, so that the same requests' next step finds its batch on
    the device: positions and stored lengths, the source of each row's token (its own last-token slot from then on), and
    per cache group the row a token's key and value go to, looked up in the group's block table ([rows, table_width],
    int32; pages of ``page_size`` tokens). ``draw_counts`` (optional, int32 [rows]): how many tokens each row's request has
    drawn so far, which a sampler's random numbers are a function of; grows by one too."""

    positions: torch.Tensor
    context_lens: torch.Tensor
    token_sources: torch.Tensor
    block_tables: list
    slots: list
    page_size: int
    draw_counts: torch.Tensor | None = None


def choose_flags(rows: int) -> int:
    """How many of a ring row's last entries ``choose`` sets to the step's number for a batch of so many rows (one for
    every 16 rows: a block of the kernel)."""
    return -(-int(rows) // 16)


def choose(values, indices, state_slots, token_slots, out=None, host_ring=None, cursor=None, advance: StepAdvance | None = None):
    """One token per row from its candidates: the best (value, index) pair by numpy's argmax rules (``values`` None: the
    smallest index; one candidate a row: that one). Rows whose ``state_slots`` entry is negative are padding and give -1. The
    token of a live row also goes to token_slots[state_slots[row]] and, with ``host_ring`` (int32 [ring rows, >= rows +
    ``choose_flags(rows)``] in page-locked host memory) to the ring row that ``cursor[0]`` names (``cursor``: int32 [3] on
    the device, its third entry zero); the row's last ``choose_flags(rows)`` entries then get the step's number
    ``cursor[1]`` (one from each block of the kernel), and row and number move on by one (the row modulo the ring's
    rows, the number modulo 2^30): a reader on the host that knows the number waits for it to appear in all of them,
    and needs no event.
    ``advance``: see StepAdvance. Returns the tokens (int32 [rows], on the device)."""
    _device_tensor(indices, "indices", torch.int32, 2)
    rows, per_row = indices.shape
    _require(per_row >= 1, "a row needs at least one candidate")
    if values is not None:
        _device_tensor(values, "values", torch.float32, 2)
        _require(values.shape == indices.shape, "values and indices differ in shape")
    _device_tensor(state_slots, "state_slots", torch.int32, 1)
    _require(state_slots.shape[0] >= rows, "state_slots has fewer entries than rows")
    _device_tensor(token_slots, "token_slots", torch.int32, 1)
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=indices.device)
    _device_tensor(out, "out", torch.int32, 1)
    _require(out.shape[0] >= rows, "out is too short")
    ring_rows = ring_stride = 0
    if host_ring is not None:
        _require(isinstance(host_ring, torch.Tensor) and host_ring.dtype == torch.int32 and host_ring.dim() == 2 and host_ring.is_contiguous()
                 and host_ring.is_pinned(), "the ring must be a contiguous int32 matrix in page-locked host memory")
        ring_rows, ring_stride = host_ring.shape
        _require(ring_stride >= rows + choose_flags(rows), "the ring's rows need an entry per row of the batch and choose_flags(rows) for the step's number")
        _device_tensor(cursor, "cursor", torch.int32, 1)
        _require(cursor.shape[0] == 3, "the cursor is (ring row, step number, blocks that are through)")
    else:
        _require(cursor is None, "a cursor without a ring")
    tables = slots = None
    n_groups = table_width = page_size = 0
    positions = context_lens = sources = draws = None
    if advance is not None:
        positions, context_lens, sources, draws = advance.positions, advance.context_lens, advance.token_sources, advance.draw_counts
        for t, name in ((positions, "positions"), (context_lens, "context_lens"), (sources, "token_sources")) + (((draws, "draw_counts"),) if draws is not None else ()):
            _device_tensor(t, name, torch.int32, 1)
            _require(t.shape[0] >= rows, f"{name} has fewer entries than rows")
        n_groups, page_size = len(advance.block_tables), int(advance.page_size)
        _require(len(advance.slots) == n_groups and n_groups <= 4, "one row of slots per block table, at most four groups")
        import ctypes

        for g, (table, slot) in enumerate(zip(advance.block_tables, advance.slots)):
            _device_tensor(table, f"block table {g}", torch.int32, 2)
            _device_tensor(slot, f"slots {g}", torch.int32, 1)
            _require(table.shape[0] >= rows and slot.shape[0] >= rows, f"group {g} has fewer rows than the batch")
            _require(g == 0 or table.shape[1] == advance.block_tables[0].shape[1], "the groups' block tables differ in width")
        table_width = advance.block_tables[0].shape[1] if n_groups else 0
        tables = (ctypes.c_void_p * max(n_groups, 1))(*[t.data_ptr() for t in advance.block_tables])
        slots = (ctypes.c_void_p * max(n_groups, 1))(*[t.data_ptr() for t in advance.slots])
    check(library().mllm_choose(_ptr(values), _ptr(indices), per_row, rows, _ptr(state_slots), _ptr(token_slots), _ptr(out),
                                _ptr(host_ring), ring_rows, ring_stride, _ptr(cursor), int(advance is not None), _ptr(positions), _ptr(context_lens),
                                _ptr(sources), _ptr(draws), tables, slots, n_groups, table_width, page_size, _stream()))
    return out


# -- a whole layer for rows that bring one token each -------------------------------------------------
@dataclass
class PendingRows:
    """Rows of the residual stream whose last sums are not taken yet:
    base + bias + partials[0] + partials[1] + ... The layer kernels for decoding leave their
    output products cut into such partial rows and take them up again in the next kernel."""

    base: torch.Tensor             # [rows, width] float32
    partials: torch.Tensor | None  # [n, rows, width] float32
    bias: torch.Tensor | None      # [width] float32

    @property
    def shape(self):
        return self.base.shape


MLP_SLICE_UNITS = 64         # hidden units a block of the feed-forward kernel takes
LAYER_KERNEL_MAX_ROWS = 64   # more rows than this go through the separate kernels


# The longest sequence that the two layer kernels decode, for up to four rows and for more: a block of the attention half
# walks all keys of its (row, head) alone, which past some 1,000 keys takes longer than the kernels it saves, the kernel
# that spreads a row's keys over many blocks among them. Measured in steps of 12 layers at GPT-2 small's sizes, layer
# kernels against separate kernels: 1 row 383 : 390 us at 500 keys, 459 : 442 at 1,200, 569 : 490 at 2,000; 8 rows
# 396 : 439, 455 : 487, 571 : 539, and 817 : 665 at 3,800; 16 rows 413 : 468 at 500, 613 : 612 at 2,000. (The feed-forward
# half changes with the attention half: alone beside the separate attention kernels it is 15 us a step behind them.)
DECODE_LAYER_REACHES = (1024, 1792)


def decode_layer_reach(rows: int) -> int:
    return DECODE_LAYER_REACHES[0] if rows <= 4 else DECODE_LAYER_REACHES[1]


_layer_kernel_rows: dict = {}


def layer_kernel_rows(width: int) -> int:
    """Rows up to which the layer kernels for decoding beat the separate kernels at this width: the
    library's own answer (mllm_decode_layer_rows, where the measurements behind it are written down)."""
    if width not in _layer_kernel_rows:
        rows = int(library().mllm_decode_layer_rows(int(width)))
        _layer_kernel_rows[width] = max(0, min(rows, LAYER_KERNEL_MAX_ROWS))
    return _layer_kernel_rows[width]


def launch_counts() -> dict:
    """kind of kernel -> how often this process has launched it so far (a launch recorded into a graph counts once, at its
    capture; replays do not count). The difference of two calls tells which kernels the work between them took, as the
    reference's launch counter does for its tests (engine/include/cuda_check.h:21-41)."""
    lib = library()
    return {lib.mllm_kernel_name(kind).decode(): int(lib.mllm_launch_count(kind)) for kind in range(lib.mllm_kernel_kinds())}


def launches_since(before: dict) -> dict:
    """The launches since ``before`` (an earlier ``launch_counts()``), kinds that were not launched left out."""
    now = launch_counts()
    return {name: now[name] - before.get(name, 0) for name in now if now[name] != before.get(name, 0)}


def _pending(hidden):
    if isinstance(hidden, PendingRows):
        base, partials, bias = hidden.base, hidden.partials, hidden.bias
    else:
        base, partials, bias = hidden, None, None
    _device_tensor(base, "the stream's rows", torch.float32, 2)
    rows, width = base.shape
    if partials is not None:
        _device_tensor(partials, "the partial rows", torch.float32, 3)
        _require(tuple(partials.shape[1:]) == (rows, width), "the partial rows do not match the stream")
    if bias is not None:
        _device_tensor(bias, "the pending bias", torch.float32, 1)
        _require(bias.shape[0] == width, "the pending bias does not match the stream")
    return base, partials, bias, 0 if partials is None else partials.shape[0]


def settle(hidden):
    """The stream as plain float32 rows: a tensor as it is, pending rows with their sums taken."""
    if not isinstance(hidden, PendingRows):
        return hidden
    base, partials, bias, n_partials = _pending(hidden)
    if n_partials == 0 and bias is None:
        return base
    out = torch.empty_like(base)
    check(library().mllm_pending_sum(_ptr(base), _ptr(partials), _ptr(bias), n_partials, _ptr(out), base.shape[0], base.shape[1], _stream()))
    return out


def decode_layer_supported(width, head_size=0, page_size=0, inner=0) -> bool:
    """Whether the layer kernels for decoding take these sizes (0: that size is not asked about)."""
    return bool(library().mllm_decode_layer_supported(int(width), int(head_size), int(page_size), int(inner)))


def _norm_vectors(gamma, beta, width):
    _device_tensor(gamma, "gamma", torch.float32, 1)
    _device_tensor(beta, "beta", torch.float32, 1)
    _require(gamma.shape[0] == width and beta.shape[0] == width, "the norm's vectors do not match the width")


def decode_attention_half(hidden, gamma, beta, eps, w_qkv, b_qkv, w_out, b_out, k_pages, v_pages, slots, token_request,
                          positions, block_tables, n_heads, n_kv_heads, head_size, scale, window=0, write_cache=True):
    """norm, q/k/v, cache write, attention and output product of a pre-norm layer's first half, for
    rows that are each the newest token of their request, in one kernel (bfloat16 only; the two
    matrices as PackedMatrix).

    ``hidden``: float32 rows or PendingRows. Returns PendingRows: the stream before this half
    with its sums taken, one partial row per head, and the output product's bias."""
    base, partials, bias, n_partials = _pending(hidden)
    rows, width = base.shape
    _norm_vectors(gamma, beta, width)
    num_pages, page_size = _check_pages(k_pages, v_pages, n_kv_heads, head_size)
    _require(k_pages.dtype == torch.bfloat16, "the layer kernels for decoding are bfloat16 only")
    if not (decode_layer_supported(width, head_size, page_size)):
        raise OperandError(f"no layer kernel for width {width}, head size {head_size}, pages of {page_size}")
    q_width, kv_width = n_heads * head_size, n_kv_heads * head_size
    for w, name in ((w_qkv, "w_qkv"), (w_out, "w_out")):
        if not (isinstance(w, PackedMatrix)):
            raise OperandError(f"{name} must be a PackedMatrix")
        _device_tensor(w.data, name, torch.bfloat16, 1)
    _require(w_qkv.shape == (q_width + 2 * kv_width, width), "w_qkv does not match the heads or the width")
    _require(w_out.shape == (width, q_width), "w_out does not match the heads or the width")
    for t, name, n in ((b_qkv, "b_qkv", q_width + 2 * kv_width), (b_out, "b_out", width)):
        if t is not None:
            _device_tensor(t, name, torch.float32, 1)
            if not (t.shape[0] == n):
                raise OperandError(f"{name} does not match its matrix")
    for t, name in ((slots, "slots"), (token_request, "token_request"), (positions, "positions")):
        _device_tensor(t, name, torch.int32, 1)
        if not (t.shape[0] >= rows):
            raise OperandError(f"{name} has fewer entries than rows")
    _device_tensor(block_tables, "block_tables", torch.int32, 2)
    summed = torch.empty_like(base)
    out = torch.empty((n_heads, rows, width), dtype=torch.float32, device=base.device)
    check(library().mllm_decode_attention_half(
        _ptr(base), _ptr(partials), _ptr(bias), n_partials, _ptr(summed), _ptr(gamma), _ptr(beta), float(eps), _ptr(w_qkv.data),
        _ptr(b_qkv), _ptr(w_out.data), _ptr(k_pages), _ptr(v_pages), _ptr(slots), _ptr(token_request), _ptr(positions),
        _ptr(block_tables), block_tables.shape[1], _ptr(out), rows, width, n_heads, n_kv_heads, head_size, page_size,
        int(window), float(scale), int(bool(write_cache)), _stream()))
    return PendingRows(summed, out, b_out)


def decode_mlp_half(hidden, gamma, beta, eps, w_up, b_up, w_down, b_down, activation=None, slice_units=MLP_SLICE_UNITS):
    """norm, up product, activation and down product of a pre-norm layer's second half in one
    kernel (bfloat16 matrices as PackedMatrix). Returns PendingRows: the stream before this half with its sums
    taken, one partial row per slice of ``slice_units`` hidden units, and the down product's bias."""
    base, partials, bias, n_partials = _pending(hidden)
    rows, width = base.shape
    _norm_vectors(gamma, beta, width)
    if not (activation in EPILOGUES):
        raise OperandError(f"unknown activation {activation!r}")
    for w, name in ((w_up, "w_up"), (w_down, "w_down")):
        if not (isinstance(w, PackedMatrix)):
            raise OperandError(f"{name} must be a PackedMatrix")
        _device_tensor(w.data, name, torch.bfloat16, 1)
    inner = w_up.rows
    if not (decode_layer_supported(width, inner=inner)):
        raise OperandError(f"no layer kernel for width {width} with {inner} hidden units")
    _require(w_up.shape == (inner, width) and w_down.shape == (width, inner), "the two matrices do not match the width")
    for t, name, n in ((b_up, "b_up", inner), (b_down, "b_down", width)):
        if t is not None:
            _device_tensor(t, name, torch.float32, 1)
            if not (t.shape[0] == n):
                raise OperandError(f"{name} does not match its matrix")
    _require(slice_units in (64, 128), "slices of 64 or 128 hidden units")
    summed = torch.empty_like(base)
    out = torch.empty(((inner + slice_units - 1) // slice_units, rows, width), dtype=torch.float32, device=base.device)
    check(library().mllm_decode_mlp_half(
        _ptr(base), _ptr(partials), _ptr(bias), n_partials, _ptr(summed), _ptr(gamma), _ptr(beta), float(eps), _ptr(w_up.data),
        _ptr(b_up), _ptr(w_down.data), _ptr(out), rows, width, inner, slice_units, EPILOGUES[activation], _stream()))
    return PendingRows(summed, out, b_down)
