"""Each kernel alone against a plain float64 reference, at sizes other than the engine's: odd
row counts, widths and vocabularies that are no power of two, head sizes in steps of 16."""

import math

import numpy as np
import pytest
import torch

import plain_gpt2 as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def K():
    from mini_llm_amd.ops import kernels

    return kernels


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a)).to(DEV).to(dtype).contiguous()


def host(t):
    return t.detach().float().cpu().double().numpy()


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).bfloat16().float().double().numpy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,vocab,npos", [(1, 64, 50, 8), (7, 96, 1000, 64), (33, 777, 513, 40)])
def test_embed(K, dtype, rows, width, vocab, npos):
    rng = np.random.default_rng(0)
    wte, wpe = rng.standard_normal((vocab, width)), rng.standard_normal((npos, width))
    tok = rng.integers(0, vocab, rows)
    pos = rng.integers(0, npos, rows)
    if rows > 2:
        tok[1] = -1  # a padding row
    out = K.embed(dev(tok, torch.int32), dev(pos, torch.int32), dev(wte, dtype), dev(wpe, dtype))
    a, b = (wte, wpe) if dtype == torch.float32 else (bf16_round(wte), bf16_round(wpe))
    ref = a[np.maximum(tok, 0)].astype(np.float32) + b[pos].astype(np.float32)
    ref[tok < 0] = 0
    np.testing.assert_allclose(host(out), ref, rtol=0, atol=1e-6)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,eps", [(1, 64, 1e-5), (5, 96, 1e-6), (9, 768, 1e-5), (3, 1030, 1e-3), (2, 2500, 1e-5),
                                            (4, 320, 1e-5), (70, 1600, 1e-5), (2, 4096, 1e-5), (2, 4100, 1e-5), (3, 6, 1e-5), (300, 1024, 1e-5)])
def test_layernorm(K, out_dtype, rows, width, eps):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((rows, width)) * 2 + 50).astype(np.float32)  # a large mean
    g, b = rng.standard_normal(width).astype(np.float32), rng.standard_normal(width).astype(np.float32)
    out = K.layernorm(dev(x), dev(g), dev(b), eps, out_dtype=out_dtype)
    ref = P.layernorm(x.astype(np.float64), g, b, eps)
    tol = 2e-5 if out_dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(host(out), ref, rtol=tol, atol=tol)
    if rows > 2:  # rows chosen by index
        idx = np.array([rows - 1, 0, rows - 1])
        out = K.layernorm(dev(x), dev(g), dev(b), eps, out_dtype=out_dtype, row_index=dev(idx, torch.int32))
        np.testing.assert_allclose(host(out), ref[idx], rtol=tol, atol=tol)


def test_layernorm_constant_row_gives_beta(K):
    b = np.linspace(-1, 1, 96).astype(np.float32)
    out = K.layernorm(dev(np.full((2, 96), 7.0)), dev(np.ones(96)), dev(b), 1e-5)
    np.testing.assert_allclose(host(out), np.stack([b, b]), atol=1e-6)


def as_weight(K, w, dtype, packed):
    """A weight on the device, row-major or in the packed layout of the matrix kernels."""
    return K.pack_matrix(dev(w, dtype)) if packed else dev(w, dtype)


def plain_packed(w, vec):
    """The packed layout of a matrix, written out element by element: chunks of 16 rows x 4*vec
    columns, row tiles outermost; piece p of a chunk is row p % 16, columns (p // 16) * vec .."""
    rows, cols = w.shape
    kc = 4 * vec
    row_tiles, k_steps = -(-rows // 16), -(-cols // kc)
    padded = np.zeros((row_tiles * 16, k_steps * kc), dtype=w.dtype)
    padded[:rows, :cols] = w
    out = np.zeros((row_tiles, k_steps, 64, vec), dtype=w.dtype)
    for p in range(64):
        out[:, :, p, :] = padded.reshape(row_tiles, 16, k_steps, kc)[:, p % 16, :, (p // 16) * vec : (p // 16 + 1) * vec]
    return out.reshape(-1)


def unpacked(packed_rows):
    """The [rows, cols] matrix that a PackedMatrix / PackedRows holds (the inverse of plain_packed)."""
    rows, cols = packed_rows.shape
    vec = 16 // packed_rows.data.element_size()
    kc = 4 * vec
    row_tiles, k_steps = -(-rows // 16), -(-cols // kc)
    flat = host(packed_rows.data.float()).reshape(row_tiles, k_steps, 64, vec)
    out = np.zeros((row_tiles * 16, k_steps * kc))
    for p in range(64):
        out.reshape(row_tiles, 16, k_steps, kc)[:, p % 16, :, (p // 16) * vec : (p // 16 + 1) * vec] = flat[:, :, p, :]
    return out[:rows, :cols]


def packed_rows_of(K, x, dtype):
    """Activations as a kernel would leave them in the packed layout (NaN where nothing is defined)."""
    rows = K.empty_packed_rows(x.shape[0], x.shape[1], dtype, DEV)
    rows.data.fill_(float("nan"))
    vec = 16 // rows.data.element_size()
    flat = plain_packed(np.asarray(x, dtype=np.float64), vec)
    mask = plain_packed(np.ones_like(np.asarray(x, dtype=np.float64)), vec) > 0
    values = torch.tensor(flat, dtype=torch.float64, device=DEV).to(dtype)
    rows.data[torch.tensor(mask, device=DEV)] = values[torch.tensor(mask, device=DEV)]
    return rows


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,n_partials", [(1, 64, 0), (17, 200, 3), (64, 768, 2), (33, 100, 0), (40, 1600, 0), (20, 1024, 2)])
def test_layernorm_leaves_packed_rows(K, dtype, rows, width, n_partials):
    rng = np.random.default_rng(rows + width)
    gamma, beta = 1 + 0.1 * rng.standard_normal(width), 0.1 * rng.standard_normal(width)
    hidden, total = _pending_rows(K, rng, rows, width, n_partials, n_partials > 0)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    out, summed = K.layernorm(hidden, dev(gamma), dev(beta), 2e-5, out_dtype=dtype, with_sums=True, packed_out=True)
    assert isinstance(out, K.PackedRows) and out.shape == (rows, width)
    np.testing.assert_allclose(unpacked(out), P.layernorm(total, gamma, beta, 2e-5), rtol=tol, atol=tol)
    np.testing.assert_allclose(host(summed), total, rtol=1e-6, atol=1e-6)
    out = K.layernorm(dev(total), dev(gamma), dev(beta), 2e-5, out_dtype=dtype, packed_out=True)
    np.testing.assert_allclose(unpacked(out), P.layernorm(total, gamma, beta, 2e-5), rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (17, 288, 320), (33, 1000, 96), (64, 192, 200), (48, 130, 1000)])
def test_products_of_few_rows_read_and_write_packed_rows(K, dtype, m, n, k):
    # x in the packed layout with NaN wherever nothing is defined (rows and columns beyond the
    # matrix): the product must not use those; the output in the packed layout on request
    rng = np.random.default_rng(m + n)
    rounded = bf16_round if dtype == torch.bfloat16 else (lambda a: a.astype(np.float32).astype(np.float64))
    x, w, b = rng.standard_normal((m, k)), rng.standard_normal((n, k)) / math.sqrt(k), rng.standard_normal(n)
    weight = as_weight(K, w, dtype, True)
    assert K.takes_packed_rows(m, weight, dtype)
    xp = packed_rows_of(K, rounded(x), dtype)
    np.testing.assert_allclose(unpacked(xp), rounded(x), rtol=0, atol=0)
    ref = rounded(x) @ rounded(w).T + b.astype(np.float32)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    out = K.linear(xp, weight, dev(b), out_dtype=torch.float32)
    np.testing.assert_allclose(host(out), ref, rtol=2e-5, atol=2e-5)
    out = K.linear(xp, weight, dev(b), activation="gelu_new", packed_out=True)
    assert isinstance(out, K.PackedRows) and out.dtype == dtype
    np.testing.assert_allclose(unpacked(out), P.gelu_new(ref), rtol=tol, atol=tol)
    res = rng.standard_normal((m, n)).astype(np.float32)
    out = K.linear(xp, weight, dev(b), residual=dev(res))
    np.testing.assert_allclose(host(out), ref + res, rtol=2e-5, atol=2e-5)
    partials = K.linear_split(xp, weight, 3)
    np.testing.assert_allclose(host(partials).astype(np.float64).sum(axis=0), rounded(x) @ rounded(w).T, rtol=2e-5, atol=2e-5)


def test_packed_rows_are_refused_where_the_kernel_for_few_rows_does_not_run(K):
    from mini_llm_amd.ops.library import KernelLibraryError

    w = torch.zeros((64, 64), device=DEV)
    assert not K.takes_packed_rows(65, w, torch.float32) and K.takes_packed_rows(64, w, torch.float32)
    assert not K.takes_packed_rows(8, torch.zeros((9000, 64), device=DEV, dtype=torch.bfloat16), torch.bfloat16)   # the wide head
    with pytest.raises(KernelLibraryError, match="few rows"):
        K.linear(K.empty_packed_rows(65, 64, torch.float32, DEV), w)
    with pytest.raises(KernelLibraryError, match="few rows"):
        K.linear(torch.zeros((65, 64), device=DEV), w, packed_out=True)
    with pytest.raises(KernelLibraryError, match="64 rows"):
        K.linear_split(K.empty_packed_rows(65, 64, torch.float32, DEV), w, 2)


@pytest.mark.parametrize("rows,cols", [(1, 1), (16, 32), (33, 65), (96, 288), (50, 777)])
@pytest.mark.parametrize("src,dst", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32)])
@pytest.mark.parametrize("transpose", [False, True])
def test_pack_matrix(K, rows, cols, src, dst, transpose):
    rng = np.random.default_rng(rows * 7 + cols)
    w = bf16_round(rng.standard_normal((rows, cols)))  # exact in every element type here
    stored = w.T if transpose else w
    packed = K.pack_matrix(dev(np.ascontiguousarray(stored), src), dst, transpose=transpose)
    assert packed.shape == (rows, cols) and packed.dtype == dst
    np.testing.assert_array_equal(host(packed.data), plain_packed(w, 4 if dst == torch.float32 else 8))


GEMM_SHAPES = [(1, 64, 64), (3, 100, 96), (17, 288, 320), (33, 1000, 96), (64, 192, 200), (65, 130, 72),
               (130, 257, 136), (200, 777, 240), (257, 96, 1024), (5, 50, 36), (40, 33, 20),
               (2100, 2010, 104), (4100, 2010, 40),  # many rows and columns: the large tile (256 x 128; in 32-bit from 256 tiles on), ragged edges
               # K in whole tiles of 64, columns in whole pieces, 65 rows or more: in bfloat16 with a packed matrix the kernel that
               # streams its operands into LDS: tiles of 128 x 64 (with two waves sharing each 64 x 64 along K from a K of 1,536 on:
               # here with an odd count of tiles), 128 x 192, 128 x 128, 256 x 128 and 256 x 256 (the last shape: 200 tiles in one
               # round of blocks, ragged on both sides), chosen by the rounds of blocks they need
               (300, 136, 192), (193, 2008, 128), (2100, 264, 64), (700, 776, 320), (300, 72, 1600), (2100, 2008, 128), (192, 8, 64),
               (1000, 2312, 128), (2040, 4088, 64), (70, 136, 128), (130, 264, 64), (2000, 6392, 192)]


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
@pytest.mark.parametrize("activation", [None, "gelu_new", "gelu"])
def test_linear_f32(K, m, n, k, activation, packed):
    rng = np.random.default_rng(m * 1000 + n)
    x, w, b = rng.standard_normal((m, k)), rng.standard_normal((n, k)) / math.sqrt(k), rng.standard_normal(n)
    res = rng.standard_normal((m, n))
    y = x.astype(np.float32).astype(np.float64) @ w.astype(np.float32).astype(np.float64).T + b.astype(np.float32)
    if activation:
        y = P.ACTIVATIONS[activation](y)
    weight = as_weight(K, w, torch.float32, packed)
    out = K.linear(dev(x), weight, dev(b), activation=activation)
    np.testing.assert_allclose(host(out), y, rtol=1e-5, atol=1e-5)
    out = K.linear(dev(x), weight, dev(b), activation=activation, residual=dev(res))
    np.testing.assert_allclose(host(out), y + res.astype(np.float32), rtol=1e-5, atol=1e-5)
    out = K.linear(dev(x), weight)
    np.testing.assert_allclose(host(out), x.astype(np.float32).astype(np.float64) @ w.astype(np.float32).astype(np.float64).T, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("rows", [40, 49, 64])
def test_few_rows_over_a_large_matrix(K, rows):
    # 40 to 64 rows over a matrix of 6 M elements (33-48 rows: three row tiles of x where the kernel
    # holds four), plain and with the q/k/v epilogue that writes the cache
    rng = np.random.default_rng(rows)
    n, k = 2512, 2400
    x, w, b = rng.standard_normal((rows, k)), rng.standard_normal((n, k)) / math.sqrt(k), rng.standard_normal(n)
    ref = bf16_round(x) @ bf16_round(w).T + b.astype(np.float32)
    weight = as_weight(K, w, torch.bfloat16, True)
    out = K.linear(dev(x, torch.bfloat16), weight, dev(b), out_dtype=torch.float32)
    np.testing.assert_allclose(host(out), ref, rtol=2e-5, atol=2e-5)
    n_heads, head_size, page_size = 13, 64, 64           # 3 x 832 = 2,496 columns
    w = w[: 3 * n_heads * head_size]
    kp = torch.full((3, n_heads, page_size, head_size), 7.0, device=DEV).to(torch.bfloat16)
    vp = torch.full_like(kp, 7.0)
    slots = rng.permutation(3 * page_size)[:rows].astype(np.int32)
    q = K.linear_qkv_cache(dev(x, torch.bfloat16), as_weight(K, w, torch.bfloat16, True), dev(b[: len(w)]), kp, vp,
                           dev(slots, torch.int32), n_heads, n_heads, head_size)
    width = n_heads * head_size
    np.testing.assert_allclose(host(q), ref[:, :width], rtol=2e-2, atol=2e-2)
    for r, slot in enumerate(slots):
        np.testing.assert_allclose(host(kp[slot // page_size, :, slot % page_size]).reshape(-1), ref[r, width : 2 * width], rtol=2e-2, atol=2e-2)
        np.testing.assert_allclose(host(vp[slot // page_size, :, slot % page_size]).reshape(-1), ref[r, 2 * width : 3 * width], rtol=2e-2, atol=2e-2)


def test_linear_f32_is_true_32_bit(K):
    # values that a reduced-precision matrix mode (tf32/bf16 inputs) would round away
    m, n, k = 8, 64, 64
    x = np.full((m, k), 1.0 + 2.0**-12, dtype=np.float32)  # 12 fraction bits: tf32 keeps 10, bf16 7
    w = np.ones((n, k), dtype=np.float32)
    out = host(K.linear(dev(x), dev(w)))
    assert (out == k * (1.0 + 2.0**-12)).all()  # exact in float32; a reduced mode gives 64.0


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_linear_bf16(K, m, n, k, out_dtype, packed):
    rng = np.random.default_rng(m * 1000 + n + 1)
    x, w, b = rng.standard_normal((m, k)), rng.standard_normal((n, k)) / math.sqrt(k), rng.standard_normal(n)
    y = bf16_round(x) @ bf16_round(w).T + b.astype(np.float32)
    weight = as_weight(K, w, torch.bfloat16, packed)
    out = K.linear(dev(x, torch.bfloat16), weight, dev(b), activation="gelu_new", out_dtype=out_dtype)
    tol = 1e-2 if out_dtype == torch.bfloat16 else 2e-5
    np.testing.assert_allclose(host(out), P.gelu_new(y), rtol=tol, atol=tol)
    if out_dtype == torch.float32:
        res = rng.standard_normal((m, n)).astype(np.float32)
        out = K.linear(dev(x, torch.bfloat16), weight, dev(b), residual=dev(res))
        np.testing.assert_allclose(host(out), y + res, rtol=2e-5, atol=2e-5)


def guarded(values, dtype, fill=float("nan")):
    """The values on the device with 64 elements of ``fill`` right behind them (the pattern of the
    reference's kernel tests: engine/tests/test_matvec_batch.cu:21-22): (view of the values, the guard)."""
    values = np.ascontiguousarray(values)
    whole = torch.full((values.size + 64,), fill, device=DEV, dtype=dtype)
    whole[: values.size] = dev(values, dtype).flatten()
    return whole[: values.size].view(*values.shape), whole[values.size :]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(5, 37, 20), (1, 16, 8), (16, 130, 72), (40, 50, 200), (64, 100, 64), (70, 37, 24), (130, 200, 96),
                                   (300, 260, 136), (33, 40, 21), (200, 70, 50), (3, 9000, 64), (300, 264, 128), (200, 72, 64), (1000, 2056, 64),
                                   (2050, 2056, 192), (1000, 2312, 128), (2040, 4088, 64), (300, 72, 1600), (70, 136, 128)])
def test_linear_reads_nothing_past_its_operands(K, dtype, m, n, k):
    # NaN guards right after every operand: an out-of-bounds read would poison the result; a known
    # value right after the output: nothing is written past it. Every kernel of the product: few
    # rows, the tiles, an unaligned K, the wide head.
    rng = np.random.default_rng(m + n + k)
    rounded = bf16_round if dtype == torch.bfloat16 else (lambda a: a.astype(np.float32).astype(np.float64))
    x, w, b = rng.standard_normal((m, k)), rng.standard_normal((n, k)) / math.sqrt(k), rng.standard_normal(n).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    xg, _ = guarded(x, dtype)
    wg, _ = guarded(w, dtype)
    bg, _ = guarded(b, torch.float32)
    rg, _ = guarded(res, torch.float32)
    og, after = guarded(np.zeros((m, n)), torch.float32, fill=123.0)
    K.linear(xg, wg, bg, residual=rg, out=og)
    np.testing.assert_allclose(host(og), rounded(x) @ rounded(w).T + b + res, rtol=2e-5, atol=2e-5)
    assert (after == 123.0).all()
    # the same with the matrix in the packed layout (its chunks hold zeros beyond the matrix, the rows of x do not)
    og, after = guarded(np.zeros((m, n)), torch.float32, fill=123.0)
    K.linear(xg, as_weight(K, w, dtype, True), bg, residual=rg, out=og)
    np.testing.assert_allclose(host(og), rounded(x) @ rounded(w).T + b + res, rtol=2e-5, atol=2e-5)
    assert (after == 123.0).all()
    if dtype == torch.bfloat16:
        ob, after = guarded(np.zeros((m, n)), torch.bfloat16, fill=123.0)
        K.linear(xg, as_weight(K, w, dtype, True), bg, out=ob)
        np.testing.assert_allclose(host(ob), rounded(x) @ rounded(w).T + b, rtol=1e-2, atol=1e-2)
        assert (after == 123.0).all()


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 64), (7, 100), (5, 768), (3, 1100), (2, 2500)])
def test_layernorm_reads_nothing_past_its_operands(K, out_dtype, rows, width):
    rng = np.random.default_rng(rows + width)
    x, gamma, beta = rng.standard_normal((rows, width)).astype(np.float32), rng.standard_normal(width).astype(np.float32), rng.standard_normal(width).astype(np.float32)
    xg, _ = guarded(x, torch.float32)
    gg, _ = guarded(gamma, torch.float32)
    bg, _ = guarded(beta, torch.float32)
    out = K.layernorm(xg, gg, bg, 1e-5, out_dtype=out_dtype)
    tol = 1e-5 if out_dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(host(out), P.layernorm(x.astype(np.float64), gamma, beta, 1e-5), rtol=tol, atol=tol)


def plain_paged_attention(q, k_all, v_all, n_heads, n_kv_heads, window):
    """Rows of q are the LAST len(q) positions of a sequence whose keys are k_all/v_all."""
    total, nq = k_all.shape[0], q.shape[0]
    qfull = np.zeros((total, q.shape[1]))
    qfull[total - nq :] = q
    out = P.multi_head_attention(qfull, k_all, v_all, n_heads, n_kv_heads, window)
    return out[total - nq :]


@pytest.mark.parametrize("path", ["general", "split_keys", "split_keys_balanced", "matrix_cores", "two_kinds"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "n_heads,n_kv_heads,head_size,page_size,window",
    [(4, 4, 16, 16, 0), (3, 3, 32, 64, 0), (5, 5, 48, 32, 0), (6, 2, 64, 16, 0), (2, 1, 80, 64, 0),
     (2, 2, 128, 64, 0), (4, 2, 32, 16, 37), (1, 1, 256, 16, 0), (12, 12, 64, 64, 0), (2, 2, 64, 128, 100)],
)
def test_paged_attention(K, path, dtype, n_heads, n_kv_heads, head_size, page_size, window):
    # general: a wave per (token, head). split_keys: the decode kernel (forced for every row by
    # promising short portions; it treats rows independently, so the promise costs only speed),
    # with the splits laid over the tables' whole reach or balanced over the longest sequence.
    # matrix_cores: the prefill kernel, a block per tile of one request's queries. two_kinds: short
    # portions first, which take the decode kernel, then long ones, which take the prefill kernel
    # (two launches where both kernels take the head size, else one as before).
    if path.startswith("split") and head_size not in (16, 32, 64, 128, 256):
        pytest.skip("the split-key kernel takes power-of-two head sizes; others go the general way")
    if path == "matrix_cores" and head_size > 128:
        pytest.skip("the matrix-core kernel takes head sizes up to 128; larger go the general way")
    rng = np.random.default_rng(n_heads * 100 + head_size)
    # three requests: (cached context, new tokens); pages handed out in a scrambled order
    shapes = [(150, 1), (200, 1), (61, 5), (0, 70), (40, 9)] if path == "two_kinds" else [(0, 70), (150, 1), (61, 9)]
    num_pages = 40
    order = rng.permutation(num_pages).tolist()
    kp = torch.full((num_pages, n_kv_heads, page_size, head_size), float("nan"), device=DEV).to(dtype)
    vp = torch.full_like(kp, float("nan"))
    max_blocks = max((c + n + page_size - 1) // page_size for c, n in shapes)
    tables = np.zeros((len(shapes), max_blocks), dtype=np.int32)
    q_rows, treq, tpos, refs = [], [], [], []
    rnd = lambda *s: bf16_round(rng.standard_normal(s)) if dtype == torch.bfloat16 else rng.standard_normal(s).astype(np.float32).astype(np.float64)
    for r, (ctx, new) in enumerate(shapes):
        total = ctx + new
        k_all, v_all = rnd(total, n_kv_heads * head_size), rnd(total, n_kv_heads * head_size)
        q = rnd(new, n_heads * head_size)
        if (ctx, new) == (0, 70):  # one far key stands out for the last query: a missed tile would show
            far = q[-1].reshape(n_heads, head_size)[:: n_heads // n_kv_heads].reshape(-1) * 4
            k_all[3] = bf16_round(far) if dtype == torch.bfloat16 else far
        n_blocks = (total + page_size - 1) // page_size
        pages = [order.pop() for _ in range(n_blocks)]
        tables[r, :n_blocks] = pages
        slots = np.array([pages[p // page_size] * page_size + p % page_size for p in range(total)], dtype=np.int32)
        # context goes in with one call, the new tokens with another (as in a later step)
        for lo, hi in ((0, ctx), (ctx, total)):
            if hi > lo:
                K.cache_write(dev(k_all[lo:hi], dtype), dev(v_all[lo:hi], dtype), kp, vp, dev(slots[lo:hi], torch.int32), n_kv_heads, head_size)
        q_rows.append(q)
        treq += [r] * new
        tpos += list(range(ctx, total))
        refs.append(plain_paged_attention(q, k_all, v_all, n_heads, n_kv_heads, window or None))
    extra = {}
    if path in ("matrix_cores", "two_kinds"):
        starts = np.cumsum([0] + [new for _, new in shapes])
        extra = dict(q_starts=dev(starts, torch.int32), context_lens=dev([c for c, _ in shapes], torch.int32))
        if path == "two_kinds":
            extra.update(short_rows=7, short_requests=3)
    else:  # a padding row in the middle
        q_rows.insert(1, np.zeros((1, n_heads * head_size)))
        treq.insert(shapes[0][1], -1)
        tpos.insert(shapes[0][1], 0)
        refs.insert(1, np.zeros((1, n_heads * head_size)))
    out = K.paged_attention(
        dev(np.concatenate(q_rows), dtype), kp, vp, dev(treq, torch.int32), dev(tpos, torch.int32), dev(tables, torch.int32),
        n_heads, n_kv_heads, head_size, 1.0 / math.sqrt(head_size), window=window,
        max_q_len={"general": None, "matrix_cores": 70, "two_kinds": 70}.get(path, 1), max_len=151 if path == "split_keys_balanced" else None, **extra,
    )
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(host(out), np.concatenate(refs), rtol=tol, atol=tol)
    if path == "split_keys":  # the same rows in the packed layout, as the output product of few rows takes them
        packed = K.paged_attention(
            dev(np.concatenate(q_rows), dtype), kp, vp, dev(treq, torch.int32), dev(tpos, torch.int32), dev(tables, torch.int32),
            n_heads, n_kv_heads, head_size, 1.0 / math.sqrt(head_size), window=window, max_q_len=1, packed_out=True)
        assert isinstance(packed, K.PackedRows)
        np.testing.assert_array_equal(unpacked(packed), host(out.float()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_heads,head_size,page_size", [(3, 64, 64), (5, 48, 16), (2, 128, 32)])
def test_prompt_attention_passes_padding_requests_by(K, dtype, n_heads, head_size, page_size):
    # A batch laid out in a padded shape has requests that are nobody: a stored length of -1, a block table of -1, and
    # (one of them) rows that no request owns. The kernels that go request by request pass them by.
    rng = np.random.default_rng(head_size)
    rnd = lambda *s: bf16_round(rng.standard_normal(s)) if dtype == torch.bfloat16 else rng.standard_normal(s).astype(np.float32).astype(np.float64)
    shapes = [(40, 70), None, (0, 33), None]          # (stored, new) of the real requests; None: padding
    padding_rows = 6                                   # rows that the first padding request spans
    num_pages = 16
    kp = torch.full((num_pages, n_heads, page_size, head_size), float("nan"), device=DEV).to(dtype)
    vp = torch.full_like(kp, float("nan"))
    max_blocks = 8
    tables = np.full((len(shapes), max_blocks), -1, dtype=np.int32)
    order = rng.permutation(num_pages).tolist()
    q_rows, refs, starts, contexts, real_rows, at = [], [], [0], [], [], 0
    for r, shape in enumerate(shapes):
        if shape is None:
            rows = padding_rows if r == 1 else 0
            q_rows.append(np.zeros((rows, n_heads * head_size)))
            contexts.append(-1)
        else:
            ctx, new = shape
            total = ctx + new
            k_all, v_all, q = rnd(total, n_heads * head_size), rnd(total, n_heads * head_size), rnd(new, n_heads * head_size)
            pages = [order.pop() for _ in range((total + page_size - 1) // page_size)]
            tables[r, : len(pages)] = pages
            slots = np.array([pages[p // page_size] * page_size + p % page_size for p in range(total)], dtype=np.int32)
            K.cache_write(dev(k_all, dtype), dev(v_all, dtype), kp, vp, dev(slots, torch.int32), n_heads, head_size)
            q_rows.append(q)
            refs.append(plain_paged_attention(q, k_all, v_all, n_heads, n_heads, None))
            contexts.append(ctx)
            rows = new
            real_rows += list(range(at, at + rows))
        at += rows
        starts.append(at)
    treq = np.concatenate([np.full(len(q), r if shapes[r] is not None else -1) for r, q in enumerate(q_rows)])
    tpos = np.concatenate([np.arange(len(q)) + max(contexts[r], 0) for r, q in enumerate(q_rows)])
    out = K.paged_attention(
        dev(np.concatenate(q_rows), dtype), kp, vp, dev(treq, torch.int32), dev(tpos, torch.int32), dev(tables, torch.int32),
        n_heads, n_heads, head_size, 1.0 / math.sqrt(head_size), max_q_len=70, max_len=128,
        q_starts=dev(starts, torch.int32), context_lens=dev(contexts, torch.int32))
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(host(out)[real_rows], np.concatenate(refs), rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "n_heads,n_kv_heads,head_size,page_size,window,lengths,min_part",
    [(12, 12, 64, 64, 0, (1500,), None),                 # one token, 1,500 keys: two runs by the kernel's own rule
     (4, 2, 32, 16, 0, (700, 3, 260), 64),               # three tokens, one with 3 keys: most of its runs are empty
     (3, 3, 128, 32, 300, (900, 450), 32),               # a window: the runs cut the window, not the sequence
     (1, 1, 16, 16, 0, (1100, 1), 16),                   # a head of 16: a round of the sweep is 256 keys
     (5, 5, 256, 64, 0, (520,), 64)],
)
def test_decode_attention_with_the_keys_in_runs(K, monkeypatch, dtype, n_heads, n_kv_heads, head_size, page_size, window, lengths, min_part):
    # Few tokens with many keys: each token's keys are cut into runs, a block each, and the block of a (token, head) that
    # is through last puts the runs together (twice over: the counters it goes by must be zero again behind a launch).
    # One far key stands out in each sequence, in a run other than the last where there are several.
    if min_part is not None:
        monkeypatch.setattr(K, "DECODE_MIN_PART_FEW", min_part)
        monkeypatch.setattr(K, "DECODE_MIN_PART_BYTES", min_part * (2 if dtype == torch.bfloat16 else 4))
    rng = np.random.default_rng(head_size + len(lengths))
    rnd = lambda *s: bf16_round(rng.standard_normal(s)) if dtype == torch.bfloat16 else rng.standard_normal(s).astype(np.float32).astype(np.float64)
    n_blocks = [(n + page_size - 1) // page_size for n in lengths]
    order = rng.permutation(sum(n_blocks) + 3).tolist()
    kp = torch.full((len(order), n_kv_heads, page_size, head_size), float("nan"), device=DEV).to(dtype)
    vp = torch.full_like(kp, float("nan"))
    tables = np.zeros((len(lengths) + 1, max(n_blocks)), dtype=np.int32)
    q_rows, refs = [], []
    for r, total in enumerate(lengths):
        k_all, v_all = rnd(total, n_kv_heads * head_size), rnd(total, n_kv_heads * head_size)
        q = rnd(1, n_heads * head_size)
        stands_out = min(total - 1, max(0, total - 1 - (window - 5 if window else total - 2)))   # the second key, or one near the window's far edge
        far = q[0].reshape(n_heads, head_size)[:: n_heads // n_kv_heads].reshape(-1) * 3
        k_all[stands_out] = bf16_round(far) if dtype == torch.bfloat16 else far
        pages = [order.pop() for _ in range(n_blocks[r])]
        tables[r + 1, : len(pages)] = pages     # row 0 of the tables belongs to nobody
        slots = np.array([pages[p // page_size] * page_size + p % page_size for p in range(total)], dtype=np.int32)
        K.cache_write(dev(k_all, dtype), dev(v_all, dtype), kp, vp, dev(slots, torch.int32), n_kv_heads, head_size)
        q_rows.append(q)
        refs.append(plain_paged_attention(q, k_all, v_all, n_heads, n_kv_heads, window or None))
    # a padding row between the tokens
    q_rows.insert(1, np.zeros((1, n_heads * head_size)))
    refs.insert(1, np.zeros((1, n_heads * head_size)))
    treq = [1, -1] + list(range(2, len(lengths) + 1))
    tpos = [lengths[0] - 1, 0] + [n - 1 for n in lengths[1:]]
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for packed_out in (False, True):
        before = K.launch_counts()
        out = K.paged_attention(
            dev(np.concatenate(q_rows), dtype), kp, vp, dev(treq, torch.int32), dev(tpos, torch.int32), dev(tables, torch.int32),
            n_heads, n_kv_heads, head_size, 1.0 / math.sqrt(head_size), window=window, max_q_len=1, max_len=max(lengths), packed_out=packed_out)
        assert K.launches_since(before) == {"attention_decode": 1}
        np.testing.assert_allclose(unpacked(out) if packed_out else host(out), np.concatenate(refs), rtol=tol, atol=tol)
    assert (kp.device.index, kp.data_ptr()) in K._arrival_counters   # runs there were
    assert all((counters == 0).all() for counters in K._arrival_counters.values())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "n_heads,n_kv_heads,head_size,page_size,window",
    [(3, 3, 32, 16, 0), (2, 2, 64, 64, 0), (4, 2, 64, 16, 150), (2, 1, 128, 8, 0), (2, 2, 128, 256, 0), (3, 3, 32, 32, 70),
     (2, 2, 48, 32, 0), (5, 5, 64, 4, 0)],
)
@pytest.mark.parametrize("copies,reach", [(1, None), (12, None), (1, 100), (12, 100)])
def test_prompt_attention_over_long_portions(K, dtype, n_heads, n_kv_heads, head_size, page_size, window, copies, reach):
    # portions of several query tiles over several key tiles, requests of different lengths in one call (one
    # with a single token, one that starts at position 0, one whose portion ends one past a tile), pages
    # scrambled and unwritten places holding NaN. In the longest request some queries look hard at one far
    # key each (the first key, keys at the two sides of tile and page edges), so that a tile that is
    # skipped, read twice or read from a wrong page shows in those rows. Once as they are (few blocks: the
    # bfloat16 kernel takes 32 queries a block) and once twelve times over (64 queries a block); with the reach of the
    # longest sequence as the block tables give it (eight waves share a block's keys where heads are 64 or less) and
    # named short (four waves: the number only decides how a block's keys are shared out).
    rng = np.random.default_rng(head_size * 10 + page_size)
    shapes = [(0, 300), (200, 129), (500, 1), (70, 65), (0, 2)] * copies
    need = sum((c + n + page_size - 1) // page_size for c, n in shapes)
    num_pages = need + 5
    order = rng.permutation(num_pages).tolist()
    kp = torch.full((num_pages, n_kv_heads, page_size, head_size), float("nan"), device=DEV).to(dtype)
    vp = torch.full_like(kp, float("nan"))
    max_blocks = max((c + n + page_size - 1) // page_size for c, n in shapes)
    tables = np.zeros((len(shapes), max_blocks), dtype=np.int32)
    q_rows, treq, tpos, refs = [], [], [], []
    rnd = lambda *s: bf16_round(rng.standard_normal(s)) if dtype == torch.bfloat16 else rng.standard_normal(s).astype(np.float32).astype(np.float64)
    group = n_heads // n_kv_heads
    for r, (ctx, new) in enumerate(shapes):
        total = ctx + new
        k_all, v_all = rnd(total, n_kv_heads * head_size), rnd(total, n_kv_heads * head_size)
        q = rnd(new, n_heads * head_size)
        if (ctx, new) == (0, 300):
            for query, key in ((299, 0), (290, 63), (280, 64), (270, 127), (260, 128), (250, 191), (240, 192), (230, page_size - 1),
                               (220, page_size), (131, 129), (128, 128), (127, 1), (200, 200 - 69), (210, 255), (211, 256)):
                if window and query - key >= window:
                    continue
                far = q[query].reshape(n_heads, head_size)[::group].reshape(-1) * 4
                k_all[key] = bf16_round(far) if dtype == torch.bfloat16 else far
        n_blocks = (total + page_size - 1) // page_size
        pages = [order.pop() for _ in range(n_blocks)]
        tables[r, :n_blocks] = pages
        slots = np.array([pages[p // page_size] * page_size + p % page_size for p in range(total)], dtype=np.int32)
        K.cache_write(dev(k_all, dtype), dev(v_all, dtype), kp, vp, dev(slots, torch.int32), n_kv_heads, head_size)
        q_rows.append(q)
        treq += [r] * new
        tpos += list(range(ctx, total))
        refs.append(plain_paged_attention(q, k_all, v_all, n_heads, n_kv_heads, window or None))
    starts = np.cumsum([0] + [new for _, new in shapes])
    out = K.paged_attention(
        dev(np.concatenate(q_rows), dtype), kp, vp, dev(treq, torch.int32), dev(tpos, torch.int32), dev(tables, torch.int32),
        n_heads, n_kv_heads, head_size, 1.0 / math.sqrt(head_size), window=window, max_q_len=300, max_len=reach,
        q_starts=dev(starts, torch.int32), context_lens=dev([c for c, _ in shapes], torch.int32))
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(host(out), np.concatenate(refs), rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_over_a_block_table_of_more_than_a_thousand_pages(K, dtype):
    # 17,000 cached keys in pages of 16 (1,066 pages, scrambled): more than the 1,024 table entries
    # the prompt kernel keeps in LDS. A portion of 40 queries and a single decoded token; one far key
    # made to stand out for each, in the table's first and last hundred entries. The plain side is
    # written out for these rows only (softmax over the keys up to each row's position).
    n_heads, head_size, page_size, total = 2, 32, 16, 17000
    rng = np.random.default_rng(12)
    rnd = lambda *s: bf16_round(rng.standard_normal(s)) if dtype == torch.bfloat16 else rng.standard_normal(s).astype(np.float32).astype(np.float64)
    width = n_heads * head_size
    n_pages = (total + page_size - 1) // page_size
    assert n_pages > 1024
    pages = rng.permutation(n_pages + 7)[:n_pages]
    k_all, v_all = rnd(total, width), rnd(total, width)
    for new, path in ((40, "matrix_cores"), (1, "split_keys")):
        q = rnd(new, width)
        k_here = k_all.copy()
        for key in (37, total - new - 50):  # a hot key near each end of the table, for the last query
            k_here[key] = (bf16_round(q[-1] * 3) if dtype == torch.bfloat16 else q[-1] * 3)
        kp = torch.full((n_pages + 7, n_heads, page_size, head_size), float("nan"), device=DEV).to(dtype)
        vp = torch.full_like(kp, float("nan"))
        slots = np.array([pages[p // page_size] * page_size + p % page_size for p in range(total)], dtype=np.int32)
        K.cache_write(dev(k_here, dtype), dev(v_all, dtype), kp, vp, dev(slots, torch.int32), n_heads, head_size)
        ref = np.zeros((new, width))
        for i in range(new):
            position = total - new + i
            for h in range(n_heads):
                cols = slice(h * head_size, (h + 1) * head_size)
                scores = k_here[: position + 1, cols] @ q[i, cols] / math.sqrt(head_size)
                weights = np.exp(scores - scores.max())
                ref[i, cols] = (weights / weights.sum()) @ v_all[: position + 1, cols]
        extra = {}
        if path == "matrix_cores":
            extra = dict(q_starts=dev([0, new], torch.int32), context_lens=dev([total - new], torch.int32))
        out = K.paged_attention(
            dev(q, dtype), kp, vp, dev([0] * new, torch.int32), dev(list(range(total - new, total)), torch.int32),
            dev(pages[None, :].astype(np.int32), torch.int32), n_heads, n_heads, head_size, 1.0 / math.sqrt(head_size),
            max_q_len=new, **extra)
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        np.testing.assert_allclose(host(out), ref, rtol=tol, atol=tol, err_msg=path)


def test_paged_attention_strided_q(K):
    # q, k, v as column slices of one fused projection
    rng = np.random.default_rng(5)
    H, hs, ps, n = 3, 32, 16, 21
    qkv = rng.standard_normal((n, 3 * H * hs)).astype(np.float32)
    t = dev(qkv)
    kp = torch.zeros((4, H, ps, hs), device=DEV)
    vp = torch.zeros_like(kp)
    table = np.array([[2, 0, 3]], dtype=np.int32)
    slots = np.array([table[0, p // ps] * ps + p % ps for p in range(n)], dtype=np.int32)
    d = H * hs
    K.cache_write(t[:, d : 2 * d], t[:, 2 * d :], kp, vp, dev(slots, torch.int32), H, hs)
    out = K.paged_attention(t[:, :d], kp, vp, dev(np.zeros(n), torch.int32), dev(np.arange(n), torch.int32), dev(table, torch.int32), H, H, hs, 1 / math.sqrt(hs))
    ref = P.multi_head_attention(qkv[:, :d].astype(np.float64), qkv[:, d : 2 * d], qkv[:, 2 * d :], H)
    np.testing.assert_allclose(host(out), ref, rtol=2e-5, atol=2e-5)


def numpy_rule_argmax(row):
    nan = np.isnan(row)
    return int(np.argmax(nan)) if nan.any() else int(np.argmax(row))


@pytest.mark.parametrize("vocab", [1, 2, 63, 64, 65, 1000, 1024, 1025, 2049, 50257])
def test_argmax_rules(K, vocab):
    # engine/tests/test_argmax.cu:50-173 : ties, signed zero, -inf, NaN, borders of waves and blocks
    rng = np.random.default_rng(vocab)
    rows = [rng.standard_normal(vocab) for _ in range(4)]
    rows.append(np.zeros(vocab)); rows[-1][::2] = -0.0           # +-0 are equal: first index wins
    rows.append(np.full(vocab, -np.inf))                          # all -inf: index 0
    t = rng.standard_normal(vocab); t[vocab // 2] = np.nan; t[vocab - 1] = np.nan; rows.append(t)  # first NaN
    t = np.full(vocab, 1.0); t[vocab - 1] = 2.0; rows.append(t)   # the maximum at the very end
    t = rng.standard_normal(vocab); t[[0, vocab // 3, vocab - 1]] = 9.0; rows.append(t)  # a tie across threads
    x = np.stack(rows).astype(np.float32)
    out = K.sample(dev(x)).cpu().numpy()
    assert out.tolist() == [numpy_rule_argmax(r) for r in x]


def test_temperature_sampling_distribution(K):
    vocab, draws = 37, 20000
    rng = np.random.default_rng(0)
    logits = (rng.standard_normal(vocab) * 2).astype(np.float32)
    x = dev(np.tile(logits, (draws, 1)))
    temps = dev(np.full(draws, 0.7))
    seeds = dev(np.full(draws, 1234), torch.int64)
    steps = dev(np.arange(draws), torch.int32)
    out = K.sample(x, temps, None, seeds, steps).cpu().numpy()
    freq = np.bincount(out, minlength=vocab) / draws
    p = P.softmax(logits.astype(np.float64) / 0.7)
    assert np.abs(freq - p).max() < 4 * np.sqrt(p.max() / draws) + 1e-3
    # the draw is a function of (seed, step) alone: same again, and in another batch order
    again = K.sample(x, temps, None, seeds, steps).cpu().numpy()
    assert (again == out).all()
    perm = rng.permutation(draws)
    shuffled = K.sample(x, temps, None, seeds, dev(np.arange(draws)[perm], torch.int32)).cpu().numpy()
    assert (shuffled == out[perm]).all()
    other = K.sample(x, temps, None, dev(np.full(draws, 99), torch.int64), steps).cpu().numpy()
    assert (other != out).mean() > 0.3
    # temperature 0 rows in the same call are greedy
    mixed = K.sample(x[:4], dev([0.0, 0.7, 0.0, 0.7]), None, seeds[:4], steps[:4]).cpu().numpy()
    assert mixed[0] == mixed[2] == int(np.argmax(logits))


def test_top_p_sampling(K):
    vocab, draws = 50, 8000
    rng = np.random.default_rng(1)
    logits = (rng.standard_normal(vocab) * 1.5).astype(np.float32)
    logits[7] = logits[11]  # equal probabilities stand or fall together
    T, top_p = 0.9, 0.6
    p = P.softmax(logits.astype(np.float64) / T)
    keep = P.top_p_keep(p, top_p)
    x = dev(np.tile(logits, (draws, 1)))
    out = K.sample(x, dev(np.full(draws, T)), dev(np.full(draws, top_p)), dev(np.full(draws, 5), torch.int64), dev(np.arange(draws), torch.int32)).cpu().numpy()
    freq = np.bincount(out, minlength=vocab) / draws
    assert freq[~keep].sum() == 0 and (freq[keep] > 0).all()
    q = np.where(keep, p, 0) / p[keep].sum()
    assert np.abs(freq - q).max() < 4 * np.sqrt(q.max() / draws) + 1e-3
    # a tiny top_p leaves the most likely token only
    out = K.sample(x[:50], dev(np.full(50, T)), dev(np.full(50, 1e-6)), dev(np.arange(50), torch.int64), dev(np.arange(50), torch.int32)).cpu().numpy()
    assert (out == int(np.argmax(logits))).all()


def test_draws_over_the_whole_vocabulary_are_the_generators(K):
    # 50,257 logits a row, rows that start at odd addresses, temperature with and without top-p:
    # every draw is argmax(logit / T + Gumbel noise) over the nucleus, with the noise of the
    # counter-based generator worked out on the host (vectorised twin of sampling.hip's uniform_open)
    vocab, rows = 50257, 6
    rng = np.random.default_rng(8)
    logits = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    temperature = np.array([0.7, 1.0, 1.3, 0.9, 0.0, 2.0], dtype=np.float32)
    top_p = np.array([1.0, 0.9, 0.5, 0.05, 0.3, 1.0], dtype=np.float32)
    seeds, steps = np.array([1, 2, 3, 4, 5, 2**40 + 17], dtype=np.int64), np.array([0, 7, 7, 300, 1, 9], dtype=np.int32)
    out = K.sample(dev(logits), dev(temperature), dev(top_p), dev(seeds, torch.int64), dev(steps, torch.int32)).cpu().numpy()

    def uniforms(seed, step):
        index = np.arange(vocab, dtype=np.uint64)
        with np.errstate(over="ignore"):
            z = np.uint64(seed) + np.uint64(0x9E3779B97F4A7C15) * np.uint64(step + 1) + np.uint64(0xD1B54A32D192ED03) * (index + np.uint64(1))
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            z = z ^ (z >> np.uint64(31))
        return (((z >> np.uint64(41)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)).astype(np.float64)   # in 32-bit like the kernel

    for r in range(rows):
        row = logits[r].astype(np.float64)
        if temperature[r] == 0:
            assert out[r] == int(np.argmax(row))
            continue
        p = P.softmax(row / temperature[r])
        # the mass of all strictly more likely tokens (the logits are all different): kept if it is
        # below top_p (P.top_p_keep's rule, here by one sort); a token whose mass is within 1e-4 of
        # top_p is at the nucleus' edge and may fall either way by rounding
        order = np.argsort(-p)
        above = np.empty(vocab)
        above[order] = np.cumsum(p[order]) - p[order]
        keep = above < top_p[r] if top_p[r] < 1 else np.ones(vocab, dtype=bool)
        edge = np.abs(above - top_p[r]) < 1e-4 if top_p[r] < 1 else np.zeros(vocab, dtype=bool)
        noisy = (row - row.max()) / temperature[r] - np.log(-np.log(uniforms(int(seeds[r]), int(steps[r]))))
        sure = keep & ~edge
        best_sure = noisy[sure].max()
        assert (sure[out[r]] and noisy[out[r]] >= best_sure - 1e-3) or (edge[out[r]] and noisy[out[r]] >= best_sure - 1e-3), f"row {r}: token {out[r]}"


def test_add(K):
    rng = np.random.default_rng(2)
    a, b = rng.standard_normal((7, 33)).astype(np.float32), rng.standard_normal((7, 33)).astype(np.float32)
    np.testing.assert_array_equal(host(K.add(dev(a), dev(b))), (a + b).astype(np.float64))
    np.testing.assert_allclose(host(K.add(dev(a), dev(b, torch.bfloat16))), a + bf16_round(b), atol=1e-6)


def test_operands_are_checked_on_the_host(K):
    from mini_llm_amd.ops.kernels import OperandError

    x = torch.zeros((4, 8), device=DEV)
    with pytest.raises(OperandError):
        K.linear(x, torch.zeros((3, 9), device=DEV))  # inner sizes differ
    with pytest.raises(OperandError):
        K.linear(torch.zeros((4, 8)), torch.zeros((3, 8)))  # CPU tensors: no CPU path
    with pytest.raises(OperandError):
        K.layernorm(x, torch.ones(7, device=DEV), torch.ones(8, device=DEV), 1e-5)
    with pytest.raises(OperandError):
        K.linear(x.t(), torch.zeros((3, 4), device=DEV))  # not contiguous
    # the library's own entry point refuses a residual sum with a 2-byte output, at every shape (a caller through
    # ctypes is not behind the checks above): no kernel would add it for some shapes and drop it for others
    from mini_llm_amd.ops.library import library

    lib = library()
    for rows in (8, 300):
        a = torch.zeros((rows, 64), device=DEV, dtype=torch.bfloat16)
        w = K.pack_matrix(torch.zeros((128, 64), device=DEV, dtype=torch.bfloat16))
        residual = torch.zeros((rows, 128), device=DEV)
        out = torch.zeros((rows, 128), device=DEV, dtype=torch.bfloat16)
        status = lib.mllm_gemm(a.data_ptr(), w.data.data_ptr(), 1, None, residual.data_ptr(), out.data_ptr(), rows, 128, 64, K.BF16, K.BF16, 0, 0, 0, None)
        assert status != 0 and b"residual" in lib.mllm_last_error()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,n_heads,n_kv_heads,head_size,page_size,width", [
    (1, 4, 4, 16, 16, 72), (9, 3, 3, 32, 64, 72), (33, 6, 2, 48, 32, 72), (64, 2, 1, 80, 16, 72), (65, 3, 3, 32, 16, 72), (300, 5, 5, 48, 64, 72),
    (2100, 14, 14, 48, 64, 72),  # enough rows and columns for the large tile
    # a width in whole tiles of 64: in bfloat16 with a packed matrix the kernel that streams its operands into LDS; heads of 40
    # and 24 (a 16-byte piece of columns stays inside a head), grouped heads, and heads of 20 (it does not: the other kernel)
    (300, 5, 5, 48, 64, 128), (700, 6, 2, 40, 32, 192), (2100, 14, 14, 24, 16, 64), (250, 3, 3, 20, 64, 64),
    (2100, 12, 12, 64, 64, 128)])  # tiles of 128 x 192 whose waves hold q columns only, or key or value columns only
@pytest.mark.parametrize("packed", [False, True])
def test_fused_qkv_projection_writes_the_cache(K, dtype, rows, n_heads, n_kv_heads, head_size, page_size, width, packed):
    rng = np.random.default_rng(rows)
    qw, kvw = n_heads * head_size, n_kv_heads * head_size
    x, w, b = rng.standard_normal((rows, width)), rng.standard_normal((qw + 2 * kvw, width)) / 8, rng.standard_normal(qw + 2 * kvw)
    num_pages = max(8, rows // page_size + 2)
    kp = torch.full((num_pages, n_kv_heads, page_size, head_size), 7.0, device=DEV).to(dtype)
    vp = torch.full_like(kp, 7.0)
    slots = rng.permutation(num_pages * page_size)[:rows].astype(np.int32)
    if rows > 2:
        slots[1] = -1  # a padding row writes nothing
    q = K.linear_qkv_cache(dev(x, dtype), as_weight(K, w, dtype, packed), dev(b), kp, vp, dev(slots, torch.int32), n_heads, n_kv_heads, head_size)
    xr, wr = (x.astype(np.float32).astype(np.float64), w.astype(np.float32).astype(np.float64)) if dtype == torch.float32 else (bf16_round(x), bf16_round(w))
    ref = xr @ wr.T + b.astype(np.float32)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(host(q), ref[:, :qw], rtol=tol, atol=tol)
    k_ref, v_ref = np.full((num_pages, n_kv_heads, page_size, head_size), 7.0), np.full((num_pages, n_kv_heads, page_size, head_size), 7.0)
    for r, slot in enumerate(slots):
        if slot >= 0:
            k_ref[slot // page_size, :, slot % page_size, :] = ref[r, qw : qw + kvw].reshape(n_kv_heads, head_size)
            v_ref[slot // page_size, :, slot % page_size, :] = ref[r, qw + kvw :].reshape(n_kv_heads, head_size)
    np.testing.assert_allclose(host(kp), k_ref, rtol=tol, atol=tol)
    np.testing.assert_allclose(host(vp), v_ref, rtol=tol, atol=tol)
    if rows <= 64 and packed:  # the same from rows in the packed layout
        kp.fill_(7.0); vp.fill_(7.0)
        q2 = K.linear_qkv_cache(packed_rows_of(K, xr, dtype), as_weight(K, w, dtype, packed), dev(b), kp, vp, dev(slots, torch.int32), n_heads, n_kv_heads, head_size)
        assert torch.equal(q2, q)
        np.testing.assert_allclose(host(kp), k_ref, rtol=tol, atol=tol)
        np.testing.assert_allclose(host(vp), v_ref, rtol=tol, atol=tol)


@pytest.mark.parametrize("path", ["general", "split_keys", "matrix_cores"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("page_size,window", [(16, 0), (64, 0), (32, 100)])
def test_attention_picks_out_single_keys(K, path, dtype, page_size, window):
    # Random keys hide a wrong page or a missed tile among hundreds of near-equal weights. Here one
    # key at a time gets a score far above the rest (at page edges, tile edges, the window's two
    # sides, the first and the last key), and the output must be that key's value row, or, for
    # the key just outside the window, must not be.
    rng = np.random.default_rng(page_size)
    H, hs, total, new = 2, 32, 333, 40
    first_allowed = max(0, (total - 1) - window + 1) if window else 0
    special = sorted({first_allowed, first_allowed + 1, page_size - 1, page_size, 2 * page_size - 1, 2 * page_size, 63, 64, 127, 128,
                      255, 256, total - 2, total - 1} | ({first_allowed - 1} if window else set()))
    special = [p for p in special if 0 <= p < total]
    n_req = len(special)
    blocks = (total + page_size - 1) // page_size
    pages = rng.permutation(n_req * blocks).reshape(n_req, blocks).astype(np.int32)
    kp = torch.zeros((n_req * blocks, H, page_size, hs), device=DEV).to(dtype)
    vp = torch.zeros_like(kp)
    q_all, refs, treq, tpos = [], [], [], []
    for r, hot in enumerate(special):
        k = bf16_round(rng.standard_normal((total, H * hs)) * 0.1)
        v = bf16_round(rng.standard_normal((total, H * hs)))
        q = bf16_round(rng.standard_normal((new, H * hs)) * 0.1)
        direction = np.tile(np.r_[1.0, np.zeros(hs - 1)], H)
        q[-1] = direction * 16.0            # the last query looks along one direction ...
        k[hot] = direction * 16.0           # ... and one key lies along it: its score is 256/sqrt(32) above the rest
        slots = np.array([pages[r, p // page_size] * page_size + p % page_size for p in range(total)], dtype=np.int32)
        K.cache_write(dev(k, dtype), dev(v, dtype), kp, vp, dev(slots, torch.int32), H, hs)
        q_all.append(q)
        treq += [r] * new
        tpos += list(range(total - new, total))
        refs.append((hot, v))
    extra = {}
    if path == "matrix_cores":
        extra = dict(q_starts=dev(np.arange(n_req + 1) * new, torch.int32), context_lens=dev([total - new] * n_req, torch.int32))
    out = host(K.paged_attention(
        dev(np.concatenate(q_all), dtype), kp, vp, dev(treq, torch.int32), dev(tpos, torch.int32), dev(pages, torch.int32),
        H, H, hs, 1.0 / math.sqrt(hs), window=window, max_q_len={"general": None, "matrix_cores": new}.get(path, 1), **extra))
    for r, (hot, v) in enumerate(refs):
        last = out[(r + 1) * new - 1]
        if hot >= first_allowed:
            np.testing.assert_allclose(last, v[hot], atol=2e-2, err_msg=f"key {hot} should carry the whole weight")
        else:
            assert np.abs(last - v[hot]).max() > 0.2, f"key {hot} lies outside the window and must not count"


@pytest.mark.parametrize("rows,cols", [(1, 1), (33, 65), (96, 288), (1000, 96), (31, 32)])
@pytest.mark.parametrize("src,dst", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float32, torch.float32)])
def test_convert_and_transpose(K, rows, cols, src, dst):
    rng = np.random.default_rng(rows + cols)
    a = rng.standard_normal((rows, cols)).astype(np.float32)
    t = dev(a, src)
    ref = host(t) if dst == torch.float32 else bf16_round(host(t))
    np.testing.assert_array_equal(host(K.convert(t, dst)), ref)
    out = K.convert(t, dst, transpose=True)
    assert tuple(out.shape) == (cols, rows) and out.is_contiguous()
    np.testing.assert_array_equal(host(out), ref.T)
    np.testing.assert_array_equal(host(K.convert(t[0].contiguous(), dst)), ref[0])


# -- a whole layer for rows that bring one token each ---------------------------------------------------
def _pending_rows(K, rng, rows, width, n_partials, with_bias):
    """A stream in pending form and its sum in float64."""
    base = rng.standard_normal((rows, width)).astype(np.float32)
    partials = (rng.standard_normal((n_partials, rows, width)) * 0.3).astype(np.float32) if n_partials else None
    bias = (rng.standard_normal(width) * 0.1).astype(np.float32) if with_bias else None
    total = base.astype(np.float64)
    if bias is not None:
        total = total + bias
    if partials is not None:
        total = total + partials.astype(np.float64).sum(axis=0)
    if partials is None and bias is None:
        return dev(base), total
    return K.PendingRows(dev(base), None if partials is None else dev(partials), None if bias is None else dev(bias)), total


@pytest.mark.parametrize(
    "width,n_heads,n_kv_heads,head_size,page_size,window,n_partials,with_bias",
    [(96, 3, 3, 32, 16, 0, 0, False), (80, 6, 2, 16, 32, 37, 5, True), (768, 12, 12, 64, 64, 0, 48, True),
     (264, 2, 1, 128, 64, 100, 3, False), (256, 1, 1, 256, 16, 0, 17, True), (2048, 4, 4, 64, 128, 0, 2, True)],
)
def test_decode_attention_half(K, width, n_heads, n_kv_heads, head_size, page_size, window, n_partials, with_bias):
    # norm, q/k/v, cache write, attention over the cache and output product in one kernel, for
    # rows that are each the newest token of a request, against the same steps one by one in
    # float64 with bfloat16 kept where the kernel keeps it (normed rows, q, k, v, mixed rows)
    rng = np.random.default_rng(width + head_size)
    q_width, kv_width = n_heads * head_size, n_kv_heads * head_size
    eps = 3e-5
    # -1: a padding row; 700 and 1500 reach beyond the keys the kernel asks for in its first go
    contexts = [0, 1, page_size - 1, page_size, 150, 700, -1, 333, 1500]
    rows = len(contexts)
    hidden, total = _pending_rows(K, rng, rows, width, n_partials, with_bias)
    gamma, beta = 1 + 0.1 * rng.standard_normal(width), 0.1 * rng.standard_normal(width)
    w_qkv = bf16_round(rng.standard_normal((q_width + 2 * kv_width, width)) * (2.0 / math.sqrt(width)))
    b_qkv = 0.1 * rng.standard_normal(q_width + 2 * kv_width)
    w_out = bf16_round(rng.standard_normal((width, q_width)) / math.sqrt(q_width))
    b_out = 0.1 * rng.standard_normal(width)

    num_pages = sum((c + 1 + page_size - 1) // page_size for c in contexts if c >= 0) + 3
    order = rng.permutation(num_pages).tolist()
    kp = torch.full((num_pages, n_kv_heads, page_size, head_size), float("nan"), device=DEV).bfloat16()
    vp = torch.full_like(kp, float("nan"))
    max_blocks = max((c + 1 + page_size - 1) // page_size for c in contexts)
    tables = np.zeros((rows, max_blocks), dtype=np.int32)
    new_slots, treq, tpos, expected = [], [], [], np.zeros((rows, width))
    expect_k, expect_v = {}, {}
    for r, ctx in enumerate(contexts):
        if ctx < 0:
            new_slots.append(-1), treq.append(-1), tpos.append(0)
            continue
        n_blocks = (ctx + 1 + page_size - 1) // page_size
        pages = [order.pop() for _ in range(n_blocks)]
        tables[r, :n_blocks] = pages
        slots = np.array([pages[p // page_size] * page_size + p % page_size for p in range(ctx + 1)], dtype=np.int32)
        k_all, v_all = bf16_round(rng.standard_normal((ctx + 1, kv_width))), bf16_round(rng.standard_normal((ctx + 1, kv_width)))
        if ctx:
            K.cache_write(dev(k_all[:ctx], torch.bfloat16), dev(v_all[:ctx], torch.bfloat16), kp, vp, dev(slots[:ctx], torch.int32), n_kv_heads, head_size)
        new_slots.append(int(slots[ctx])), treq.append(r), tpos.append(ctx)
        normed = bf16_round(P.layernorm(total[r : r + 1], gamma, beta, eps))
        qkv = bf16_round(normed @ w_qkv.T + b_qkv)[0]
        k_all[ctx], v_all[ctx] = qkv[q_width : q_width + kv_width], qkv[q_width + kv_width :]
        expect_k[int(slots[ctx])], expect_v[int(slots[ctx])] = k_all[ctx], v_all[ctx]
        mixed = bf16_round(plain_paged_attention(qkv[None, :q_width], k_all, v_all, n_heads, n_kv_heads, window or None))
        expected[r] = total[r] + mixed[0] @ w_out.T + b_out
    k_before, v_before = kp.clone(), vp.clone()
    out = K.decode_attention_half(
        hidden, dev(gamma), dev(beta), eps, as_weight(K, w_qkv, torch.bfloat16, True), dev(b_qkv), as_weight(K, w_out, torch.bfloat16, True), dev(b_out), kp, vp,
        dev(new_slots, torch.int32), dev(treq, torch.int32), dev(tpos, torch.int32), dev(tables, torch.int32),
        n_heads, n_kv_heads, head_size, 1.0 / math.sqrt(head_size), window=window)
    assert out.partials.shape == (n_heads, rows, width)
    live = [r for r, c in enumerate(contexts) if c >= 0]
    np.testing.assert_allclose(host(out.base)[live], total[live], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(K.settle(out))[live], expected[live], rtol=5e-3, atol=5e-3)
    assert torch.isfinite(K.settle(out)).all()  # the padding row too
    # the new keys and values are in their slots, rounded to bfloat16; nothing else was written
    for pages, before, expect in ((kp, k_before, expect_k), (vp, v_before, expect_v)):
        flat, flat_before = pages.permute(0, 2, 1, 3).reshape(-1, kv_width), before.permute(0, 2, 1, 3).reshape(-1, kv_width)
        for slot, row in expect.items():
            np.testing.assert_allclose(host(flat[slot]), row, rtol=1e-2, atol=1e-2)
            flat_before[slot] = flat[slot]
        assert torch.equal(flat.view(torch.int16), flat_before.view(torch.int16))


def test_decode_attention_half_reads_a_cache_it_does_not_write(K):
    # write_cache=False: the token's own key and value still count, the pages stay as they were
    rng = np.random.default_rng(5)
    width, n_heads, head_size, page_size = 64, 2, 32, 16
    hidden, total = _pending_rows(K, rng, 1, width, 0, False)
    kp = torch.zeros((2, n_heads, page_size, head_size), device=DEV).bfloat16()
    vp = torch.zeros_like(kp)
    args = (dev(np.ones(width)), dev(np.zeros(width)), 1e-5, as_weight(K, rng.standard_normal((3 * width, width)) * 0.2, torch.bfloat16, True), None,
            as_weight(K, rng.standard_normal((width, width)) * 0.2, torch.bfloat16, True), None, kp, vp, dev([3], torch.int32), dev([0], torch.int32),
            dev([3], torch.int32), dev([[0]], torch.int32), n_heads, n_heads, head_size, 0.25)
    reading = K.settle(K.decode_attention_half(hidden, *args, write_cache=False))
    assert not kp.any() and not vp.any()
    writing = K.settle(K.decode_attention_half(hidden, *args, write_cache=True))
    assert kp.any() and vp.any()
    assert torch.equal(reading, writing)


@pytest.mark.parametrize(
    "width,inner,rows,activation,slice_units,n_partials,with_bias",
    [(96, 320, 5, "gelu", 64, 3, True), (768, 3072, 8, "gelu_new", 64, 12, True), (240, 200, 19, "gelu_new", 128, 0, False),
     (2048, 512, 33, "gelu", 128, 2, False), (1032, 136, 16, None, 64, 5, True), (8, 8, 1, "gelu", 64, 1, False)],
)
def test_decode_mlp_half(K, width, inner, rows, activation, slice_units, n_partials, with_bias):
    rng = np.random.default_rng(width + inner)
    eps = 1e-6
    hidden, total = _pending_rows(K, rng, rows, width, n_partials, with_bias)
    gamma, beta = 1 + 0.1 * rng.standard_normal(width), 0.1 * rng.standard_normal(width)
    w_up, b_up = bf16_round(rng.standard_normal((inner, width)) * (2.0 / math.sqrt(width))), 0.1 * rng.standard_normal(inner)
    w_down, b_down = bf16_round(rng.standard_normal((width, inner)) / math.sqrt(inner)), 0.1 * rng.standard_normal(width)
    act = {"gelu": P.gelu_erf, "gelu_new": P.gelu_new, None: lambda x: x}[activation]
    normed = bf16_round(P.layernorm(total, gamma, beta, eps))
    expected = total + bf16_round(act(normed @ w_up.T + b_up)) @ w_down.T + b_down
    out = K.decode_mlp_half(hidden, dev(gamma), dev(beta), eps, as_weight(K, w_up, torch.bfloat16, True), dev(b_up), as_weight(K, w_down, torch.bfloat16, True),
                            dev(b_down), activation=activation, slice_units=slice_units)
    assert out.partials.shape == ((inner + slice_units - 1) // slice_units, rows, width)
    np.testing.assert_allclose(host(out.base), total, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(K.settle(out)), expected, rtol=5e-3, atol=5e-3)


def test_layer_kernels_refuse_what_they_do_not_take(K):
    assert K.decode_layer_supported(768, 64, 64, 3072)
    assert not K.decode_layer_supported(4096)          # wider than a block's threads cover
    assert not K.decode_layer_supported(100)           # rows that are no multiple of 16 bytes
    assert not K.decode_layer_supported(96, 48, 16)    # a head size that is no power of two
    assert not K.decode_layer_supported(96, 32, 24)    # pages that are no power of two
    x = torch.zeros((1, 96), device=DEV)
    ones = torch.ones(96, device=DEV)
    with pytest.raises(K.OperandError):
        K.decode_mlp_half(x, ones, ones, 1e-5, K.pack_matrix(torch.zeros((100, 96), device=DEV).bfloat16()), None, K.pack_matrix(torch.zeros((96, 100), device=DEV).bfloat16()), None)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,n_partials,with_bias", [(1, 64, 0, False), (5, 96, 3, True), (9, 768, 48, True), (3, 1032, 17, False), (2, 2500, 9, True),
                                                            # few rows of many partial rows each: groups of threads share a row's sums
                                                            (4, 1000, 33, True), (7, 64, 16, False), (64, 1024, 21, True), (65, 768, 48, False)])
def test_layernorm_of_pending_rows(K, out_dtype, rows, width, n_partials, with_bias):
    # the sums are taken on the way into the norm; row_index picks and repeats rows
    rng = np.random.default_rng(rows + width)
    hidden, total = _pending_rows(K, rng, rows, width, n_partials, with_bias)
    gamma, beta = 1 + 0.1 * rng.standard_normal(width), 0.1 * rng.standard_normal(width)
    index = np.array([rows - 1, 0, rows - 1], dtype=np.int32)
    tol = 1e-5 if out_dtype == torch.float32 else 1e-2
    out = K.layernorm(hidden, dev(gamma), dev(beta), 2e-5, out_dtype=out_dtype)
    np.testing.assert_allclose(host(out), P.layernorm(total, gamma, beta, 2e-5), rtol=tol, atol=tol)
    out = K.layernorm(hidden, dev(gamma), dev(beta), 2e-5, out_dtype=out_dtype, row_index=dev(index, torch.int32))
    np.testing.assert_allclose(host(out), P.layernorm(total[index], gamma, beta, 2e-5), rtol=tol, atol=tol)
    np.testing.assert_allclose(host(K.settle(hidden)), total, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_layernorm_gives_the_summed_rows_too(K, out_dtype, with_bias):
    rng = np.random.default_rng(12)
    rows, width = 37, 200
    gamma, beta = 1 + 0.1 * rng.standard_normal(width), 0.1 * rng.standard_normal(width)
    tol = 1e-5 if out_dtype == torch.float32 else 1e-2
    for n_partials in (0, 1, 5):
        hidden, total = _pending_rows(K, rng, rows, width, n_partials, with_bias)
        out, summed = K.layernorm(hidden, dev(gamma), dev(beta), 2e-5, out_dtype=out_dtype, with_sums=True)
        np.testing.assert_allclose(host(summed), total, rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(host(out), P.layernorm(total, gamma, beta, 2e-5), rtol=tol, atol=tol)
    plain = dev(total)
    out, summed = K.layernorm(plain, dev(gamma), dev(beta), 2e-5, out_dtype=out_dtype, with_sums=True)
    assert summed is plain
    np.testing.assert_allclose(host(out), P.layernorm(total, gamma, beta, 2e-5), rtol=tol, atol=tol)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k,k_blocks", [(1, 40, 2048, 8), (20, 100, 1000, 3), (64, 1024, 1104, 4), (48, 200, 520, 2), (33, 16, 64, 16), (7, 50, 96, 1),
                                            (65, 40, 2048, 4), (300, 130, 1000, 3), (129, 64, 520, 8), (200, 70, 96, 2),
                                            (300, 136, 1024, 3), (513, 72, 640, 8), (2100, 776, 3072, 2)])
def test_linear_split_leaves_partial_products(K, m, n, k, k_blocks, dtype, packed):
    # the product cut along K: the partial products add up to it, whatever the cut (also one that
    # leaves the last blocks without any k); up to 64 rows in the kernel for few rows, more in the tiled one
    rng = np.random.default_rng(m + n + k)
    rounded = bf16_round if dtype == torch.bfloat16 else (lambda a: a.astype(np.float32).astype(np.float64))
    x, w = rng.standard_normal((m, k)), rng.standard_normal((n, k)) / math.sqrt(k)
    partials = K.linear_split(dev(x, dtype), as_weight(K, w, dtype, packed), k_blocks)
    assert tuple(partials.shape) == (k_blocks, m, n) and partials.dtype == torch.float32
    np.testing.assert_allclose(host(partials).astype(np.float64).sum(axis=0), rounded(x) @ rounded(w).T, rtol=2e-5, atol=2e-5)
    if k == 2048:
        assert (host(partials) != 0).any(axis=(1, 2)).all()  # every block had its share


def test_split_blocks_follow_the_shape(K):
    # few output columns and a long K are cut; many columns, or a short K, are not
    big = lambda n, k, dtype, rows=1: K.split_blocks(torch.empty((n, k), dtype=dtype, device=DEV), dtype, rows)
    assert big(1024, 4096, torch.bfloat16) == 4 and big(768, 3072, torch.float32) == 8
    assert big(4096, 1024, torch.bfloat16) == 1 and big(1024, 96, torch.bfloat16) == 1 and big(64, 64, torch.float32) == 1
    assert big(1024, 4096, torch.bfloat16, 64) == 4 and big(1024, 4096, torch.bfloat16, 512) == 4
    assert big(1024, 4096, torch.bfloat16, 2048) == 1 and big(4096, 1024, torch.bfloat16, 512) == 1


def test_embed_without_a_position_table(K):
    rng = np.random.default_rng(6)
    wte = rng.standard_normal((30, 72)).astype(np.float32)
    out = K.embed(dev([3, -1, 29], torch.int32), dev([5, 0, 900], torch.int32), dev(wte), None)
    np.testing.assert_array_equal(host(out), np.stack([wte[3], np.zeros(72, dtype=np.float32), wte[29]]))


def test_embed_takes_tokens_from_slots(K):
    # rows whose source is not negative take their token from the slot the sampler left it in
    rng = np.random.default_rng(4)
    wte, wpe = rng.standard_normal((50, 96)).astype(np.float32), rng.standard_normal((16, 96)).astype(np.float32)
    tokens = dev([7, -5, 9, 11], torch.int32)
    out = K.embed(tokens, dev([0, 3, 1, 15], torch.int32), dev(wte), dev(wpe), token_sources=dev([-1, 2, -1, 0], torch.int32),
                  token_slots=dev([40, 41, 42], torch.int32))
    assert tokens.tolist() == [7, 42, 9, 40]
    np.testing.assert_allclose(host(out), np.stack([wte[t] + wpe[p] for t, p in zip([7, 42, 9, 40], [0, 3, 1, 15])]), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,n,k", [(8, 50257, 768), (1, 777, 240), (40, 1000, 96), (100, 409, 72), (256, 5000, 64), (33, 130, 1600)])
@pytest.mark.parametrize("packed", [False, True])
def test_the_best_columns_of_a_product_give_the_argmax(K, dtype, rows, n, k, packed):
    # the head of a greedy step: the product's sums are not written, only the best (sum, column) of each of its waves'
    # columns; choosing among them must give numpy's argmax of the sums, ties to the smaller index
    rng = np.random.default_rng(rows + n)
    x, w = rng.standard_normal((rows, k)), rng.standard_normal((n, k)) / 8
    w[n // 2] = w[3]            # equal columns, far apart: equal sums, whatever the order of a kernel's additions
    w[n - 1] = w[3]
    x[rows // 2] = w[3] * 50    # a row whose best columns are those three
    xr, wr = (x.astype(np.float32).astype(np.float64), w.astype(np.float32).astype(np.float64)) if dtype == torch.float32 else (bf16_round(x), bf16_round(w))
    ref = xr @ wr.T
    values, indices = K.linear_best(dev(x, dtype), as_weight(K, w, dtype, packed))
    per_row = K.best_per_row(rows, as_weight(K, w, dtype, packed), dtype)
    assert values.shape == indices.shape == (rows, per_row) and per_row >= 1
    v, i = host(values), indices.cpu().numpy()
    # every column lies in exactly one wave's share, and each entry is the best of its share
    real = i < n
    assert (i[~real] == 0x7FFFFFFF).all() and np.isneginf(v[~real]).all()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for r in range(rows):
        np.testing.assert_allclose(v[r][real[r]], ref[r, i[r][real[r]]], rtol=tol, atol=tol * 4)
    slots = np.arange(rows, dtype=np.int32)[::-1].copy()
    last = torch.full((rows + 3,), -7, dtype=torch.int32, device=DEV)
    tokens = K.choose(values, indices, dev(slots, torch.int32), last).cpu().numpy()
    for r in range(rows):
        assert ref[r, tokens[r]] >= ref[r].max() - tol * 4 * max(1.0, abs(ref[r]).max()), (r, tokens[r], ref[r].argmax())
    assert tokens[rows // 2] == 3                                        # of the three equal columns the first
    assert last.cpu().numpy()[:rows].tolist() == tokens[::-1].tolist() and (last.cpu().numpy()[rows:] == -7).all()
    # the same tokens as the sampler's argmax over the logits the plain product writes
    logits = K.linear(dev(x, dtype), as_weight(K, w, dtype, packed), out_dtype=torch.float32)
    assert tokens.tolist() == K.sample(logits).cpu().numpy().tolist()


def test_the_best_column_of_a_row_with_a_nan_is_the_first_nan(K):
    x = np.ones((3, 64), dtype=np.float32)
    w = np.random.default_rng(0).standard_normal((300, 64)).astype(np.float32)
    w[170, 5] = np.nan
    w[40, 9] = np.nan
    values, indices = K.linear_best(dev(x), dev(w))
    tokens = K.choose(values, indices, dev([0, 1, 2], torch.int32), torch.zeros(3, dtype=torch.int32, device=DEV))
    assert tokens.cpu().tolist() == [40, 40, 40]


def test_choose_moves_a_decode_batch_on_by_one_token(K):
    # what the end of a captured decode step does besides choosing: positions, stored lengths, the cache row of the next
    # token in every group (-1 where the table has no page yet), the token's source, a ring row in page-locked memory
    rng = np.random.default_rng(5)
    rows, width, page = 6, 5, 16
    live = np.array([3, 0, -1, 2, 7, -1], dtype=np.int32)         # state slots; negative: padding
    positions = np.array([15, 31, 0, 40, 79, 0], dtype=np.int32)  # the next ones: 16 (a new page), 32 (no page yet), 41, 80 (beyond the table)
    tables = [rng.integers(0, 90, (rows, width)).astype(np.int32) for _ in range(2)]
    tables[0][1, 2] = -1
    tables[1][1, 2] = -1
    indices = rng.integers(0, 1000, (rows, 1)).astype(np.int32)
    d = lambda a: dev(a, torch.int32)
    pos_d, ctx_d, src_d = d(positions), d(positions), d(np.full(rows, -1))
    tab_d, slot_d = [d(t) for t in tables], [d(np.full(rows, -5)) for _ in tables]
    last = torch.full((9,), -1, dtype=torch.int32, device=DEV)
    ring = torch.full((3, 8), -9, dtype=torch.int32).pin_memory()
    cursor = d([2, 41, 0])
    draws = d(np.arange(rows) * 10)   # how many tokens each row's request has drawn: one more with every step, for live rows
    advance = K.StepAdvance(pos_d, ctx_d, src_d, tab_d, slot_d, page, draw_counts=draws)
    for turn in range(2):
        tokens = K.choose(None, d(indices), d(live), last, host_ring=ring, cursor=cursor, advance=advance)
        torch.cuda.synchronize()
        want = np.where(live >= 0, indices[:, 0], -1)
        assert tokens.cpu().numpy().tolist() == want.tolist()
        ring_row = (2 + turn) % 3
        assert ring[ring_row, :rows].tolist() == want.tolist() and cursor.cpu().tolist() == [(ring_row + 1) % 3, 42 + turn, 0]
        assert ring[ring_row, 7].item() == 41 + turn          # the step's number, behind its tokens
        now = positions + (turn + 1) * (live >= 0)
        assert pos_d.cpu().numpy().tolist() == now.tolist() and ctx_d.cpu().numpy().tolist() == now.tolist()
        assert src_d.cpu().numpy().tolist() == np.where(live >= 0, live, -1).tolist()
        assert draws.cpu().numpy().tolist() == (np.arange(rows) * 10 + (turn + 1) * (live >= 0)).tolist()
        for table, slots in zip(tables, slot_d):
            expect = []
            for r in range(rows):
                block = now[r] // page
                if live[r] < 0:
                    expect.append(-5)
                elif block >= width or table[r, block] < 0:
                    expect.append(-1)
                else:
                    expect.append(int(table[r, block]) * page + now[r] % page)
            assert slots.cpu().numpy().tolist() == expect
    assert last.cpu().numpy().tolist() == [indices[1, 0], -1, indices[3, 0], indices[0, 0], -1, -1, -1, indices[4, 0], -1]
    assert (ring[:, rows:7] == -9).all() and ring[1, 7].item() == -9


def test_choose_over_several_blocks(K):
    # more than 16 rows: a block of the kernel takes 16; each leaves the step's number in an entry of its own at the end
    # of the ring row, and the block that finishes last moves the cursor
    rng = np.random.default_rng(6)
    rows, per_row, page = 40, 700, 16
    values = rng.standard_normal((rows, per_row)).astype(np.float32)
    indices = rng.permutation(rows * per_row).reshape(rows, per_row).astype(np.int32)
    live = rng.permutation(64)[:rows].astype(np.int32)
    live[[3, 17, 39]] = -1
    positions = rng.integers(0, 60, rows).astype(np.int32)
    table = rng.integers(0, 50, (rows, 4)).astype(np.int32)
    d = lambda a: dev(a, torch.int32)
    pos_d, ctx_d, src_d, slot_d = d(positions), d(positions), d(np.full(rows, -1)), d(np.full(rows, -5))
    last = torch.full((64,), -1, dtype=torch.int32, device=DEV)
    flags = K.choose_flags(rows)
    assert flags == 3
    ring = torch.full((4, rows + flags), -9, dtype=torch.int32).pin_memory()
    cursor = d([1, 1000, 0])
    want = np.where(live >= 0, indices[np.arange(rows), values.argmax(axis=1)], -1)
    for turn in range(3):
        tokens = K.choose(dev(values), d(indices), d(live), last, host_ring=ring, cursor=cursor,
                          advance=K.StepAdvance(pos_d, ctx_d, src_d, [d(table)], [slot_d], page))
        torch.cuda.synchronize()
        assert tokens.cpu().numpy().tolist() == want.tolist()
        ring_row = (1 + turn) % 4
        assert ring[ring_row, :rows].tolist() == want.tolist() and ring[ring_row, rows:].tolist() == [1000 + turn] * 3
        assert cursor.cpu().tolist() == [(ring_row + 1) % 4, 1001 + turn, 0]
        assert pos_d.cpu().numpy().tolist() == (positions + (turn + 1) * (live >= 0)).tolist()
    assert last.cpu().numpy()[live[live >= 0]].tolist() == want[live >= 0].tolist()
