"""The row-streaming Linear launch for rows that keep the irrep component contiguous (``cueq_linear_rows_mul_ir``).

GPU: through the C ABI against the float64 product of the same inputs (bfloat16 and float32), both weight orientations,
every supported number of components and extent, ragged row counts, several parts per weight block.  Tolerance relative
to ``max|ref|``: bfloat16 2^-8 (one rounding of the result; the accumulation is float32), float32 1e-5.
CPU: the argument checks, which return before anything touches a device.
"""

import ctypes as C

import pytest
import torch

from cuequivariance_amd import _lib

BF16, F16, F32, F64 = 3, 2, 0, 1


def _table(rows):
    return (C.c_int64 * (len(rows[0]) * len(rows)))(*[v for r in rows for v in r])


def test_argument_checks_without_a_device():
    lib = _lib.load()
    buf = (C.c_char * 4096)()
    ptr = C.addressof(buf) + (-C.addressof(buf)) % 16
    call = lambda dtype, M, N, K, lda, ldc, rows, nparts=None: lib.cueq_linear_rows_mul_ir(
        dtype, 1, M, N, K, ptr, lda, ptr, 9 * 128 * 128, ptr, ldc, _table(rows), len(rows) if nparts is None else nparts, 1.0, None)
    one = [(0, 0, 0, 3)]
    assert call(F64, 64, 128, 128, 384, 384, one) == -2  # float64: not built
    assert call(BF16, 64, 128, 128, 512, 512, [(0, 0, 0, 4)]) == -2  # 4 components: not built
    assert call(BF16, 64, 48, 128, 384, 384, one) == -2  # extent not a multiple of 32
    assert call(BF16, 64, 128, 96, 384, 384, one) == -2  # bfloat16 contraction not a multiple of 64
    assert call(BF16, 64, 128, 128, 380, 384, one) == -2  # row stride not a multiple of 16 bytes
    assert call(BF16, 64, 128, 128, 384, 384, [(8, 0, 0, 3)]) == -1  # part runs past the row
    assert call(BF16, 64, 128, 128, 384, 384, one * 49) == -4  # too many parts
    five = [(0, 128 * 128 * s, 0, 3) for s in range(5)]
    assert call(BF16, 64, 128, 128, 384, 384, five) == -4  # five blocks of one D: 5 x 34 KB + staging exceed 160 KB
    assert b"local data share" in lib.cueq_last_error()
    assert call(BF16, 0, 128, 128, 384, 384, one) == 0  # nothing to do


def _reference(A, W, parts, K, N, contraction_major, alpha, ldc):
    out = torch.zeros(A.shape[0], ldc, dtype=torch.float64, device=A.device)
    for a_off, w_off, c_off, D in parts:
        blk = W[w_off: w_off + K * N].double()
        blk = blk.view(K, N) if contraction_major else blk.view(N, K).t()
        x = A[:, a_off: a_off + K * D].double().view(-1, K, D)
        out[:, c_off: c_off + N * D] = alpha * torch.einsum("zui,uv->zvi", x, blk).reshape(-1, N * D)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("contraction_major", [1, 0])
@pytest.mark.parametrize(
    "M,K,N,dims",
    [
        (1000, 128, 128, [1, 3, 5]),  # the irreps of the benchmark's Linear
        (1000, 128, 128, [5, 5]),  # two parts of one D sharing a weight block
        (15, 128, 128, [7]),
        (4097, 64, 96, [3, 1, 3]),
        (333, 64, 32, [5, 3, 1, 7, 5, 3, 1]),
        (65, 128, 64, [7, 7, 1, 1]),
        (20_000, 128, 32, [3, 3, 3, 1, 1, 5]),
        (1, 64, 128, [5, 1]),
        (200, 64, 64, [3] * 20 + [1] * 20),  # more parts than a block has wavefronts
        (48, 128, 128, [3] * 24 + [1] * 24),  # the most parts a launch takes
        (77, 32, 64, [3, 1]),  # (float32 only: a bfloat16 slice is 64 channels)
        (130, 96, 96, [5, 1, 3]),  # (float32 only)
        (900, 128, 128, [1, 1]),  # parts of one component only
    ],
)
def test_against_float64_product(device, dtype, contraction_major, M, K, N, dims):
    if dtype != torch.float32 and K % 64:
        pytest.skip("a slice of 2-byte elements is 64 channels")
    lib = _lib.load()
    g = torch.Generator(device=device).manual_seed(M + K + N + sum(dims))
    nparts = len(dims)
    lda, ldc = sum(K * d for d in dims) + 8, sum(N * d for d in dims) + 16
    # one weight block per distinct D (parts of equal D share it)
    ds = sorted(set(dims))
    A = torch.randn(M, lda, device=device, generator=g).to(dtype)
    W = torch.randn(len(ds) * K * N + 8, device=device, generator=g).to(dtype)
    # input blocks in order, output blocks in reverse order
    a_offs = [sum(K * d for d in dims[:p]) for p in range(nparts)]
    c_offs = [16 + sum(N * d for d in dims[p + 1:]) for p in range(nparts)]
    parts = [(a_offs[p], ds.index(dims[p]) * K * N, c_offs[p], dims[p]) for p in range(nparts)]
    out = torch.full((M, ldc), 7.0, device=device).to(dtype)
    alpha = 0.37
    stream = torch.cuda.current_stream(device).cuda_stream
    code = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}[dtype]
    _lib.check(lib.cueq_linear_rows_mul_ir(code, contraction_major, M, N, K, A.data_ptr(), lda, W.data_ptr(), W.numel(), out.data_ptr(), ldc,
                                           _table(parts), nparts, alpha, stream), "cueq_linear_rows_mul_ir")
    ref = _reference(A, W, parts, K, N, contraction_major, alpha, ldc)
    written = torch.zeros(ldc, dtype=torch.bool, device=device)
    for _, _, c_off, d in parts:
        written[c_off: c_off + N * d] = True
    got = out.double()
    assert (got[:, ~written] == 7.0).all()  # columns of no part stay as they were
    err = (got[:, written] - ref[:, written]).abs().max().item()
    tol = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 1e-5}[dtype]
    assert err <= tol * ref.abs().max().item(), err


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize(
    "rows,K,N,dims",
    [
        (3000, 128, 128, [1, 3, 5]),
        (999, 64, 64, [3]),
        (517, 128, 64, [5, 1]),
        (70, 32, 96, [3, 7]),
        (1, 96, 32, [1]),
        (20_011, 64, 128, [7, 5, 3, 1, 3]),
    ],
)
def test_weight_gradient_against_float64_product(device, dtype, rows, K, N, dims):
    """``cueq_linear_dw_mul_ir`` + the ordered sum of its chunks against ``einsum('zui,zvi->uv')`` in float64.  The
    products of bfloat16 inputs are exact in float32, so both dtypes are held to float32 accumulation error."""
    lib = _lib.load()
    g = torch.Generator(device=device).manual_seed(rows + K + N)
    lda, ldg = sum(K * d for d in dims) + 8, sum(N * d for d in dims) + 16
    A = torch.randn(rows, lda, device=device, generator=g).to(dtype)
    G = torch.randn(rows, ldg, device=device, generator=g).to(dtype)
    a_offs = [8 + sum(K * d for d in dims[:p]) for p in range(len(dims))]
    c_offs = [16 + sum(N * d for d in dims[p + 1:]) for p in range(len(dims))]  # (the cotangent's blocks in reverse order)
    table = _table([(a, c, d) for a, c, d in zip(a_offs, c_offs, dims)])
    first = (C.c_int32 * (len(dims) + 1))()
    items = lib.cueq_linear_dw_mul_ir_items(rows, table, len(dims), first)
    assert items == first[len(dims)] and all(first[p] < first[p + 1] for p in range(len(dims)))
    part = torch.full((items, K * N), float("nan"), device=device)
    alpha = 0.61
    stream = torch.cuda.current_stream(device).cuda_stream
    code = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}[dtype]
    _lib.check(lib.cueq_linear_dw_mul_ir(code, K, N, rows, A.data_ptr(), lda, G.data_ptr(), ldg, table, len(dims), part.data_ptr(), alpha, stream),
               "cueq_linear_dw_mul_ir")
    for p, (a, c, d) in enumerate(zip(a_offs, c_offs, dims)):
        got = part[first[p]: first[p + 1]].double().sum(0).view(K, N)
        x = A[:, a: a + K * d].double().view(rows, K, d)
        y = G[:, c: c + N * d].double().view(rows, N, d)
        ref = alpha * torch.einsum("zui,zvi->uv", x, y)
        err = (got - ref).abs().max().item()
        assert err <= 2e-6 * max(1.0, (x.abs().max() * y.abs().max()).item()) * (rows * d) ** 0.5 + 1e-5 * ref.abs().max().item(), (p, err)


@pytest.mark.parametrize("es", [2, 4])
@pytest.mark.parametrize("extent", [32, 64, 96, 128])
@pytest.mark.parametrize("d", [1, 3, 5, 7])
def test_weight_gradient_requests_stay_inside_the_row_piece(es, extent, d):
    """The requests of ``cueq_linear_dw_mul_ir`` carry no condition (``csrc/linear_dw_mul_ir.hip``, ``dw_body``): thread ``tid``
    asks for the 16-byte vectors ``E0 + min(v * step, lim)`` of its row's piece, ``E0`` replaced by 0 when the thread's first
    vector lies past the piece.  Restated here for every supported extent and block size: no request may reach past the
    ``extent * d`` elements of the piece - for the last row of a tensor that would be past the tensor (a piece of 32 floats
    was read up to its element 127 before ``E0`` was replaced)."""
    epv = 16 // es
    zr, epl = 2 * epv, 128 // es
    vectors = extent * d // epv
    for tid in range(256):
        line0, l8 = (tid >> 3) // zr, tid & 7
        has = line0 * 8 + l8 < vectors
        lim = ((vectors - 1 - line0 * 8 - l8) // (8 * (32 // zr))) * (32 // zr) * epl if has else 0
        e0 = line0 * epl + l8 * epv if has else 0
        for v in range(d):
            first = e0 + min(v * (32 // zr) * epl, lim)
            assert first % epv == 0 and first + epv <= extent * d, (tid, v, first)


def test_weight_gradient_argument_checks_without_a_device():
    lib = _lib.load()
    buf = (C.c_char * 4096)()
    ptr = C.addressof(buf) + (-C.addressof(buf)) % 16
    call = lambda dtype, K, N, lda, ldg, rows_: lib.cueq_linear_dw_mul_ir(dtype, K, N, 64, ptr, lda, ptr, ldg, _table(rows_), len(rows_), ptr, 1.0, None)
    assert call(F64, 128, 128, 384, 384, [(0, 0, 3)]) == -2
    assert call(BF16, 128, 48, 384, 384, [(0, 0, 3)]) == -2
    assert call(BF16, 128, 128, 384, 384, [(0, 0, 2)]) == -2  # two components: not built
    assert call(BF16, 128, 128, 384, 384, [(8, 0, 3)]) == -1  # runs past the row
    assert call(BF16, 128, 128, 380, 384, [(0, 0, 3)]) == -2  # row stride
    assert lib.cueq_linear_dw_mul_ir_items(1000, _table([(0, 0, 3)]), 0, None) == -1
