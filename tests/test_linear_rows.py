"""The row-streaming Linear launch ``cueq_linear_rows`` (all weight blocks of a launch resident in the local data share).

GPU: against the float64 product of the same inputs (bfloat16 and float32), both weight orientations, every supported
extent, ragged row counts, several parts per weight block, and through ``cuet.Linear`` at the benchmark's size against the
tiled launch it replaces.  Tolerance relative to ``max|ref|``: bfloat16 2^-8 (one rounding of the result; the accumulation
is float32), float32 1e-5.
CPU: the argument checks, which return before anything touches a device.
"""

import ctypes as C

import pytest
import torch

from cuequivariance_amd import _lib, cue

BF16, F16, F32, F64 = 3, 2, 0, 1


def _table(rows):
    return (C.c_int64 * (3 * len(rows)))(*[v for r in rows for v in r])


def test_argument_checks_without_a_device():
    lib = _lib.load()
    buf = (C.c_char * 4096)()
    ptr = C.addressof(buf) + (-C.addressof(buf)) % 16
    one = _table([(0, 0, 0)])
    call = lambda dtype, M, N, K, lda, ldc, table, nparts: lib.cueq_linear_rows(dtype, 1, M, N, K, ptr, lda, ptr, 9 * 128 * 128, ptr, ldc, table, nparts, 1.0, None)
    assert call(F64, 64, 128, 128, 128, 128, one, 1) == -2  # float64: not built
    assert call(BF16, 64, 48, 128, 128, 128, one, 1) == -2  # extent not a multiple of 32
    assert call(BF16, 64, 128, 160, 160, 128, one, 1) == -2  # contraction above 128
    assert call(BF16, 64, 128, 128, 128, 128, one, 49) == -4  # too many parts
    assert call(BF16, 64, 128, 128, 100, 128, one, 1) == -2  # row stride not a multiple of 16 bytes
    assert call(BF16, 64, 128, 128, 128, 128, _table([(8, 0, 0)]), 1) == -1  # part runs past the row
    assert call(BF16, 64, 128, 128, 128, 128, _table([(0, 4, 0)]), 1) == -1  # weight offset not a multiple of 8
    assert call(BF16, 64, 128, 128, 128, 128, _table([(0, 9 * 128 * 128 - 8, 0)]), 1) == -1  # weight block past the end
    nine = _table([(0, 128 * 128 * s, 0) for s in range(9)])
    assert call(BF16, 64, 128, 128, 128, 128, nine, 9) == -4  # nine distinct weight blocks
    five = _table([(0, 128 * 128 * s, 0) for s in range(5)])
    assert call(BF16, 64, 128, 128, 128, 128, five, 5) == -4  # 5 x 34 KB of weights + staging exceed 160 KB
    assert b"local data share" in lib.cueq_last_error()
    three = _table([(0, 128 * 128 * s, 0) for s in range(3)])
    assert call(F32, 64, 128, 128, 128, 128, three, 3) == -4  # three float32 blocks of 66 KB do not fit (three bfloat16 ones do)
    assert call(BF16, 0, 128, 128, 128, 128, one, 1) == 0  # nothing to do


def _reference(A, W, parts, K, N, contraction_major, alpha, ldc):
    out = torch.zeros(A.shape[0], ldc, dtype=torch.float64, device=A.device)
    for a_off, w_off, c_off in parts:
        blk = W[w_off : w_off + K * N].double()
        blk = blk.view(K, N) if contraction_major else blk.view(N, K).t()
        out[:, c_off : c_off + N] = alpha * (A[:, a_off : a_off + K].double() @ blk)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("contraction_major", [1, 0])
@pytest.mark.parametrize(
    "M,K,N,nblocks,nparts",
    [
        (1000, 128, 128, 2, 9),
        (31, 128, 128, 1, 1),
        (4097, 64, 96, 2, 3),
        (333, 32, 32, 3, 7),
        (65, 96, 64, 3, 4),
        (50_000, 128, 32, 2, 6),
        (1, 32, 128, 1, 2),
        (200, 64, 64, 2, 40),  # more parts than a block has wavefronts
        (40, 128, 128, 3, 48),  # the most parts a launch takes, fewer units than wavefronts
    ],
)
def test_linear_rows_against_float64_product(device, dtype, contraction_major, M, K, N, nblocks, nparts):
    lib = _lib.load()
    g = torch.Generator(device=device).manual_seed(M + K + N)
    lda, ldc = nparts * K + 8, nparts * N + 16
    es = 4 if dtype == torch.float32 else 2
    nblocks = min(nblocks, (160 * 1024 - 8 * 32 * 144) // (N * (es * K + 16)))  # what the local data share holds
    A = torch.randn(M, lda, device=device, generator=g).to(dtype)
    W = torch.randn(nblocks * K * N + 8, device=device, generator=g).to(dtype)
    # parts in scrambled column order, weight blocks shared between parts
    parts = [(((p + 1) % nparts) * K, (p % nblocks) * K * N, (nparts - 1 - p) * N + 16) for p in range(nparts)]
    assert len({p[2] for p in parts}) == nparts
    out = torch.full((M, ldc), 7.0, device=device).to(dtype)
    alpha = 0.37
    stream = torch.cuda.current_stream(device).cuda_stream
    code = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}[dtype]
    _lib.check(lib.cueq_linear_rows(code, contraction_major, M, N, K, A.data_ptr(), lda, W.data_ptr(), W.numel(), out.data_ptr(), ldc, _table(parts),
                                    nparts, alpha, stream), "cueq_linear_rows")
    ref = _reference(A, W, parts, K, N, contraction_major, alpha, ldc)
    written = torch.zeros(ldc, dtype=torch.bool, device=device)
    for _, _, c_off in parts:
        written[c_off : c_off + N] = True
    got = out.double()
    assert (got[:, ~written] == 7.0).all()  # columns of no part stay as they were
    err = (got[:, written] - ref[:, written]).abs().max().item()
    tol = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 1e-5}[dtype]
    assert err <= tol * ref.abs().max().item(), err


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,launches", [(torch.bfloat16, 2), (torch.float32, 6)])
def test_linear_module_takes_the_streaming_launch_and_agrees_with_the_tiled_one(device, dtype, launches):
    from cuequivariance_amd import cuet
    from cuequivariance_amd.cuet import dense

    irreps = cue.Irreps("O3", "128x0e+128x1o+128x2e")
    m = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
    Z = 200_000
    g = torch.Generator(device=device).manual_seed(5)
    w = torch.randn(1, m.weight_numel, device=device, generator=g).to(dtype).requires_grad_(True)
    x = torch.randn(Z, irreps.dim, device=device, generator=g).to(dtype).requires_grad_(True)
    cot = torch.randn(Z, irreps.dim, device=device, generator=g).to(dtype)
    lib = _lib.load()
    lib.cueq_timing_begin()
    y = m(x, w)
    gx, gw = torch.autograd.grad(y, [x, w], cot)
    torch.cuda.synchronize()
    names = dict(_lib.timing_end())
    # bfloat16: the three weight blocks fit one launch each way; float32: one launch per block
    assert names.get("linear_rows", (0, 0))[0] == launches, names
    saved = dense._rows_tables
    try:
        dense._rows_tables = lambda K, N, plist: None
        m2 = cuet.Linear(irreps, irreps, layout=cue.ir_mul, internal_weights=False, method="fused_tp")
        y2 = m2(x, w)
        gx2, gw2 = torch.autograd.grad(y2, [x, w], cot)
    finally:
        dense._rows_tables = saved
    # same products, same float32 accumulation over 128 terms in a different order: at most one rounding step apart
    tol = 2.0 ** -7 if dtype == torch.bfloat16 else 2e-6
    for a, b in ((y, y2), (gx, gx2)):
        assert (a.float() - b.float()).abs().max().item() <= tol * b.float().abs().max().item()
    assert torch.equal(gw, gw2)
