"""The C-ABI library loads on a host without a GPU and exports what ``include/cueq_amd.h`` declares."""

import ctypes
import re
from pathlib import Path

import pytest

from cuequivariance_amd import _lib, cue
from cuequivariance_amd.tables import U1dTables

ROOT = Path(__file__).resolve().parent.parent


def declared_entry_points():
    text = (ROOT / "include" / "cueq_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cueq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_entry_points():
    assert declared_entry_points() == sorted(_lib.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_entry_points():
        assert hasattr(lib, name), name
    assert b"gfx950" in lib.cueq_version()


def test_error_reporting_without_device():
    lib = _lib.load()
    rc = lib.cueq_u1d_plan_create(None, None)
    assert rc == -1 and b"null" in lib.cueq_last_error()
    with pytest.raises(_lib.CueqError):
        _lib.check(rc, "cueq_u1d_plan_create")


@pytest.mark.parametrize("math_code", [0, 1])
def test_table_hash_agrees_between_python_and_c(math_code):
    lib = _lib.load()
    e = cue.descriptors.channelwise_tensor_product(
        cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e"), "0e+1o+2e"
    )
    t = U1dTables.from_polynomial(e.polynomial.flatten_coefficient_modes().squeeze_modes())
    for tables in (t, t.backward((True, True, True)), t.backward((False, True, False))):
        desc, keep = _lib.make_desc(tables, math_code)
        h = ctypes.c_uint64()
        has_spec = lib.cueq_u1d_desc_info(ctypes.byref(desc), ctypes.byref(h))
        assert h.value == tables.content_hash(math_code)
        # kernels for this descriptor (forward and the all-gradients backward) are generated at build time
        assert has_spec == (0 if tables.num_outputs == 1 and tables.num_inputs == 4 else 1)


def test_dense_entries_refuse_bad_arguments_before_any_launch():
    """Argument checks of the tiled-GEMM family run on the host: no GPU is touched when a request is refused."""
    lib = _lib.load()
    F32, F64, BF16 = _lib.F32, _lib.F64, _lib.BF16
    p = 4096  # a fake, 16-byte aligned address: never dereferenced by a refused call
    # dtype outside float32 / bfloat16 / half
    assert lib.cueq_gemm(F64, F64, 0, 0, 8, 8, 8, p, 8, 0, p, 8, 0, p, 8, 0, 1, 1.0, 0, None) == -2
    assert b"float32, bfloat16 or half" in lib.cueq_last_error()
    # negative extent, null operand
    assert lib.cueq_gemm(F32, F32, 0, 0, -1, 8, 8, p, 8, 0, p, 8, 0, p, 8, 0, 1, 1.0, 0, None) == -1
    assert lib.cueq_gemm(F32, F32, 0, 0, 8, 8, 8, None, 8, 0, p, 8, 0, p, 8, 0, 1, 1.0, 0, None) == -1
    # empty problems succeed without a launch
    assert lib.cueq_gemm(F32, F32, 0, 0, 0, 8, 8, None, 8, 0, None, 8, 0, None, 8, 0, 1, 1.0, 0, None) == 0
    # grouped: unknown mode; rows-grouped keeps the dtype
    assert lib.cueq_gemm_grouped(F32, F32, 7, 8, 8, 8, p, 8, 0, p, 8, 0, p, 8, 0, 1, p, 2, 0, 64, 1.0, 0, None) == -1
    assert lib.cueq_gemm_grouped(BF16, F32, 1, 8, 8, 8, p, 8, 0, p, 8, 0, p, 8, 0, 1, p, 2, 0, 64, 1.0, 0, None) == -2
    # table-driven: the contraction is cut only for contraction-major operands
    assert lib.cueq_gemm_table(F32, F32, 0, 0, 8, 8, 8, p, 8, p, 8, p, 8, p, 1, 4, 64, 1.0, 0, None) == -2
    # fused gate backward: K beyond 128, C not a multiple of 32
    args = (p, p, 160, p, None, 160, None, None, None, p, 64, 1, p, None, 160, 0, None, None, None)
    assert lib.cueq_gate_bwd_input(BF16, 64, 128, 160, *args) == -2 and b"K must be" in lib.cueq_last_error()
    args = (p, p, 128, p, None, 128, None, None, None, p, 64, 1, p, None, 128, 0, None, None, None)
    assert lib.cueq_gate_bwd_input(BF16, 48, 128, 128, *args) == -2
    # LayerNorm with layout change: D beyond 256
    assert lib.cueq_layer_norm_t_fwd(F32, 64, 512, p, None, None, 1e-5, p, p, p, None) == -2
    # segmented transpose: element size, aliasing
    assert lib.cueq_segmented_transpose(3, 4, 4, p, p, 2 * p, None) == -2
    assert lib.cueq_segmented_transpose(4, 4, 4, p, p, p, None) == -1 and b"in place" in lib.cueq_last_error()
    # fully-connected stages: block width, operand width
    assert lib.cueq_fc_combine(F32, F32, 4, p, 1, p, 1, p, 1, p, 1, p, 512, 0, None) == -1
    assert lib.cueq_fc_rowdot(F32, F32, 4, p, 1, p, 1, p, 1, 100, p, 1, 0, None) == -2
    # LayerNorm fused into the gated projection: bfloat16 only, row count, weights that do not fit the local data share
    ln = lambda dtype, C, M, K, ldc: lib.cueq_ln_dual_gate(dtype, C, M, K, p, p, K, p, K, None, None, 1e-5, None, None, None, p, ldc, p, K, p, p, None)
    assert ln(F32, 256, 8192, 128, 8192) == -2 and b"bfloat16" in lib.cueq_last_error()
    assert ln(BF16, 256, 2048, 128, 2048) == -2 and b"at least 4096" in lib.cueq_last_error()
    assert ln(BF16, 256, 8192, 160, 8192) == -2
    assert ln(BF16, 1024, 8192, 128, 8192) == -2  # 2 x 1024 x 256 bytes of weights
    assert ln(BF16, 256, 8192, 128, 4096) == -4  # result rows shorter than M
    assert ln(BF16, 256, 0, 128, 0) == 0
    # gate backward continued through the LayerNorm: bfloat16 only, the LayerNorm's input rows given and aligned
    lnb = lambda dtype, lx, ldlx: lib.cueq_gate_bwd_input_ln(dtype, 256, 8192, 128, p, p, 128, p, 128, None, None, None, p, 8192, p, 128, 0, lx, ldlx, p, p,
                                                             None, None)
    assert lnb(F32, p, 128) == -2 and lnb(BF16, None, 128) == -1 and lnb(BF16, p + 8, 128) == -2 and lnb(BF16, p, 100) == -2



def test_option_set_by_the_program_survives_the_environment_sync(monkeypatch):
    """An option set with ``cueq_set_option`` stays as set when the launch path looks at the environment (only a change
    of the variable is pushed); assigning the variable afterwards is followed."""
    monkeypatch.delenv("CUEQ_DETERMINISTIC", raising=False)
    lib = _lib.load()
    _lib._env_seen["CUEQ_DETERMINISTIC"] = None  # what load() records when the variable is unset
    try:
        assert lib.cueq_set_option(b"deterministic", 1) == 0
        _lib.sync_options_from_env()
        assert lib.cueq_get_option(b"deterministic") == 1
        _lib.set_option("deterministic", 0)
        _lib.sync_options_from_env()
        assert _lib.get_option("deterministic") == 0
        monkeypatch.setenv("CUEQ_DETERMINISTIC", "1")
        _lib.sync_options_from_env()
        assert _lib.get_option("deterministic") == 1
        monkeypatch.delenv("CUEQ_DETERMINISTIC")
        _lib.sync_options_from_env()
        assert _lib.get_option("deterministic") == 0
        with pytest.raises(_lib.CueqError):
            _lib.set_option("no_such_option", 1)
    finally:
        lib.cueq_set_option(b"deterministic", 0)
        _lib._env_seen["CUEQ_DETERMINISTIC"] = None
