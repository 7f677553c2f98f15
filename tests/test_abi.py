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
