"""ctypes binding of ``libcueq_amd.so`` (the C ABI declared in ``include/cueq_amd.h``).

The library is loaded from inside the package directory.  There is no fallback: if the
shared object is missing or an entry point fails, an exception is raised.
"""

from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

import os

# The in-tree build; CUEQ_AMD_LIBRARY may point at another build of the same ABI.
LIB_PATH = Path(os.environ.get("CUEQ_AMD_LIBRARY") or (Path(__file__).resolve().parent / "libcueq_amd.so"))

# enum cueq_dtype
F32, F64, F16, BF16 = 0, 1, 2, 3
# enum cueq_batch_dim
BATCH_DIM_AUTO, BATCH_DIM_SHARED, BATCH_DIM_BATCHED, BATCH_DIM_INDEXED = -1, 0, 1, 2

EXPORTED_SYMBOLS = (
    "cueq_last_error",
    "cueq_version",
    "cueq_set_option",
    "cueq_get_option",
    "cueq_timing_begin",
    "cueq_timing_end",
    "cueq_calibrate",
    "cueq_u1d_plan_create",
    "cueq_u1d_plan_destroy",
    "cueq_u1d_plan_info",
    "cueq_u1d_desc_info",
    "cueq_u1d_desc_serves",
    "cueq_u1d_workspace_size",
    "cueq_u1d_run",
    "cueq_u1d_static_scratch_bytes",
    "cueq_u1d_run_static",
    "cueq_segment_csr_workspace",
    "cueq_segment_csr_build",
    "cueq_segment_csr_build_async",
    "cueq_seg_gemm",
    "cueq_seg_outer_workspace",
    "cueq_seg_outer",
    "cueq_seg_rowdot",
    "cueq_gemm_nt",
    "cueq_gemm",
    "cueq_gemm_table",
    "cueq_linear_rows",
    "cueq_linear_rows_mul_ir",
    "cueq_linear_dw_mul_ir_items",
    "cueq_linear_dw_mul_ir",
    "cueq_fc_combine",
    "cueq_fc_rowdot",
    "cueq_outer_rows",
    "cueq_outer_rows_contract",
    "cueq_gemm_grouped",
    "cueq_segmented_transpose",
    "cueq_layer_norm_t_fwd",
    "cueq_layer_norm_t_bwd_workspace",
    "cueq_layer_norm_t_bwd",
    "cueq_dual_gate",
    "cueq_ln_dual_gate",
    "cueq_gate_bwd_input",
    "cueq_gate_bwd_input_ln",
    "cueq_gemm_tn_items",
    "cueq_gemm_tn",
    "cueq_transpose",
    "cueq_layer_norm_fwd",
    "cueq_layer_norm_bwd_workspace",
    "cueq_layer_norm_bwd",
    "cueq_gate_fwd",
    "cueq_gate_bwd",
    "cueq_sum_cols",
    "cueq_sum_rows_workspace",
    "cueq_sum_rows",
)


class U1dDesc(C.Structure):
    _fields_ = [
        ("math_dtype", C.c_int32),
        ("operand_extent", C.c_int64),
        ("num_inputs", C.c_int32),
        ("num_outputs", C.c_int32),
        ("buffer_dim", C.POINTER(C.c_int32)),
        ("buffer_num_segments", C.POINTER(C.c_int32)),
        ("num_operations", C.c_int32),
        ("num_operands", C.POINTER(C.c_int32)),
        ("operations", C.POINTER(C.c_int32)),
        ("num_paths", C.POINTER(C.c_int32)),
        ("path_indices_start", C.POINTER(C.c_int64)),
        ("path_coefficients_start", C.POINTER(C.c_int64)),
        ("path_indices", C.POINTER(C.c_int32)),
        ("path_indices_len", C.c_int64),
        ("path_coefficients", C.POINTER(C.c_double)),
        ("path_coefficients_len", C.c_int64),
        ("layout_num_groups", C.POINTER(C.c_int32)),
        ("layout_group_dims", C.POINTER(C.c_int32)),
    ]


class U1dBuffer(C.Structure):
    _fields_ = [
        ("data", C.c_void_p),
        ("rows", C.c_int64),
        ("dtype", C.c_int32),
        ("batch_dim", C.c_int32),
        ("index", C.c_void_p),
        ("index_is_64", C.c_int32),
        ("csr_offsets", C.c_void_p),
        ("csr_perm", C.c_void_p),
    ]


class GemmProblem(C.Structure):
    _fields_ = [
        ("a_off", C.c_int64), ("c_off", C.c_int64), ("b_off", C.c_int64), ("alpha", C.c_double),
        ("s_col", C.c_int32), ("trans_b", C.c_int32), ("accumulate", C.c_int32), ("reserved", C.c_int32),
    ]


class OuterEntry(C.Structure):
    _fields_ = [("a_off", C.c_int64), ("c_off", C.c_int64), ("alpha", C.c_double), ("s_col", C.c_int32),
                ("reserved", C.c_int32)]


class TimingEntry(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("launches", C.c_int64), ("total_ms", C.c_double)]


class CueqError(RuntimeError):
    pass


_lock = threading.Lock()
_lib = None


def load() -> C.CDLL:
    """Load the shared library once and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m cuequivariance_amd.build` "
                "(hipcc, gfx950). This package has no non-HIP execution path."
            )
        lib = C.CDLL(str(LIB_PATH))
        lib.cueq_last_error.restype = C.c_char_p
        lib.cueq_version.restype = C.c_char_p
        lib.cueq_timing_begin.restype = C.c_int
        lib.cueq_set_option.argtypes = [C.c_char_p, C.c_int32]
        lib.cueq_set_option.restype = C.c_int
        lib.cueq_get_option.argtypes = [C.c_char_p]
        lib.cueq_get_option.restype = C.c_int
        lib.cueq_timing_end.argtypes = [C.POINTER(TimingEntry), C.c_int]
        lib.cueq_timing_end.restype = C.c_int
        lib.cueq_calibrate.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
        lib.cueq_calibrate.restype = C.c_int
        lib.cueq_u1d_plan_create.argtypes = [C.POINTER(U1dDesc), C.POINTER(C.c_void_p)]
        lib.cueq_u1d_plan_create.restype = C.c_int
        lib.cueq_u1d_plan_destroy.argtypes = [C.c_void_p]
        lib.cueq_u1d_plan_destroy.restype = None
        lib.cueq_u1d_plan_info.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
        lib.cueq_u1d_plan_info.restype = C.c_int
        lib.cueq_u1d_desc_info.argtypes = [C.POINTER(U1dDesc), C.POINTER(C.c_uint64)]
        lib.cueq_u1d_desc_info.restype = C.c_int
        lib.cueq_u1d_desc_serves.argtypes = [C.POINTER(U1dDesc), C.c_int32]
        lib.cueq_u1d_desc_serves.restype = C.c_int
        lib.cueq_u1d_workspace_size.argtypes = [C.c_void_p, C.POINTER(U1dBuffer), C.c_int64]
        lib.cueq_u1d_workspace_size.restype = C.c_int64
        lib.cueq_u1d_run.argtypes = [C.c_void_p, C.POINTER(U1dBuffer), C.c_int64, C.c_void_p, C.c_int64, C.c_void_p]
        lib.cueq_u1d_run.restype = C.c_int
        lib.cueq_u1d_static_scratch_bytes.argtypes = []
        lib.cueq_u1d_static_scratch_bytes.restype = C.c_int64
        lib.cueq_u1d_run_static.argtypes = [C.c_void_p, C.POINTER(U1dBuffer), C.c_int64, C.c_void_p]
        lib.cueq_u1d_run_static.restype = C.c_int
        lib.cueq_segment_csr_workspace.argtypes = [C.c_int64, C.c_int64]
        lib.cueq_segment_csr_workspace.restype = C.c_int64
        lib.cueq_segment_csr_build.argtypes = [
            C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
        ]
        lib.cueq_segment_csr_build.restype = C.c_int
        lib.cueq_segment_csr_build_async.argtypes = lib.cueq_segment_csr_build.argtypes
        lib.cueq_segment_csr_build_async.restype = C.c_int
        lib.cueq_seg_gemm.argtypes = [
            C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
            C.c_int64, C.c_int64, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p,
        ]
        lib.cueq_seg_gemm.restype = C.c_int
        lib.cueq_seg_outer_workspace.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int64]
        lib.cueq_seg_outer_workspace.restype = C.c_int64
        lib.cueq_seg_outer.argtypes = [
            C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
            C.c_void_p, C.c_int64, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int64,
            C.c_void_p,
        ]
        lib.cueq_seg_outer.restype = C.c_int
        lib.cueq_seg_rowdot.argtypes = [
            C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
            C.c_int64, C.c_int64, C.POINTER(GemmProblem), C.c_void_p,
        ]
        lib.cueq_seg_rowdot.restype = C.c_int
        i32, i64, ptr, f64 = C.c_int32, C.c_int64, C.c_void_p, C.c_double
        lib.cueq_gemm_nt.argtypes = [i32, i32, i64, i64, i64, ptr, i64, i64, ptr, i64, i64, ptr, i64, i64, i64, f64, i32, ptr]
        lib.cueq_gemm_nt.restype = C.c_int
        lib.cueq_gemm.argtypes = [i32, i32, i32, i32, i64, i64, i64, ptr, i64, i64, ptr, i64, i64, ptr, i64, i64, i64, f64, i32, ptr]
        lib.cueq_gemm.restype = C.c_int
        lib.cueq_gemm_grouped.argtypes = [i32, i32, i32, i64, i64, i64, ptr, i64, i64, ptr, i64, i64, ptr, i64, i64, i64, ptr, i64, i32, i64,
                                          f64, i32, ptr]
        lib.cueq_gemm_grouped.restype = C.c_int
        lib.cueq_gemm_table.argtypes = [i32, i32, i32, i32, i64, i64, i64, ptr, i64, ptr, i64, ptr, i64, ptr, i64, i64, i64, f64, i32, ptr]
        lib.cueq_gemm_table.restype = C.c_int
        lib.cueq_linear_rows.argtypes = [i32, i32, i64, i64, i64, ptr, i64, ptr, i64, ptr, i64, ptr, i64, f64, ptr]
        lib.cueq_linear_rows.restype = C.c_int
        lib.cueq_linear_rows_mul_ir.argtypes = [i32, i32, i64, i64, i64, ptr, i64, ptr, i64, ptr, i64, ptr, i64, f64, ptr]
        lib.cueq_linear_rows_mul_ir.restype = C.c_int
        lib.cueq_linear_dw_mul_ir_items.argtypes = [i64, ptr, i32, ptr]
        lib.cueq_linear_dw_mul_ir_items.restype = i64
        lib.cueq_linear_dw_mul_ir.argtypes = [i32, i64, i64, i64, ptr, i64, ptr, i64, ptr, i32, ptr, f64, ptr]
        lib.cueq_linear_dw_mul_ir.restype = C.c_int
        lib.cueq_fc_combine.argtypes = [i32, i32, i64, ptr, i64, ptr, i64, ptr, i64, ptr, i32, ptr, i32, i32, ptr]
        lib.cueq_fc_combine.restype = C.c_int
        lib.cueq_fc_rowdot.argtypes = [i32, i32, i64, ptr, i64, ptr, i64, ptr, i64, i32, ptr, i32, i32, ptr]
        lib.cueq_fc_rowdot.restype = C.c_int
        lib.cueq_outer_rows.argtypes = [i32, i64, ptr, i64, ptr, i64, ptr, i64, ptr, i32, i32, i32, i32, ptr]
        lib.cueq_outer_rows.restype = C.c_int
        lib.cueq_outer_rows_contract.argtypes = [i32, i32, i64, ptr, i64, ptr, i64, ptr, i64, ptr, ptr, ptr, i32, i32, i32, i32, ptr]
        lib.cueq_outer_rows_contract.restype = C.c_int
        lib.cueq_segmented_transpose.argtypes = [i32, i64, i64, ptr, ptr, ptr, ptr]
        lib.cueq_segmented_transpose.restype = C.c_int
        lib.cueq_layer_norm_t_fwd.argtypes = [i32, i64, i64, ptr, ptr, ptr, f64, ptr, ptr, ptr, ptr]
        lib.cueq_layer_norm_t_fwd.restype = C.c_int
        lib.cueq_layer_norm_t_bwd_workspace.argtypes = [i32, i64, i64]
        lib.cueq_layer_norm_t_bwd_workspace.restype = C.c_int64
        lib.cueq_layer_norm_t_bwd.argtypes = [i32, i64, i64, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, i64, ptr]
        lib.cueq_layer_norm_t_bwd.restype = C.c_int
        lib.cueq_dual_gate.argtypes = [i32, i32, i64, i64, i64, ptr, ptr, i64, ptr, ptr, i64, ptr, ptr, i32, ptr, i32, ptr, ptr, ptr, i64, ptr]
        lib.cueq_dual_gate.restype = C.c_int
        lib.cueq_ln_dual_gate.argtypes = [i32, i64, i64, i64, ptr, ptr, i64, ptr, i64, ptr, ptr, C.c_double, ptr, ptr, ptr, ptr, i64, ptr, i64, ptr, ptr, ptr]
        lib.cueq_ln_dual_gate.restype = C.c_int
        lib.cueq_gate_bwd_input.argtypes = [i32, i64, i64, i64, ptr, ptr, i64, ptr, ptr, i64, ptr, ptr, ptr, ptr, i64,
                                            i32, ptr, ptr, i64, i32, ptr, ptr, ptr]
        lib.cueq_gate_bwd_input.restype = C.c_int
        lib.cueq_gate_bwd_input_ln.argtypes = [i32, i64, i64, i64, ptr, ptr, i64, ptr, i64, ptr, ptr, ptr, ptr, i64, ptr, i64, i32, ptr, i64, ptr, ptr, ptr, ptr]
        lib.cueq_gate_bwd_input_ln.restype = C.c_int
        lib.cueq_gemm_tn_items.argtypes = [i64, i32]
        lib.cueq_gemm_tn_items.restype = i64
        lib.cueq_gemm_tn.argtypes = [i32, i64, i64, i64, ptr, i64, i64, ptr, i64, i64, i32, ptr, f64, ptr]
        lib.cueq_gemm_tn.restype = C.c_int
        lib.cueq_transpose.argtypes = [i32, i64, i64, i64, ptr, ptr, ptr]
        lib.cueq_transpose.restype = C.c_int
        lib.cueq_layer_norm_fwd.argtypes = [i32, i64, i64, ptr, ptr, ptr, f64, ptr, ptr, ptr, ptr]
        lib.cueq_layer_norm_fwd.restype = C.c_int
        lib.cueq_layer_norm_bwd_workspace.argtypes = [i64, i64]
        lib.cueq_layer_norm_bwd_workspace.restype = i64
        lib.cueq_layer_norm_bwd.argtypes = [i32, i64, i64, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, i64, ptr]
        lib.cueq_layer_norm_bwd.restype = C.c_int
        lib.cueq_gate_fwd.argtypes = [i32, i64, i64, ptr, ptr, ptr, ptr, i32, ptr, i32, ptr, ptr]
        lib.cueq_gate_fwd.restype = C.c_int
        lib.cueq_gate_bwd.argtypes = [i32, i64, i64, ptr, ptr, ptr, ptr, ptr, i32, ptr, i32, ptr, ptr, ptr]
        lib.cueq_gate_bwd.restype = C.c_int
        lib.cueq_sum_cols.argtypes = [i32, i64, i64, ptr, ptr, ptr]
        lib.cueq_sum_cols.restype = C.c_int
        lib.cueq_sum_rows_workspace.argtypes = [i64, i64]
        lib.cueq_sum_rows_workspace.restype = i64
        lib.cueq_sum_rows.argtypes = [i32, i64, i64, ptr, ptr, ptr, i64, ptr]
        lib.cueq_sum_rows.restype = C.c_int
        # the library has read the environment itself at this point: remember what it saw, so that the first launch does
        # not push those values again over an option set by cueq_set_option in the meantime
        for env, _ in _ENV_OPTIONS:
            _env_seen[env] = os.environ.get(env)
        _lib = lib
    return _lib


_ENV_OPTIONS = (("CUEQ_DETERMINISTIC", b"deterministic"), ("CUEQ_FORCE_GENERIC", b"force_generic"))
_env_seen: dict = {}


def sync_options_from_env() -> None:
    """The library reads CUEQ_DETERMINISTIC / CUEQ_FORCE_GENERIC once, when it is loaded; a process that changes them
    afterwards (``os.environ[...] = "1"``) is followed here: called by the Python launch paths, two dictionary lookups
    when nothing changed.  Only a *change* of a variable is pushed, so an option set with ``set_option`` stays as set
    until the variable of the same name is assigned a different value."""
    lib = load()
    for env, name in _ENV_OPTIONS:
        v = os.environ.get(env)
        if _env_seen.get(env) != v:
            _env_seen[env] = v
            lib.cueq_set_option(name, 1 if (v and v[0] == "1") else 0)


def set_option(name: str, value: int) -> None:
    """``cueq_set_option`` ("deterministic", "force_generic"); raises for an unknown name."""
    check(load().cueq_set_option(name.encode(), int(value)), f"cueq_set_option({name!r})")


def get_option(name: str) -> int:
    return int(load().cueq_get_option(name.encode()))


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().cueq_last_error().decode("utf-8", "replace")
        raise CueqError(f"{what} failed (status {status}): {msg}")


def int32_array(values):
    return (C.c_int32 * max(1, len(values)))(*values)


def int64_array(values):
    return (C.c_int64 * max(1, len(values)))(*values)


def double_array(values):
    return (C.c_double * max(1, len(values)))(*values)


def make_desc(tables, math_code: int):
    """(U1dDesc, keep-alive arrays) for a ``U1dTables``."""
    keep = dict(
        buffer_dim=int32_array(tables.buffer_dim),
        nseg=int32_array(tables.buffer_num_segments),
        num_operands=int32_array(tables.num_operands),
        operations=int32_array(tables.operations),
        num_paths=int32_array(tables.num_paths),
        pis=int64_array(tables.path_indices_start),
        pcs=int64_array(tables.path_coefficients_start),
        pi=int32_array(tables.path_indices),
        pc=double_array(tables.path_coefficients),
    )
    layouts = getattr(tables, "layouts", ())
    if layouts:
        keep["lay_n"] = int32_array([len(lay) for lay in layouts])
        keep["lay_d"] = int32_array([d for lay in layouts for d in lay])
    desc = U1dDesc(
        math_dtype=math_code,
        operand_extent=tables.operand_extent,
        num_inputs=tables.num_inputs,
        num_outputs=tables.num_outputs,
        buffer_dim=keep["buffer_dim"],
        buffer_num_segments=keep["nseg"],
        num_operations=len(tables.num_operands),
        num_operands=keep["num_operands"],
        operations=keep["operations"],
        num_paths=keep["num_paths"],
        path_indices_start=keep["pis"],
        path_coefficients_start=keep["pcs"],
        path_indices=keep["pi"],
        path_indices_len=len(tables.path_indices),
        path_coefficients=keep["pc"],
        path_coefficients_len=len(tables.path_coefficients),
    )
    if layouts:
        desc.layout_num_groups = keep["lay_n"]
        desc.layout_group_dims = keep["lay_d"]
    return desc, keep


def timing_begin() -> None:
    check(load().cueq_timing_begin(), "cueq_timing_begin")


def timing_end() -> dict:
    """{kernel name: (launches, total milliseconds)} of the kernels launched since ``timing_begin``."""
    buf = (TimingEntry * 64)()
    n = load().cueq_timing_end(buf, 64)
    return {buf[i].name.decode(): (int(buf[i].launches), float(buf[i].total_ms)) for i in range(n)}
