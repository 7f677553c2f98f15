"""Descriptor-specialised kernels at first use.

The library ships straight-line kernels for the descriptors listed in ``codegen/registry.py``; every other descriptor
would run on the table-driven kernels, which are twenty to a hundred times slower on large workloads.  Unless this module is switched off
(``CUEQ_AMD_JIT=0`` in the environment, or ``enable(False)``), the first plan of a descriptor that has no specialised
kernels yet generates a translation unit - the same kind the build generates for channel-wise products
(``codegen/channelwise.py``) and symmetric contractions (``codegen/symmetric.py``), a general straight-line one
(``codegen/general.py``) for anything else -, compiles it with ``hipcc`` for gfx950 into a small shared object next to a
cache key, and loads it: its static initialiser registers the kernels with the library (``cueq::register_u1d_spec``), and the plan that
is created right afterwards finds them.  The reference's uniform-1d operator is compiled at first use as well
(``SegmentedPolynomialFromUniform1dJit``, ``cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:82``).

Compiling takes a few seconds per descriptor and math type (tens for the largest), once per machine: shared objects are kept under
``CUEQ_AMD_JIT_CACHE`` (default ``~/.cache/cuequivariance_amd``), keyed by the table hash and the library build.
When ``hipcc`` is missing or the cache cannot be written the plan runs on the table-driven kernels and says so once.
(The test suite switches it off except where it is the subject: dozens of small descriptors would each be compiled.)
"""

from __future__ import annotations

import ctypes as C
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
from pathlib import Path
from typing import Optional

from . import _lib
from .tables import U1dTables

__all__ = ["enable", "enabled", "ensure_plan", "ensure_specialised", "fully_connected_unit", "is_channelwise", "is_symmetric_contraction", "cache_dir"]

_enabled: Optional[bool] = None
_lock = threading.Lock()
_loaded: dict = {}  # table hash -> ctypes handle (kept: the registered kernels live in the object)
_failed: set = set()

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"


def enable(on: bool = True) -> None:
    """Turn compilation at first use on or off for this process (overrides ``CUEQ_AMD_JIT``)."""
    global _enabled
    _enabled = bool(on)


def enabled() -> bool:
    if _enabled is not None:
        return _enabled
    return os.environ.get("CUEQ_AMD_JIT", "1") not in ("", "0", "false", "False")


def cache_dir() -> Path:
    root = os.environ.get("CUEQ_AMD_JIT_CACHE")
    base = Path(root) if root else Path.home() / ".cache" / "cuequivariance_amd"
    st = _lib.LIB_PATH.stat()
    build = hashlib.sha1(f"{_lib.LIB_PATH}:{st.st_size}:{st.st_mtime_ns}".encode()).hexdigest()[:12]
    d = base / f"jit-{build}"
    d.mkdir(parents=True, exist_ok=True)
    return d


def is_channelwise(t: U1dTables) -> bool:
    return (t.num_inputs == 3 and t.num_outputs == 1 and tuple(t.operations) == (0, 1, 2, 3) and tuple(t.buffer_dim) == (1, 1, 0, 1)
            and len(t.num_operands) == 1)


def _tuning(st, T: str) -> dict:
    """Wavefronts per SIMD, prefetching and the number of wavefronts the blocks are dealt out to, from a register
    estimate (accumulators + operand sets; doubles take two registers).  A descriptor whose kernels would be left with
    one wavefront per SIMD is split over two or four wavefronts with disjoint x1 segments when it has that many."""
    from .codegen import channelwise as cw

    per = 2 if T == "double" else 1
    most = len(cw._split_blocks(st, 4))

    def part(n, ns):
        return -(-n // ns)

    def fwd_regs(ns, sets):
        return (part(st.nseg_out, ns) + sets * (part(st.nseg_x1 + st.nseg_w, ns) + 4) + 30) * per

    def bwd_regs(ns):
        return (part(st.nseg_out, ns) + part(2 * st.nseg_x1 + st.nseg_w, ns) + st.nseg_x2 + 30) * per

    fwd = None
    for ns in (1, 2, 4):
        if ns > most:
            break
        if fwd_regs(ns, 2) <= 250:
            fwd = dict(fwd_split=ns, fwd_waves=2, fwd_prefetch=True)
        elif fwd_regs(ns, 1) <= 250:
            fwd = dict(fwd_split=ns, fwd_waves=2, fwd_prefetch=False)
        if fwd:
            break
    if fwd is None:
        fwd = dict(fwd_split=1, fwd_waves=1, fwd_prefetch=fwd_regs(1, 2) <= 500)
    bwd = dict(bwd_split=1, bwd_waves=1)
    for ns in (1, 2, 4):
        if ns > most:
            break
        if bwd_regs(ns) <= 250:
            bwd = dict(bwd_split=ns, bwd_waves=2)
            break
    return dict(fwd, **bwd)


_IO_NAME = {_lib.BF16: "bf16", _lib.F16: "f16"}  # element types of buffers that differ from the (float) arithmetic type


def _has_spec(t: U1dTables, code: int, io_code: Optional[int] = None) -> bool:
    """Whether kernels generated for these tables are registered with the library: for buffers of the arithmetic type
    ``code``, or of the 16-bit type ``io_code``."""
    desc, keep = _lib.make_desc(t, code)
    if io_code is None or io_code == code:
        return bool(_lib.load().cueq_u1d_desc_info(C.byref(desc), None))
    return bool(_lib.load().cueq_u1d_desc_serves(C.byref(desc), io_code))


def is_symmetric_contraction(poly) -> bool:
    """``w[u], x[u] (one to three times) -> out[u]`` in every operation, one uniform extent: the form
    ``codegen/symmetric.py`` generates kernels for."""
    if poly is None or poly.num_inputs != 2 or poly.num_outputs != 1 or not poly.operations:
        return False
    extents = {s for ope in poly.operands for s in ope.segments}
    if len(extents) != 1 or len(next(iter(extents))) != 1:
        return False
    for ope, stp in poly.operations:
        bufs = tuple(ope.buffers)
        if len(bufs) < 3 or len(bufs) > 5 or bufs[0] != 0 or bufs[-1] != 2 or any(b != 1 for b in bufs[1:-1]):
            return False
    return True


def is_row_weight_fully_connected(t: U1dTables, origin) -> bool:
    """Tables flattened from a fully connected product ``origin`` (``uvw,iu,jv,kw+ijk``, second operand of multiplicity one,
    one multiplicity per operand) - the form ``codegen/fullyconnected_rows.py`` generates kernels for when every batch row
    brings its own weights."""
    from .codegen import fullyconnected_rows as fcr

    if origin is None or t.layouts or t.num_inputs != 3 or t.num_outputs != 1 or tuple(t.buffer_dim) != (1, 0, 0, 1):
        return False
    st = fcr.analyze(origin)
    return (st is not None and t.operand_extent == st.Wd and
            list(t.buffer_num_segments) == [st.width_w // st.Wd, st.width_x1, st.width_x2, st.width_out // st.Wd])


def is_channelwise_with_harmonics(t: U1dTables, origin) -> bool:
    """Tables of ``cue.fused.channelwise_spherical`` (``origin``: its ``FusedHarmonics``): a channel-wise product whose second
    operand is the spherical harmonics of the 3-vector in buffer 2."""
    from .cue.fused import FusedHarmonics

    return (isinstance(origin, FusedHarmonics) and t.num_inputs == 3 and t.num_outputs == 1 and tuple(t.buffer_dim) == (1, 1, 0, 1)
            and t.buffer_num_segments[2] == 3 and not t.layout(0) and not t.layout(2))


def _family(t: U1dTables, polynomial=None, origin=None) -> Optional[str]:
    """The family generator that serves these tables: "channelwise" (which addresses x1 and the output through their
    layouts), "symmetric" (likewise for x and the output), "fc_rows" (a fully connected product with a weight row per batch row;
    ``origin`` is the polynomial the tables were flattened from) or None."""
    if is_channelwise_with_harmonics(t, origin):
        return "channelwise_sh"
    if is_channelwise(t) and not t.layout(0) and not t.layout(2):
        return "channelwise"
    if not t.layout(0) and is_symmetric_contraction(polynomial):
        return "symmetric"
    if is_row_weight_fully_connected(t, origin):
        return "fc_rows"
    return None


def has_fused_backward(t: U1dTables, polynomial=None, origin=None) -> bool:
    """Families whose unit computes every gradient in one pass over the operands (preferred over a kernel per gradient)."""
    return _family(t, polynomial, origin) in ("channelwise", "channelwise_sh", "fc_rows")


def ensure_plan(tables: U1dTables, math_code: int, root_tables: Optional[U1dTables] = None, root_polynomial=None,
                root_origin=None, io_code: Optional[int] = None) -> bool:
    """Kernels for one plan: first the family unit of its root (the forward plan of a channel-wise product or symmetric
    contraction holds the kernels of its backward plans too), then, if the plan still has none, a unit of its own from
    the general generator (``codegen/general.py``: second derivatives, harmonics, flattened dense products, ...).
    ``io_code``: the element type of the buffers when it is not the arithmetic type (bfloat16 / half with float arithmetic:
    a unit of its own per element type)."""
    if io_code == math_code:
        io_code = None
    if io_code is not None and (math_code != _lib.F32 or io_code not in _IO_NAME):
        return False
    if _has_spec(tables, math_code, io_code):
        return True
    if not enabled():
        return False
    if root_tables is not None and _family(root_tables, root_polynomial, root_origin):
        ensure_specialised(root_tables, math_code, root_polynomial, origin=root_origin, io_code=io_code)
        if _has_spec(tables, math_code, io_code):
            return True
    return ensure_specialised(tables, math_code, None, general=True, io_code=io_code)


def ensure_specialised(tables: U1dTables, math_code: int, polynomial=None, general: bool = False, origin=None,
                       io_code: Optional[int] = None) -> bool:
    """Make sure specialised kernels for ``tables`` (forward) and for its backward are registered with the library,
    compiling them if this module is enabled and the descriptor is a channel-wise product or (given the flattened
    ``polynomial`` the tables came from) a symmetric contraction - or, with ``general``, anything the general generator
    covers.  Returns whether they are."""
    from .codegen import general as gen

    if _has_spec(tables, math_code, io_code):
        return True
    family = _family(tables, polynomial, origin)
    if not enabled() or not (family or (general and gen.supported(tables))):
        return False
    if io_code is not None and family == "fc_rows":
        return False  # (that family is generated for buffers of the arithmetic type only)
    key = tables.content_hash(math_code)
    slot = key if io_code is None else (key, io_code)
    with _lock:
        if slot in _loaded or _has_spec(tables, math_code, io_code):
            return True
        if slot in _failed:
            return False
        try:
            _loaded[slot] = _build_and_load(tables, math_code, key, polynomial, origin, _IO_NAME.get(io_code))
        except Exception as e:  # compilation is an optimisation: the table-driven kernels still serve the plan
            _failed.add(slot)
            print(f"[cueq_amd.jit] specialised kernels for descriptor {key:016x} not built: {e}", file=sys.stderr, flush=True)
            return False
    return _has_spec(tables, math_code, io_code)


def _build_and_load(t: U1dTables, code: int, key: int, polynomial=None, origin=None, io: Optional[str] = None):
    from .codegen import channelwise as cw
    from .codegen import symmetric as sc

    T = "float" if code == _lib.F32 else "double"
    name = f"jit_{key:016x}"
    # the object's name carries a hash of the emitted source, so a changed generator (or tuning) never meets a stale object
    family = _family(t, polynomial, origin)
    if family is None:
        from .codegen import general as gen

        src = gen.emit_unit(t, T, name, key, io=io)
        what = f"general plan, {sum(t.num_paths)} paths, extent {t.operand_extent}"
    elif family == "channelwise":
        _, paths = t.operation(0)
        st = cw.analyze(t.operand_extent, t.buffer_num_segments, [(*idx, c) for idx, c in paths], t.layout(1), t.layout(3))
        tb = t.backward((True, True, True))
        src = cw.emit_unit(st, T, name, key, tb.content_hash(code), io=io, **_tuning(st, T))
        what = f"{st.num_paths} paths, extent {st.extent}"
    elif family == "channelwise_sh":
        tp = U1dTables.from_polynomial(origin.product)
        _, paths = tp.operation(0)
        st = cw.analyze(tp.operand_extent, tp.buffer_num_segments, [(*idx, c) for idx, c in paths], t.layout(1), t.layout(3), origin.terms)
        src = cw.emit_unit(st, T, name, key, t.backward((True, True, True)).content_hash(code), io=io, **_tuning(st, T))
        what = f"{st.num_paths} paths, extent {st.extent}, spherical harmonics of degrees {list(origin.ls)} in the kernels"
    elif family == "fc_rows":
        from .codegen import fullyconnected_rows as fcr

        st = fcr.analyze(origin)
        src = fcr.emit_unit(st, T, name, key, t.backward((True, True, True)).content_hash(code))
        what = f"fully connected, weights per row, {len(st.blocks)} blocks, U = {st.U}, W = {st.Wd}"
    else:
        st = sc.analyze(polynomial, t.layout(1), t.layout(2))
        bwd = {(dw, dx): t.backward((dw, dx)).content_hash(code) for dw, dx in ((True, True), (True, False), (False, True))}
        src = sc.emit_unit(st, T, name, key, bwd, io=io)
        what = f"symmetric contraction, {len(st.terms)} folded terms, extent {st.extent}"
    so = cache_dir() / f"u1d_{name}_{io or T}_{hashlib.sha1(src.encode()).hexdigest()[:10]}.so"
    if not so.exists():
        _compile(src, so, f"descriptor {key:016x} ({T}{', buffers of ' + io if io else ''}, {what})")
    _lib.load()  # the library the object links against is already in the process
    return C.CDLL(str(so))


def _compile(src: str, so: Path, what: str, link_library: bool = True) -> None:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    with tempfile.TemporaryDirectory(dir=so.parent) as tmp:
        hip = Path(tmp) / (so.stem + ".hip")
        hip.write_text(src)
        out = Path(tmp) / so.name
        cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-Wno-unused-command-line-argument", f"-I{INCLUDE}", f"-I{CSRC}", str(hip), "-o", str(out)]
        if link_library:
            cmd += [f"-L{_lib.LIB_PATH.parent}", f"-l:{_lib.LIB_PATH.name}", f"-Wl,-rpath,{_lib.LIB_PATH.parent}"]
        print(f"[cueq_amd.jit] compiling kernels for {what} ...", file=sys.stderr, flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed:\n{r.stderr[-2000:]}")
        os.replace(out, so)  # atomic: another process may be compiling the same descriptor


PREBUILT = Path(__file__).resolve().parent / "prebuilt"


def _starts(irreps) -> list:
    out, off = [], 0
    for mul, ir in irreps:
        out.append(off)
        off += mul * ir.dim
    return out


def prebuild_fully_connected(force: bool = False) -> list:
    """Compile the fused kernels of the fully connected products listed in ``codegen/registry.py`` into
    ``cuequivariance_amd/prebuilt/`` (called when the library is built; the objects are named by the hash of their
    source, so a changed generator never meets a stale object).  Returns the objects."""
    from . import cue, cuet
    from .codegen import fullyconnected as fc
    from .codegen import registry

    PREBUILT.mkdir(exist_ok=True)
    wanted = []
    for i1, i2, i3 in registry.FULLY_CONNECTED:
        m = cuet.FullyConnectedTensorProduct(cue.Irreps("O3", i1), cue.Irreps("O3", i2), cue.Irreps("O3", i3), layout=cue.ir_mul,
                                             internal_weights=False)
        dense = next(x for x in m.modules() if type(x).__name__ == "SegmentedPolynomialDense")
        # both row orders of the first operand and the output: ir_mul (the kernels' own) and mul_ir (the modules' default)
        mul_ir = ([(o, mul, ir.dim) for o, (mul, ir) in zip(_starts(m.irreps_in1), m.irreps_in1)],
                  [(o, mul, ir.dim) for o, (mul, ir) in zip(_starts(m.irreps_out), m.irreps_out)])
        for T in ("float", "uint16_t", "f16bits"):
            for blocks, tag in (((None, None), ""), (mul_ir, ", mul_ir rows")):
                src = fc.emit_unit(dense.paths, dense.input_sizes[2], dense.input_sizes[1], dense.out_size, T, *blocks)
                so = PREBUILT / f"fc_{hashlib.sha1(src.encode()).hexdigest()[:16]}_{T}.so"
                if force or not so.exists():
                    _compile(src, so, f"the fully connected product {i1} (x) {i2} -> {i3} ({T}{tag})", link_library=False)
                wanted.append(so)
    for old in PREBUILT.glob("fc_*.so"):
        if old not in wanted:
            old.unlink()
    return wanted


def fully_connected_unit(paths, n2: int, width_in: int, width_out: int, T: str, in_blocks=None, out_blocks=None):
    """The fused kernels of ``codegen/fullyconnected.py`` for one fully connected product and element type (``float`` or
    ``uint16_t`` for bfloat16), compiled at first use and loaded: a ``ctypes`` handle with ``fcj_fwd``, ``fcj_dx1``,
    ``fcj_dx2``, ``fcj_dx12`` (both input gradients in one pass; returns -2 for products it does not cover) and ``fcj_dw``, or ``None`` when this module is off, the product is outside what the generator covers, or the compiler
    failed (the caller then runs the table-driven GEMMs)."""
    from .codegen import fullyconnected as fc

    if not enabled() or not fc.supported(paths, n2, width_in, width_out, 4 if T == "float" else 2):
        return None
    src = fc.emit_unit(paths, n2, width_in, width_out, T, in_blocks, out_blocks)
    key = "fc_" + hashlib.sha1(src.encode()).hexdigest()[:16]
    with _lock:
        if key in _loaded:
            return _loaded[key]
        if key in _failed:
            return None
        try:
            so = PREBUILT / f"{key}_{T}.so"  # compiled with the library for the registered products
            if not so.exists():
                so = cache_dir() / f"{key}_{T}.so"
            if not so.exists():
                _compile(src, so, f"a fully connected product ({T}, {len(paths)} paths, {width_in} x {n2} -> {width_out})", link_library=False)
            h = C.CDLL(str(so))
            i64, vp = C.c_int64, C.c_void_p
            h.fcj_fwd.argtypes = [i64, vp, vp, i64, vp, i64, vp, i64, vp]
            h.fcj_dx1.argtypes = [i64, vp, vp, i64, vp, i64, vp, i64, vp]
            h.fcj_dx2.argtypes = [i64, vp, vp, i64, vp, i64, vp, i64, vp, i64, vp]
            h.fcj_dx12.argtypes = [i64, vp, vp, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, vp]
            h.fcj_dw_blocks.argtypes = [i64]
            h.fcj_dw.argtypes = [i64, vp, i64, vp, i64, vp, i64, vp, i64, vp]
            for f in (h.fcj_fwd, h.fcj_dx1, h.fcj_dx2, h.fcj_dx12, h.fcj_dw_blocks, h.fcj_dw):
                f.restype = C.c_int
            _loaded[key] = h
            return h
        except Exception as e:
            _failed.add(key)
            print(f"[cueq_amd.jit] fused fully connected kernels not built: {e}", file=sys.stderr, flush=True)
            return None
