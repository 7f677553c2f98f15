"""The ``uniform_1d`` operator on MI355X: same call signature as the reference's closed op.

``uniform_1d(name, math_dtype, operand_extent, ..., batch_size, tensors)`` takes exactly the
21 positional arguments of ``torch.ops.cuequivariance.uniform_1d`` as called at
``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:55-77,294-316``
and returns the list of output tensors.  It differs from the reference in how it runs:

* the path tables are compiled once into a device-resident plan (``cueq_u1d_plan_create``);
* scatter into indexed outputs is a gather over rows grouped by output row (no atomics);
* backward is the same operator applied to the transposed tables (the path table is reused,
  only the roles of the buffers change, as in
  ``cuequivariance/cuequivariance/segmented_polynomials/segmented_polynomial.py:1003-1133``),
  so gradients of any order work.

Everything executes through the C ABI in ``libcueq_amd.so``; CPU tensors are rejected.
"""

from __future__ import annotations

import ctypes as C
import threading
import warnings
from collections import OrderedDict
from typing import List, Optional, Sequence

import torch

from .. import _lib
from .. import jit as _jit
from .._lib import BATCH_DIM_AUTO, BATCH_DIM_BATCHED, BATCH_DIM_INDEXED, BATCH_DIM_SHARED
from ..tables import U1dTables

__all__ = [
    "uniform_1d",
    "BATCH_DIM_AUTO",
    "BATCH_DIM_SHARED",
    "BATCH_DIM_BATCHED",
    "BATCH_DIM_INDEXED",
    "Uniform1dPlan",
]

_DTYPE_CODE = {
    torch.float32: _lib.F32,
    torch.float64: _lib.F64,
    torch.float16: _lib.F16,
    torch.bfloat16: _lib.BF16,
}


_traced_plans: "OrderedDict[str, Uniform1dPlan]" = OrderedDict()
_PLAIN_TENSORS = (torch.Tensor, torch.nn.Parameter)
_traced_lock = threading.Lock()
_DTYPE_BY_NAME = {"float32": torch.float32, "float64": torch.float64}


def _plan_by_key(key: str) -> "Uniform1dPlan":
    """The plan a traced graph names: the one that wrote the key while it is known here, else one built from the key (a
    graph saved by one process and loaded by another carries everything the plan is made of)."""
    with _traced_lock:
        plan = _traced_plans.get(key)
        if plan is not None:
            _traced_plans.move_to_end(key)
            return plan
    name, dtype_name, packed = key.split("|", 2)
    plan = _cached_plan(Uniform1dPlan(U1dTables.unpack(packed), _DTYPE_BY_NAME[dtype_name], name=name))
    _remember_traced(key, plan)
    return plan


def _remember_traced(key: str, plan: "Uniform1dPlan") -> None:
    with _traced_lock:
        _traced_plans[key] = plan
        while len(_traced_plans) > 256:
            _traced_plans.popitem(last=False)


class Uniform1dPlan:
    """Flat descriptor tables + lazily created device plans (one per GPU) + derived backward plans."""

    def __init__(self, tables: U1dTables, math_dtype: torch.dtype, name: str = "segmented_polynomial"):
        if math_dtype not in (torch.float32, torch.float64):
            raise ValueError(f"uniform_1d: math_dtype must be float32 or float64, got {math_dtype}")
        self.tables = tables
        self.name = name
        self.math_dtype = math_dtype
        self.widths = tuple(tables.width(b) for b in range(tables.num_inputs + tables.num_outputs))
        self._configs: dict = {}  # resolved call configurations by call shape
        self._handles: dict[int, int] = {}
        self._backward: dict[tuple, "Uniform1dPlan"] = {}
        self._choice: dict = {}
        self._io_seen: set = set()  # 16-bit element types whose kernels were looked for (and compiled, when that is on)
        self.jit_root = None  # for a backward plan: the forward plan, whose translation unit holds its kernels
        self.polynomial = None  # the flattened polynomial the tables came from, when the caller has it
        self.origin = None      # the polynomial that one was flattened from (a fully connected product's descriptor)
        self._lock = threading.Lock()
        # under this text a traced graph (torch.compile, torch.export, torch.jit.trace) names the plan: operator name,
        # arithmetic type and the packed tables, so that a saved graph stays valid where this object does not exist
        self.traced_key = f"{name.replace('|', '/')}|{str(math_dtype).split('.')[-1]}|{tables.pack()}"
        _remember_traced(self.traced_key, self)

    def __getattr__(self, item):
        # table fields (operand_extent, num_inputs, buffer_dim, ...) read through
        if item == "tables":
            raise AttributeError(item)
        return getattr(self.tables, item)

    # ------------------------------------------------------------------ geometry
    def width(self, b: int) -> int:
        return self.tables.width(b)

    def key(self) -> tuple:
        return (self.math_dtype, self.tables)


    def specialised(self, device: torch.device) -> bool:
        """True when kernels generated for exactly these tables are linked into the library."""
        h = self.handle(device)
        return bool(_lib.load().cueq_u1d_plan_info(h, None))

    # ------------------------------------------------------------------ device plan
    def handle(self, device: torch.device) -> int:
        idx = device.index if device.index is not None else torch.cuda.current_device()
        h = self._handles.get(idx)
        if h is not None:
            return h
        with self._lock:
            h = self._handles.get(idx)
            if h is not None:
                return h
            lib = _lib.load()
            if _jit.enabled():  # kernels generated for this descriptor at first use (off by default)
                root = self.jit_root or self
                _jit.ensure_plan(self.tables, _DTYPE_CODE[self.math_dtype], root.tables, root.polynomial, root.origin)
            desc, keep = _lib.make_desc(self.tables, _DTYPE_CODE[self.math_dtype])
            out = C.c_void_p()
            with torch.cuda.device(idx):
                _lib.check(lib.cueq_u1d_plan_create(C.byref(desc), C.byref(out)), "cueq_u1d_plan_create")
            self._handles[idx] = out.value
            if (not _jit.enabled() and self.jit_root is None and not lib.cueq_u1d_plan_info(out.value, None)
                    and (_jit.is_channelwise(self.tables) or _jit.is_symmetric_contraction(self.polynomial))):
                warnings.warn(
                    f"uniform_1d[{self.name}]: no specialised kernels are built for this descriptor, the "
                    "table-driven kernels (20 to 100 times slower on large workloads) will run; compilation at first use is switched "
                    "off (CUEQ_AMD_JIT=0 / cuequivariance_amd.jit.enable(False))",
                    stacklevel=2)
            return out.value

    def ensure_io(self, dtype: torch.dtype) -> None:
        """Kernels for buffers that all hold the 16-bit ``dtype`` while the arithmetic is float32: a unit of their own, linked
        into the library for the registered descriptors, compiled at first use for others (when that is switched on).  The
        device plans find such a unit as soon as it is registered."""
        if self.math_dtype != torch.float32 or dtype not in (torch.bfloat16, torch.float16) or dtype in self._io_seen:
            return
        with self._lock:
            if dtype not in self._io_seen:
                if _jit.enabled():
                    root = self.jit_root or self
                    _jit.ensure_plan(self.tables, _DTYPE_CODE[self.math_dtype], root.tables, root.polynomial, root.origin,
                                     io_code=_DTYPE_CODE[dtype])
                self._io_seen.add(dtype)

    def serves(self, dtype: torch.dtype) -> bool:
        """True when kernels generated for exactly these tables and buffers of ``dtype`` are registered with the library."""
        return _jit._has_spec(self.tables, _DTYPE_CODE[self.math_dtype], _DTYPE_CODE[dtype])

    def __del__(self):
        try:
            lib = _lib.load()
            for h in self._handles.values():
                lib.cueq_u1d_plan_destroy(h)
        except Exception:
            pass

    # ------------------------------------------------------------------ transposition
    def backward_plan(self, needs_grad: tuple) -> "Uniform1dPlan":
        """Plan computing the gradients of the flagged inputs (see ``U1dTables.backward``)."""
        needs_grad = tuple(bool(x) for x in needs_grad)
        plan = self._backward.get(needs_grad)
        if plan is None:
            plan = Uniform1dPlan(self.tables.backward(needs_grad), self.math_dtype, name=self.name + "_bwd")
            plan.jit_root = self if self.jit_root is None else None
            self._backward[needs_grad] = plan
        return plan


def _backward_choice(plan: Uniform1dPlan, needs: tuple, device: torch.device) -> tuple:
    """The gradient plan to run for ``needs``: the exact one when it has specialised kernels (or nothing better exists),
    else the plan for all inputs when that one has them - computing a gradient nobody asked for costs far less than
    leaving the specialised kernels.  Returns ``(plan, needs it computes)``; remembered per plan."""
    key = (needs, device.index)
    hit = plan._choice.get(key)
    if hit is None:
        exact = plan.backward_plan(needs)
        hit = (exact, needs)
        if not all(needs) and device.type == "cuda":
            everything = (True,) * len(needs)
            full = plan.backward_plan(everything)
            if _jit.has_fused_backward(plan.tables, plan.polynomial, plan.origin):
                # the fused backward of the family reads every operand once for all three gradients: preferred over a
                # unit per gradient from the general generator
                if full.specialised(device):
                    hit = (full, everything)
            elif not exact.specialised(device) and full.specialised(device):
                hit = (full, everything)
        plan._choice[key] = hit
    return hit


_plan_cache: "OrderedDict[tuple, Uniform1dPlan]" = OrderedDict()
_plan_cache_lock = threading.Lock()


_seam_plans: dict = {}  # argument lists of ``uniform_1d`` (as tuples) -> plan


def _cached_plan(plan: Uniform1dPlan) -> Uniform1dPlan:
    k = plan.key()
    with _plan_cache_lock:
        hit = _plan_cache.get(k)
        if hit is not None:
            _plan_cache.move_to_end(k)
            return hit
        _plan_cache[k] = plan
        while len(_plan_cache) > 256:
            _plan_cache.popitem(last=False)
        return plan


# ---------------------------------------------------------------------- CSR cache
_csr_cache: "OrderedDict[tuple, tuple]" = OrderedDict()


def _segment_csr(index: torch.Tensor, nrows: int):
    """(offsets[nrows+1], perm[n]) grouping batch ids by output row.

    Eager mode: built once per index tensor and cached (the build checks on the host that the ids are in range and
    skips the sort when they are sorted already).  While the current stream is being captured into a HIP graph the
    grouping is recorded into the graph instead (device-side work only, nothing cached), so every replay regroups from
    whatever the index buffer holds then.  Index tensors made under ``torch.inference_mode()`` carry no version counter
    and are not cached either."""
    lib = _lib.load()
    n = index.numel()
    capturing = torch.cuda.is_current_stream_capturing()
    cacheable = not capturing and not index.is_inference()
    if cacheable:
        key = (index.data_ptr(), index._version, n, int(nrows), index.dtype, index.device)
        hit = _csr_cache.get(key)
        if hit is not None:
            _csr_cache.move_to_end(key)
            return hit[1], hit[2]
    offsets = torch.empty(nrows + 1, dtype=torch.int64, device=index.device)
    perm = torch.empty(max(n, 1), dtype=torch.int64, device=index.device)
    ws_bytes = lib.cueq_segment_csr_workspace(n, nrows)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=index.device)
    stream = torch.cuda.current_stream(index.device).cuda_stream
    build = lib.cueq_segment_csr_build_async if capturing else lib.cueq_segment_csr_build
    _lib.check(
        build(index.data_ptr(), 1 if index.dtype == torch.int64 else 0, n, nrows,
              offsets.data_ptr(), perm.data_ptr(), ws.data_ptr(), ws_bytes, stream),
        "cueq_segment_csr_build",
    )
    if cacheable:
        # the index tensor is kept alive with the entry so its address cannot be reused meanwhile
        _csr_cache[key] = (index, offsets, perm)
        while len(_csr_cache) > 32:
            _csr_cache.popitem(last=False)
    return offsets, perm


# ---------------------------------------------------------------------- execution
class _CallConfig:
    """Resolved batching of one call: per buffer the mode, the index tensor slot and the row count.  Also holds what the
    launches of this call shape reuse: prepared argument records (by dtype signature) and the configurations of its
    backward calls."""

    __slots__ = ("modes", "index_of", "rows", "batch", "records", "backward")

    def __init__(self, modes, index_of, rows, batch):
        self.modes = tuple(modes)
        self.index_of = tuple(index_of)
        self.rows = tuple(rows)
        self.batch = int(batch)
        self.records: dict = {}
        self.backward: dict = {}

    def backward_config(self, computed: tuple) -> "_CallConfig":
        """The configuration of the gradient call for the inputs flagged in ``computed`` (its outputs are their gradients)."""
        hit = self.backward.get(computed)
        if hit is None:
            flagged = [i for i, n in enumerate(computed) if n]
            hit = self.backward[computed] = _CallConfig(
                list(self.modes) + [self.modes[i] for i in flagged], list(self.index_of) + [self.index_of[i] for i in flagged],
                list(self.rows) + [self.rows[i] for i in flagged], self.batch)
        return hit


class _LaunchRecord:
    """The argument array of ``cueq_u1d_run`` for one call shape and dtype signature, with every field that does not change
    from call to call filled in once; a launch writes the data / index / grouping pointers only."""

    __slots__ = ("bufs", "proxies", "out_dtypes")

    def __init__(self, plan: "Uniform1dPlan", cfg: _CallConfig, in_dtypes, idx_dtypes):
        nin, nout = plan.num_inputs, plan.num_outputs
        self.bufs = (_lib.U1dBuffer * (nin + nout))()
        self.proxies = [self.bufs[b] for b in range(nin + nout)]  # (one ctypes proxy per buffer, made once)
        self.out_dtypes = []
        for b in range(nin + nout):
            bb = self.proxies[b]
            if b < nin:
                dtype = in_dtypes[b]
                if dtype not in _DTYPE_CODE:
                    raise ValueError(f"uniform_1d: unsupported dtype {dtype} for input {b}")
            else:
                src = plan.dtypes[b]
                dtype = plan.math_dtype if src < 0 else in_dtypes[src]
                self.out_dtypes.append(dtype)
            bb.rows = cfg.rows[b]
            bb.dtype = _DTYPE_CODE[dtype]
            bb.batch_dim = cfg.modes[b]
            if cfg.modes[b] == BATCH_DIM_INDEXED:
                bb.index_is_64 = 1 if idx_dtypes[cfg.index_of[b]] == torch.int64 else 0


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device: torch.device):
    """Context that makes ``device`` current; nothing to do (and nothing to pay) when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _launch(plan: Uniform1dPlan, cfg: _CallConfig, inputs: Sequence[torch.Tensor],
            indices: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    nin, nout = plan.num_inputs, plan.num_outputs
    device = inputs[0].device if nin else indices[0].device
    if device.type != "cuda":
        raise RuntimeError("uniform_1d runs on the GPU only; got tensors on " + str(device))
    lib = _lib.load()
    _lib.sync_options_from_env()
    sig = (tuple([t.dtype for t in inputs]), tuple([i.dtype for i in indices]))
    pool = cfg.records.get(sig)
    if pool is None:
        pool = cfg.records[sig] = []
    try:
        rec = pool.pop()  # (a record is used by one launch at a time: list.pop / append are atomic)
    except IndexError:
        rec = _LaunchRecord(plan, cfg, sig[0], sig[1])
        if nin and sig[0][0].itemsize == 2 and all(d == sig[0][0] for d in sig[0]):
            plan.ensure_io(sig[0][0])
    modes, widths = cfg.modes, plan.widths
    with _on_device(device):
        handle = plan._handles.get(device.index)
        if handle is None:
            handle = plan.handle(device)
        proxies = rec.proxies
        keep = []
        for b in range(nin):
            t = inputs[b]
            if t.dim() != 2 or t.shape[1] != widths[b]:
                raise ValueError(f"uniform_1d: input {b} has shape {tuple(t.shape)}, expected (rows, {widths[b]})")
            if not t.is_contiguous():
                t = t.contiguous()
                keep.append(t)
            bb = proxies[b]
            bb.data = t.data_ptr()
            if modes[b] == BATCH_DIM_INDEXED:
                bb.index = indices[cfg.index_of[b]].data_ptr()
        outputs = []
        for o in range(nout):
            b = nin + o
            out = torch.empty((cfg.rows[b], widths[b]), dtype=rec.out_dtypes[o], device=device)
            outputs.append(out)
            bb = proxies[b]
            bb.data = out.data_ptr()
            if modes[b] == BATCH_DIM_INDEXED:
                idx = indices[cfg.index_of[b]]
                bb.index = idx.data_ptr()
                offsets, perm = _segment_csr(idx, cfg.rows[b])
                keep += [offsets, perm]
                bb.csr_offsets = offsets.data_ptr()
                bb.csr_perm = perm.data_ptr()
        ws_bytes = lib.cueq_u1d_workspace_size(handle, rec.bufs, cfg.batch)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=device) if ws_bytes > 0 else None
        stream = torch._C._cuda_getCurrentRawStream(device.index if device.index is not None else torch.cuda.current_device())
        status = lib.cueq_u1d_run(handle, rec.bufs, cfg.batch, ws.data_ptr() if ws is not None else None, ws_bytes, stream)
        if status != 0:
            _lib.check(status, f"cueq_u1d_run[{plan.name}]")
    pool.append(rec)
    return outputs


class _Uniform1dFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, plan: Uniform1dPlan, cfg: _CallConfig, num_index: int, *tensors):
        nin = plan.num_inputs
        inputs, indices = tensors[:nin], tensors[nin: nin + num_index]
        ctx.plan, ctx.cfg, ctx.num_index = plan, cfg, num_index
        ctx.save_for_backward(*tensors)
        outs = _launch(plan, cfg, [t.detach() for t in inputs], indices)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grad_outputs):
        plan, cfg, num_index = ctx.plan, ctx.cfg, ctx.num_index
        nin, nout = plan.num_inputs, plan.num_outputs
        tensors = ctx.saved_tensors
        inputs, indices = tensors[:nin], tensors[nin:]
        needs = tuple(ctx.needs_input_grad[3: 3 + nin])
        if not any(needs):
            return (None,) * (3 + len(tensors))
        bplan, computed = _backward_choice(plan, needs, inputs[0].device)
        cots = []
        for o, g in enumerate(grad_outputs):
            b = nin + o
            if g is None:
                src = plan.dtypes[b]
                g = torch.zeros((cfg.rows[b], plan.width(b)), device=inputs[0].device,
                                dtype=plan.math_dtype if src < 0 else inputs[src].dtype)
            cots.append(g)
        flagged = [i for i, n in enumerate(computed) if n]
        bcfg = cfg.backward_config(computed)
        if torch.is_grad_enabled():  # (create_graph: the gradient call is recorded, derivatives of any order)
            grads = _Uniform1dFunction.apply(bplan, bcfg, num_index, *inputs, *cots, *indices)
        else:
            grads = _launch(bplan, bcfg, [t.detach() for t in inputs] + cots, indices)
        out = [None, None, None] + [None] * len(tensors)
        for g, i in zip(grads, flagged):
            if needs[i]:
                out[3 + i] = g
        return tuple(out)


# ---------------------------------------------------------------------- traced execution
# Under torch.compile / torch.export the launch is one opaque operator (the Python above it - resolving batch modes
# and row counts - is traced as ordinary integer arithmetic); eager calls keep the lighter autograd.Function path.
@torch.library.custom_op("cuequivariance_amd::u1d_launch", mutates_args=(), device_types="cuda")
def _u1d_launch_op(plan_key: str, modes: List[int], index_of: List[int], rows: List[int], batch: int,
                   tensors: List[torch.Tensor]) -> List[torch.Tensor]:
    plan = _plan_by_key(plan_key)
    nin = plan.num_inputs
    outs = _launch(plan, _CallConfig(modes, index_of, rows, batch), [t.detach() for t in tensors[:nin]], tensors[nin:])
    return list(outs)


@_u1d_launch_op.register_fake
def _u1d_launch_fake(plan_key, modes, index_of, rows, batch, tensors):
    plan = _plan_by_key(plan_key)
    nin = plan.num_inputs
    outs = []
    for o in range(plan.num_outputs):
        src = plan.dtypes[nin + o]
        outs.append(tensors[0].new_empty((rows[nin + o], plan.width(nin + o)), dtype=plan.math_dtype if src < 0 else tensors[src].dtype))
    return outs


def _u1d_setup_context(ctx, inputs, output):
    plan_key, modes, index_of, rows, batch, tensors = inputs
    ctx.meta = (plan_key, tuple(modes), tuple(index_of), tuple(rows), batch)
    ctx.save_for_backward(*tensors)


def _u1d_backward(ctx, grad_outputs):
    plan_key, modes, index_of, rows, batch = ctx.meta
    plan = _plan_by_key(plan_key)
    nin = plan.num_inputs
    tensors = ctx.saved_tensors
    inputs, indices = tensors[:nin], tensors[nin:]
    flags = ctx.needs_input_grad[5]
    if isinstance(flags, bool):
        flags = [flags] * len(tensors)
    needs = tuple(bool(f) for f in flags[:nin])
    grads: List[Optional[torch.Tensor]] = [None] * len(tensors)
    if any(needs):
        bplan, computed = _backward_choice(plan, needs, inputs[0].device)
        cots = []
        for o, g in enumerate(grad_outputs):
            if g is None:
                src = plan.dtypes[nin + o]
                g = torch.zeros((rows[nin + o], plan.width(nin + o)), device=inputs[0].device,
                                dtype=plan.math_dtype if src < 0 else inputs[src].dtype)
            cots.append(g)
        flagged = [i for i, n in enumerate(computed) if n]
        got = _u1d_launch_op(bplan.traced_key, list(modes) + [modes[i] for i in flagged], list(index_of) + [index_of[i] for i in flagged],
                             list(rows) + [rows[i] for i in flagged], batch, [*inputs, *cots, *indices])
        for g, i in zip(got, flagged):
            if needs[i]:
                grads[i] = g
    return None, None, None, None, None, grads


torch.library.register_autograd("cuequivariance_amd::u1d_launch", _u1d_backward, setup_context=_u1d_setup_context)


def run_plan(plan: Uniform1dPlan, batch_dim: Sequence[int], index_buffer: Sequence[int], batch_size: int,
             num_index: int, tensors: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """Resolve AUTO batch dims and sizes (same rules as the reference op's caller) and execute."""
    nin, nout = plan.num_inputs, plan.num_outputs
    if len(tensors) != nin + num_index:
        raise ValueError(f"uniform_1d: expected {nin} inputs + {num_index} index tensors, got {len(tensors)}")
    inputs, indices = list(tensors[:nin]), list(tensors[nin:])
    for k, idx in enumerate(indices):
        if idx.dtype not in (torch.int32, torch.int64) or idx.dim() != 1:
            raise ValueError(f"uniform_1d: index tensor {k} must be a 1-D int32/int64 tensor")
        if not idx.is_contiguous():
            indices[k] = idx.contiguous()
    # the resolution below depends on these numbers only: resolved once per call shape
    key = (tuple(batch_dim), tuple(index_buffer), batch_size, tuple([t.shape[0] for t in inputs]), tuple([i.shape[0] for i in indices]))
    cfg = plan._configs.get(key) if not torch.compiler.is_compiling() else None
    if cfg is not None and inputs and type(inputs[0]) in _PLAIN_TENSORS:
        return list(_Uniform1dFunction.apply(plan, cfg, num_index, *inputs, *indices))
    modes = list(batch_dim)
    batch = batch_size
    # batch size: the common length of index tensors and of batched (multi-row) inputs
    candidates = [idx.shape[0] for idx in indices]
    for b in range(nin):
        if modes[b] == BATCH_DIM_INDEXED:
            continue
        r = inputs[b].shape[0]
        if modes[b] == BATCH_DIM_BATCHED or (modes[b] == BATCH_DIM_AUTO and r != 1):
            candidates.append(r)
    if batch == BATCH_DIM_AUTO:
        batch = candidates[0] if candidates else 1
    for c in candidates:
        if c != batch:
            raise ValueError(f"uniform_1d: inconsistent batch sizes {sorted(set(candidates + [batch]))}")
    rows = [0] * (nin + nout)
    for b in range(nin):
        rows[b] = inputs[b].shape[0]
        if modes[b] == BATCH_DIM_AUTO:
            modes[b] = BATCH_DIM_SHARED if (rows[b] == 1 and batch != 1) else BATCH_DIM_BATCHED
        if modes[b] == BATCH_DIM_BATCHED and rows[b] == 1 and batch != 1:
            modes[b] = BATCH_DIM_SHARED
        if modes[b] == BATCH_DIM_INDEXED:
            assert index_buffer[b] >= 0
    for o in range(nout):
        b = nin + o
        if modes[b] == BATCH_DIM_INDEXED:
            rows[b] = int(index_buffer[nin + nout + index_buffer[b]])
        elif modes[b] == BATCH_DIM_SHARED:
            rows[b] = 1
        else:
            modes[b] = BATCH_DIM_BATCHED
            rows[b] = batch
    # (traced: under Dynamo, or called with the tracer's tensor subclasses when a composite operator is decomposed)
    if torch.jit.is_tracing():  # (the tracer hands out sizes as tensors: row counts become constants of the trace)
        rows, batch = [int(r) for r in rows], int(batch)
    if torch.compiler.is_compiling() or torch.jit.is_tracing() or (inputs and type(inputs[0]) not in _PLAIN_TENSORS):
        return list(_u1d_launch_op(plan.traced_key, modes, list(index_buffer[: nin + nout]), rows, batch, [*inputs, *indices]))
    cfg = _CallConfig(modes, list(index_buffer[: nin + nout]), rows, batch)
    if len(plan._configs) >= 64:  # (call shapes of a module are few; a stream of ever new batch sizes starts over)
        plan._configs.clear()
    plan._configs[key] = cfg
    outs = _Uniform1dFunction.apply(plan, cfg, num_index, *inputs, *indices)
    return list(outs)


def uniform_1d(
    name: str,
    math_dtype: torch.dtype,
    operand_extent: int,
    num_inputs: int,
    num_outputs: int,
    num_index: int,
    buffer_dim: List[int],
    buffer_num_segments: List[int],
    batch_dim: List[int],
    index_buffer: List[int],
    dtypes: List[int],
    num_operations: int,
    num_operands: List[int],
    operations: List[int],
    num_paths: List[int],
    path_indices_start: List[int],
    path_coefficients_start: List[int],
    path_indices: List[int],
    path_coefficients: List[float],
    batch_size: int,
    tensors: List[torch.Tensor],
) -> List[torch.Tensor]:
    """Drop-in for ``torch.ops.cuequivariance.uniform_1d`` (argument meaning unchanged).

    ``tensors`` = the inputs followed by the index tensors; ``index_buffer`` maps every buffer to
    its index tensor (or -1) and then lists, per index tensor, the row count of the buffer it
    addresses; ``dtypes[num_inputs + k]`` names the input whose dtype output ``k`` inherits
    (-1: the math dtype).  Differentiable to any order.
    """
    if len(num_operands) != num_operations:
        raise ValueError("uniform_1d: num_operations does not match num_operands")
    # the frontend passes the same lists on every call: the plan is looked up by their values (tuples hash in a few
    # microseconds; building and hashing the tables takes a hundred and more for a few hundred paths)
    key = (name, math_dtype, operand_extent, num_inputs, num_outputs, tuple(buffer_dim), tuple(buffer_num_segments), tuple(dtypes),
           tuple(num_operands), tuple(operations), tuple(num_paths), tuple(path_indices_start), tuple(path_coefficients_start),
           tuple(path_indices), tuple(path_coefficients))
    plan = _seam_plans.get(key)
    if plan is None:
        plan = _cached_plan(
            Uniform1dPlan(
                U1dTables.make(
                    operand_extent, num_inputs, num_outputs, buffer_dim, buffer_num_segments, dtypes, num_operands,
                    operations, num_paths, path_indices_start, path_coefficients_start, path_indices, path_coefficients,
                ),
                math_dtype,
                name=name,
            )
        )
        with _plan_cache_lock:
            if len(_seam_plans) >= 256:
                _seam_plans.pop(next(iter(_seam_plans)))
            _seam_plans[key] = plan
    return run_plan(plan, batch_dim, index_buffer, batch_size, num_index, tensors)
