"""``cueq_u1d_run_static`` (the entry point that allocates nothing) against ``cueq_u1d_run`` through the C ABI.

Two call shapes whose kernels need the workspace - the fused channel-wise backward (per-channel-half partials of the
x2 gradient) and a batch-reduced output on the table-driven kernels (per-chunk partial rows) - each run twice in a
row, the second time on a smaller input, so stale contents of the shared static array would show.  Both paths are
bit-reproducible, so the results are compared exactly (tighter than the 1e-5 * max|ref| bound of float32).
"""

import ctypes as C

import pytest
import torch

from cuequivariance_amd import _lib, cue
from cuequivariance_amd.codegen.registry import channelwise_tables
from cuequivariance_amd.tables import U1dTables

pytestmark = pytest.mark.gpu


def _plan(tables: U1dTables, math_code: int) -> C.c_void_p:
    lib = _lib.load()
    desc, keep = _lib.make_desc(tables, math_code)
    out = C.c_void_p()
    _lib.check(lib.cueq_u1d_plan_create(C.byref(desc), C.byref(out)), "cueq_u1d_plan_create")
    return out


def _buffers(tensors, modes):
    bufs = (_lib.U1dBuffer * len(tensors))()
    for b, (t, mode) in enumerate(zip(tensors, modes)):
        bufs[b].data = t.data_ptr()
        bufs[b].rows = t.shape[0]
        bufs[b].dtype = _lib.F32
        bufs[b].batch_dim = mode
    return bufs


def _run_both(plan, tables, inputs, modes, out_rows, batch):
    """Outputs of cueq_u1d_run (torch workspace) and cueq_u1d_run_static on the same inputs."""
    lib = _lib.load()
    dev = inputs[0].device
    nin = tables.num_inputs
    stream = torch.cuda.current_stream(dev).cuda_stream
    results = []
    for static in (False, True):
        outs = [torch.full((out_rows[o], tables.width(nin + o)), float("nan"), device=dev) for o in range(tables.num_outputs)]
        bufs = _buffers([*inputs, *outs], modes)
        need = lib.cueq_u1d_workspace_size(plan, bufs, batch)
        assert 0 < need <= lib.cueq_u1d_static_scratch_bytes()
        if static:
            # the entry point's contract: nothing is allocated - neither through torch nor underneath it
            torch.cuda.synchronize(dev)
            before = (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev), torch.cuda.mem_get_info(dev)[0])
            _lib.check(lib.cueq_u1d_run_static(plan, bufs, batch, stream), "cueq_u1d_run_static")
            torch.cuda.synchronize(dev)
            assert (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev), torch.cuda.mem_get_info(dev)[0]) == before
        else:
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
            _lib.check(lib.cueq_u1d_run(plan, bufs, batch, ws.data_ptr(), need, stream), "cueq_u1d_run")
        torch.cuda.synchronize(dev)
        results.append(outs)
    return results


def test_static_scratch_matches_workspace_run(device):
    lib = _lib.load()
    B, S = _lib.BATCH_DIM_BATCHED, _lib.BATCH_DIM_SHARED
    # (a) fused backward of the 128-channel, l <= 3 channel-wise product, every operand batched:
    #     inputs w, x1, x2, g -> outputs dw, dx1, dx2; the x2 gradient goes through per-channel-half partials
    fwd = channelwise_tables("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o")
    bwd = fwd.backward((True, True, True))
    plan_a = _plan(bwd, _lib.F32)
    assert lib.cueq_u1d_plan_info(plan_a, None) == 1, "generated kernels are not linked into the library"
    # (b) table-driven kernels, a batch-reduced (one-row) output: the weight gradient of a small product with shared
    #     weights, summed over more batch rows than one chunk holds
    small = channelwise_tables("8x0e+8x1o", "0e+1o", "0e+1o")
    bwd_w = small.backward((True, False, False))
    plan_b = _plan(bwd_w, _lib.F32)
    g = torch.Generator().manual_seed(5)
    try:
        for batch_a, batch_b in ((700, 9000), (130, 5000)):  # second round: smaller inputs
            ins = [torch.randn(batch_a, bwd.width(b), generator=g).to(device) for b in range(4)]
            ref, got = _run_both(plan_a, bwd, ins, [B] * 7, [batch_a] * 3, batch_a)
            for name, r, q in zip(("dw", "dx1", "dx2"), ref, got):
                assert not torch.isnan(q).any(), name
                assert torch.equal(r, q), f"fused backward {name}, batch {batch_a}"
            ins = [torch.randn(1 if b == 0 else batch_b, bwd_w.width(b), generator=g).to(device) for b in range(4)]
            ref, got = _run_both(plan_b, bwd_w, ins, [S, B, B, B, S], [1], batch_b)
            assert not torch.isnan(got[0]).any()
            assert torch.equal(ref[0], got[0]), f"batch-reduced output, batch {batch_b}"
        # recorded into a HIP graph (after the eager calls above, which looked the array's address up on this device):
        # every replay gives what the eager call gives
        batch_c = 300
        ins = [torch.randn(batch_c, bwd.width(b), generator=g).to(device) for b in range(4)]
        ref, _ = _run_both(plan_a, bwd, ins, [B] * 7, [batch_c] * 3, batch_c)
        outs = [torch.zeros(batch_c, bwd.width(4 + o), device=device) for o in range(3)]
        bufs_c = _buffers([*ins, *outs], [B] * 7)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                _lib.check(lib.cueq_u1d_run_static(plan_a, bufs_c, batch_c, torch.cuda.current_stream().cuda_stream), "cueq_u1d_run_static")
        torch.cuda.current_stream().wait_stream(side)
        for replay in range(3):
            for o in outs:
                o.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for name, r, q in zip(("dw", "dx1", "dx2"), ref, outs):
                assert torch.equal(r, q), f"graph replay {replay}: {name}"
        # beyond the static array: refused with a clear error, nothing launched
        batch = 400_000  # 400 000 rows x 2 halves x 16 floats = 51 MB of partials
        bufs = (_lib.U1dBuffer * 7)()
        for b in range(7):
            bufs[b].data = 4096
            bufs[b].rows = batch
            bufs[b].dtype = _lib.F32
            bufs[b].batch_dim = B
        assert lib.cueq_u1d_workspace_size(plan_a, bufs, batch) > lib.cueq_u1d_static_scratch_bytes()
        assert lib.cueq_u1d_run_static(plan_a, bufs, batch, None) == -4
        assert b"static array" in lib.cueq_last_error()
    finally:
        lib.cueq_u1d_plan_destroy(plan_a)
        lib.cueq_u1d_plan_destroy(plan_b)
