#!/usr/bin/env python3
"""Benchmark of the segmented-polynomial hot path on one MI355X.

Workload (BASELINE.json configs[1]): MACE-style indexed edge convolution -- channel-wise tensor
product of gathered node features ``128x0e+128x1o+128x2e+128x3o`` (5 000 nodes) with spherical
harmonics ``0e+1o+2e+3o`` of 100 000 random unit edge vectors and per-edge weights ``[E, 2944]``,
scatter-summed onto the 5 000 receiver nodes (receivers sorted, int32 indices); one step is the
forward pass plus the backward pass for the gradients of node features, edge attributes and weights.

Prints ONE JSON line: whole-job edges/s with inputs resident in HBM, the roofline position of the
dominant kernel (fused backward) from HIP-event timings taken inside the timed region, and the CPU
oracle timed on a bounded sample of the same workload on this box's host cores.  Run without
``--workload`` the line also carries a ``secondary`` object: the same workload in float64 and with the
ordered (bit-reproducible) node-gradient sum, and every other BASELINE.json configuration (channel-wise
batch 4096, symmetric contraction, Linear and fully connected product in fp32 / bf16, triangle update in
bf16 / fp32), each with its step time, throughput, both roofline fractions (algorithmic bytes against
8 TB/s; flops against the matrix-core or vector peak) and the binding roof, plus CPU baselines of the
dense workloads and the one-thread figure of the headline workload.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# published dense peaks, TFLOP/s: matrix cores per input type, and the fp32 vector units
MFMA_PEAK = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}
_DTYPES = {"bf16": "bfloat16", "fp16": "float16", "fp32": "float32", None: "float32"}
_DT_NAME = {"bfloat16": "bf16", "float16": "f16", "float32": "f32"}
VALU_PEAK_F32 = 157.3

# Bytes that left the L2 per launch at the default workload (5000 nodes, 100000 edges, fp32), from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE; KiB per dispatch) scaled by what the same
# counters read for a 1 GiB copy (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000).  Not measurable from inside this
# process: the figures are those of the profile named in TRAFFIC_SOURCE, taken with these kernels.
TRAFFIC_SOURCE = "profiles/channelwise_c128_l3_fp32_cfg2_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this command, not of this run)"
MEASURED_TRAFFIC_BYTES = {
    ("c128_l3_bwd_float", 5000, 100_000): 4.270e9,
    ("c128_l3_fwd_float", 5000, 100_000): 2.143e9,
}

# What the memory system of this part delivers to kernels of the access shape used here (64-thread workgroups, a dword per
# lane and instruction; `python bench.py --calibrate`, profiles/memory_system_calibration.txt): a read stream, a copy (bytes
# read + written) and float atomic adds.  With the measured traffic above they give the least time this decomposition of the
# headline step can take: forward = its L2-miss traffic at the read rate; backward = the longer of its 2.05e8 atomic adds
# (edges x 2048 values of the node gradient) at the atomic rate and its L2-miss traffic at the copy rate.
CAL_READ_BPS, CAL_COPY_BPS, CAL_ATOMIC_ADDS_PER_S = 7.09e12, 5.81e12, 3.2e11
CAL_SOURCE = ("profiles/memory_system_calibration.txt (read 7.09 TB/s, copy 5.81 TB/s, 3.2e11 float atomic adds/s) with the traffic of "
              "profiles/channelwise_c128_l3_fp32_cfg2_hbm_traffic.txt")


def design_ceiling(N: int, E: int, alg: dict):
    """Least times (s) of forward and backward of the default headline workload for this decomposition on this part, or None."""
    f, b = MEASURED_TRAFFIC_BYTES.get(("c128_l3_fwd_float", N, E)), MEASURED_TRAFFIC_BYTES.get(("c128_l3_bwd_float", N, E))
    if f is None or b is None:
        return None
    return {"fwd": f / CAL_READ_BPS, "bwd": max(E * 2048 / CAL_ATOMIC_ADDS_PER_S, b / CAL_COPY_BPS)}


# Vector (wave64) instructions the generated kernels execute per batch element (sample, edge, node), forward and backward,
# counted with rocprofv3 --pmc SQ_INSTS_VALU over one launch each and divided by the batch size (summary and command:
# profiles/uniform1d_fp32_valu_instruction_counts.txt).  A wave64 instruction is at most 64 fused multiply-adds =
# 128 flops, and the published fp32 vector peak (157.3 TFLOP/s) is one such instruction per SIMD every two clocks, so
# instructions x 128 / time against that peak is the issue utilisation of the vector units.
VALU_INSTS_PER_ELEMENT = {"cfg1": (242, 376), "cfg2": (1020, 2510), "cfg3": (1734, 4180)}
VALU_SOURCE = "profiles/uniform1d_fp32_valu_instruction_counts.txt (rocprofv3 --pmc SQ_INSTS_VALU of an earlier run of these kernels)"


def algorithmic_bytes(E: int, N: int, W: int, D1: int, D2: int, D3: int, s: int) -> dict:
    """Compulsory traffic: every distinct input element read once, every output element written once."""
    fwd = E * (W + D2) * s + 2 * E * 4 + N * D1 * s + N * D3 * s
    bwd = 2 * E * (W + D2) * s + 2 * E * 4 + 2 * N * D1 * s + N * D3 * s
    return {"fwd": fwd, "bwd": bwd}


def make_inputs(torch, cue, N: int, E: int, dtype, seed: int = 0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    node = torch.randn(N, 2048, dtype=torch.float64, generator=g)
    vec = torch.randn(E, 3, dtype=torch.float64, generator=g)
    vec = vec / vec.norm(dim=1, keepdim=True)
    sh = torch.from_numpy(cue.descriptors.spherical_harmonics_values(cue.O3(1, -1), [0, 1, 2, 3], vec.numpy()))
    w = torch.randn(E, 2944, dtype=torch.float64, generator=g)
    senders = torch.randint(0, N, (E,), generator=g, dtype=torch.int32)
    receivers = torch.randint(0, N, (E,), generator=g, dtype=torch.int32)
    order = torch.sort(receivers, stable=True)[1]
    senders, receivers = senders[order].contiguous(), receivers[order].contiguous()
    cot = torch.randn(N, 12672, dtype=torch.float64, generator=g)
    return node.to(dtype), sh.to(dtype), w.to(dtype), senders, receivers, cot.to(dtype)


def cpu_baseline(torch, cue, module, host, sample_edges: int, sample_nodes: int, threads: int = 0) -> dict:
    """The CPU oracle (restatement of the reference's PyTorch executor) on a slice of the same inputs."""
    from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

    node, sh, w, senders, receivers, cot = host
    cores = threads if threads > 0 else min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    spec = spec_from_polynomial(module.f._polynomial_orig)
    # a contiguous slice of edges (receivers stay sorted) with indices folded into the first sample_nodes rows
    snd = (senders[:sample_edges] % sample_nodes).contiguous()
    rcv = (receivers[:sample_edges] % sample_nodes).contiguous()
    rcv = torch.sort(rcv)[0]

    def once():
        a = [w[:sample_edges].clone().requires_grad_(True), node[:sample_nodes].clone().requires_grad_(True),
             sh[:sample_edges].clone().requires_grad_(True)]
        t0 = time.perf_counter()
        out = naive_segmented_polynomial(spec, a, {1: snd}, {0: sample_nodes}, {0: rcv})[0]
        torch.autograd.grad(out, a, cot[:sample_nodes])
        return time.perf_counter() - t0

    once()
    times = [once() for _ in range(3)]
    t = statistics.median(times)
    return {
        "value": sample_edges / t,
        "unit": "edges/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{sample_edges} edges onto {sample_nodes} nodes of the same workload, fwd+bwd, "
                  f"{node.dtype}, median of 3 after 1 warm-up ({t:.2f} s each)".replace("torch.", ""),
    }


def _roofs(bytes_, flops, seconds, flop_peak_tflops, flop_roof: str) -> dict:
    """Position of a measured time against both roofs; the binding roof is the one whose minimum time is longer."""
    hbm = bytes_ / seconds / 1e9 / HBM_PEAK_GBS
    cmp_ = flops / seconds / 1e12 / flop_peak_tflops if flops else 0.0
    t_hbm, t_cmp = bytes_ / (HBM_PEAK_GBS * 1e9), (flops / (flop_peak_tflops * 1e12) if flops else 0.0)
    bound = "hbm" if t_hbm >= t_cmp else flop_roof
    return {"hbm_frac": hbm, f"{flop_roof}_frac": cmp_, "bound": bound, "frac": hbm if bound == "hbm" else cmp_,
            "algorithmic_bytes": bytes_, "flops": flops}


def secondary(torch, cue, cuet, _lib, dev, wl: str, dtype_name, steps: int, warmup: int, graph: bool = False,
              calling_thread_autograd: bool = False) -> dict:
    """One secondary workload (BASELINE.json configs[0], [2], [3], [4]); same timing discipline as the headline line.
    Both roofs are reported: algorithmic bytes against 8 TB/s and flops against the matrix-core peak of the input type
    (dense workloads) or the fp32 vector peak (path-table workloads)."""
    if wl == "cfg1":
        Z = 4096
        i1, i2 = cue.Irreps("O3", "32x0e+32x1o+32x2e"), cue.Irreps("O3", "0e+1o+2e")
        m = cuet.ChannelWiseTensorProduct(i1, i2, ["0e", "1o", "2e"], layout=cue.ir_mul, shared_weights=False,
                                          internal_weights=False, device=dev, dtype=torch.float32)
        g = torch.Generator(device=dev).manual_seed(0)
        x1 = torch.randn(Z, i1.dim, device=dev, generator=g, requires_grad=True)
        x2 = torch.randn(Z, i2.dim, device=dev, generator=g, requires_grad=True)
        w = torch.randn(Z, m.weight_numel, device=dev, generator=g, requires_grad=True)
        cot = torch.randn(Z, m.irreps_out.dim, device=dev, generator=g)

        def step():
            return torch.autograd.grad(m(x1, x2, w), [x1, x2, w], cot)

        unit, units, dt = "samples/s", Z, "f32"
        d1, d2, dw, do = i1.dim, i2.dim, m.weight_numel, m.irreps_out.dim
        alg = {"fwd": Z * (d1 + d2 + dw + do) * 4, "bwd": Z * (2 * (d1 + d2 + dw) + do) * 4}
        flops = {k: Z * n * 128 for k, n in zip(("fwd", "bwd"), VALU_INSTS_PER_ELEMENT["cfg1"])}  # executed vector instructions x 128
        flop_roof, flop_peak = "valu", VALU_PEAK_F32
        desc = ("configs[0]: channel-wise TP 32x0e+32x1o+32x2e (x) 0e+1o+2e, outputs up to l = 2, batch 4096, per-sample weights, "
                "fwd + bwd (dx1, dx2, dw); 69 MB of traffic: launch-latency regime")
    elif wl == "cfg3":
        Z = 50_000
        dtype = torch.bfloat16 if dtype_name == "bf16" else torch.float32  # (bf16: the buffers; the arithmetic stays float32)
        m = cuet.SymmetricContraction(cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "128x0e+128x1o"),
                                      3, 10, layout=cue.ir_mul, dtype=dtype, device=dev)
        g = torch.Generator(device=dev).manual_seed(0)
        x = torch.randn(Z, 2048, device=dev, generator=g).to(dtype).requires_grad_(True)
        idx = torch.randint(0, 10, (Z,), device=dev, generator=g, dtype=torch.int32)
        with torch.no_grad():
            m.weight.mul_(1.0 / m.weight.shape[1] ** 0.5)
        cot = torch.randn(Z, 512, device=dev, generator=g).to(dtype)

        def step():
            return torch.autograd.grad(m(x, idx), [m.weight, x], cot)

        unit, units, dt = "nodes/s", Z, "f32"
        # every distinct element once: fwd reads x and writes out; bwd reads x, g and writes dx (weights 10 x 3712 negligible)
        es = x.element_size()
        alg = {"fwd": Z * (2048 + 512) * es, "bwd": Z * (2048 + 512 + 2048) * es}
        flops = {k: Z * n * 128 for k, n in zip(("fwd", "bwd"), VALU_INSTS_PER_ELEMENT["cfg3"])}  # executed vector instructions x 128
        flop_roof, flop_peak = "valu", VALU_PEAK_F32
        desc = ("configs[2]: symmetric contraction 128x(0e+1o+2e+3o) -> 128x(0e+1o), degree 3, 10 element types, "
                "50000 nodes, int32 element index, fwd + bwd (dw, dx)" + ("; buffers of bfloat16, arithmetic in float32" if es == 2 else ""))
    elif wl in ("cfg4", "cfg4mi"):
        Z = 200_000
        dtype = getattr(torch, _DTYPES[dtype_name])
        irreps = cue.Irreps("O3", "128x0e+128x1o+128x2e")
        # cfg4mi: the same Linear on mul_ir rows (the module's default layout), addressed inside the dense kernels
        m = cuet.Linear(irreps, irreps, layout=cue.mul_ir if wl == "cfg4mi" else cue.ir_mul, internal_weights=False, method="fused_tp")
        g = torch.Generator(device=dev).manual_seed(0)
        x = torch.randn(Z, 1152, device=dev, generator=g).to(dtype).requires_grad_(True)
        w = torch.randn(1, m.weight_numel, device=dev, generator=g).to(dtype).requires_grad_(True)
        cot = torch.randn(Z, 1152, device=dev, generator=g).to(dtype)

        def step():
            return torch.autograd.grad(m(x, w), [w, x], cot)

        unit, units, dt = "rows/s", Z, _DT_NAME[str(dtype).replace("torch.", "")]
        es = 4 if dtype == torch.float32 else 2
        f = 2 * Z * 128 * 128 * 9
        flops = {"fwd": f, "bwd": 2 * f}
        # fwd reads x, writes out; bwd reads x and g, writes dx (weights 49152 elements negligible)
        alg = {"fwd": 2 * Z * 1152 * es, "bwd": 3 * Z * 1152 * es}
        flop_roof, flop_peak = "mfma", MFMA_PEAK[dt]
        desc = "configs[3]: Linear 128x0e+128x1o+128x2e -> same, batch 200000, shared weights, fwd + bwd (dw, dx)"
        if wl == "cfg4mi":
            desc += "; rows in mul_ir, addressed as they lie by the dense kernels (no transposition pass)"
    elif wl in ("cfg4fc", "cfg4fcmi"):
        Z = 50_000
        dtype = getattr(torch, _DTYPES[dtype_name])
        i1, i2 = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e")
        # cfg4fcmi: the same product on mul_ir rows (the module's default layout), taken as they lie by the fused kernels
        m = cuet.FullyConnectedTensorProduct(i1, i2, i1, layout=cue.mul_ir if wl == "cfg4fcmi" else cue.ir_mul, internal_weights=False)
        g = torch.Generator(device=dev).manual_seed(0)
        x1 = torch.randn(Z, i1.dim, device=dev, generator=g).to(dtype).requires_grad_(True)
        x2 = torch.randn(Z, i2.dim, device=dev, generator=g).to(dtype).requires_grad_(True)
        w = torch.randn(1, m.weight_numel, device=dev, generator=g).to(dtype).requires_grad_(True)
        cot = torch.randn(Z, i1.dim, device=dev, generator=g).to(dtype)

        def step():
            return torch.autograd.grad(m(x1, x2, w), [w, x1, x2], cot)

        unit, units, dt = "rows/s", Z, _DT_NAME[str(dtype).replace("torch.", "")]
        es = 4 if dtype == torch.float32 else 2
        # every distinct element once: fwd reads x1, x2 and writes out; bwd reads x1, x2, g and writes dx1, dx2 (weights 20480 negligible)
        alg = {"fwd": Z * (256 + 9 + 256) * es, "bwd": Z * (256 + 9 + 256 + 256 + 9) * es}
        # 11 distinct (weight block, x1 component) products of 64 x 64 per row; forward, dx1, dx2 and dw contract each once
        f = 2 * Z * 64 * 64 * 11
        flops = {"fwd": f, "bwd": 3 * f}
        flop_roof, flop_peak = "mfma", MFMA_PEAK[dt]
        if dtype == torch.float32:
            # the float32 kernels form the products g W^T once for both input gradients: three contractions are executed
            fc_executed_flops = 3 * f
        desc = ("configs[3]: FullyConnectedTensorProduct 64x0e+64x1o (x) 0e+1o+2e -> 64x0e+64x1o, batch 50000, shared weights, "
                "fwd + bwd (dw, dx1, dx2)")
        if wl == "cfg4fcmi":
            desc += "; rows in mul_ir, taken as they lie by the fused kernels (no transposition pass)"
    elif wl == "fcgen":
        # a fully connected product whose second operand has multiplicity above one (no BASELINE config; sizes chosen here): the
        # products of the two operands in HBM, then a Linear map on the matrix cores
        Z = 50_000
        dtype = getattr(torch, _DTYPES[dtype_name])
        i1, i2 = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "16x0e+16x1o")
        m = cuet.FullyConnectedTensorProduct(i1, i2, i1, layout=cue.ir_mul, internal_weights=False)
        g = torch.Generator(device=dev).manual_seed(0)
        x1 = torch.randn(Z, i1.dim, device=dev, generator=g).to(dtype).requires_grad_(True)
        x2 = torch.randn(Z, i2.dim, device=dev, generator=g).to(dtype).requires_grad_(True)
        w = torch.randn(1, m.weight_numel, device=dev, generator=g).to(dtype).requires_grad_(True)
        cot = torch.randn(Z, i1.dim, device=dev, generator=g).to(dtype)

        def step():
            return torch.autograd.grad(m(x1, x2, w), [w, x1, x2], cot)

        unit, units, dt = "rows/s", Z, _DT_NAME[str(dtype).replace("torch.", "")]
        es = 4 if dtype == torch.float32 else 2
        # every distinct element once: fwd reads x1, x2 and writes out; bwd reads x1, x2, g and writes dx1, dx2 (weights 655360 elements)
        alg = {"fwd": Z * (256 + 64 + 256) * es, "bwd": Z * (256 + 64 + 256 + 256 + 64) * es}
        # 10 flattened paths, each a (64 * 16) x 64 contraction per row; forward, product gradient and weight gradient contract each once
        f = 2 * Z * 64 * 16 * 64 * 10
        flops = {"fwd": f, "bwd": 2 * f}
        flop_roof, flop_peak = "mfma", MFMA_PEAK[dt]
        desc = ("next row (the general fully connected form u_v_uvw_w): FullyConnectedTensorProduct 64x0e+64x1o (x) 16x0e+16x1o -> "
                "64x0e+64x1o, batch 50000, shared weights, fwd + bwd (dw, dx1, dx2); products of the two operands in HBM (10240 values per "
                "row), then a Linear map on the matrix cores")
    elif wl == "cfg2sh":
        # configs[1] with the spherical harmonics of the edge vectors evaluated inside the edge kernels (the step before the
        # product in a MACE interaction block): inputs are the raw edge vectors, gradients also with respect to them
        N, E = 5_000, 100_000
        i1 = cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o")
        m = cuet.ChannelWiseSphericalTensorProduct(i1, [0, 1, 2, 3], "0e+1o+2e+3o", layout=cue.ir_mul, shared_weights=False,
                                                   internal_weights=False, device=dev, dtype=torch.float32)
        g = torch.Generator(device=dev).manual_seed(0)
        x1 = torch.randn(N, i1.dim, device=dev, generator=g, requires_grad=True)
        vec = torch.randn(E, 3, device=dev, generator=g, requires_grad=True)
        w = torch.randn(E, m.weight_numel, device=dev, generator=g, requires_grad=True)
        snd = torch.randint(0, N, (E,), device=dev, generator=g, dtype=torch.int32)
        rcv = torch.sort(torch.randint(0, N, (E,), device=dev, generator=g, dtype=torch.int32))[0]
        cot = torch.randn(N, m.irreps_out.dim, device=dev, generator=g)

        def step():
            return torch.autograd.grad(m(x1, vec, w, indices_1=snd, indices_out=rcv, size_out=N), [w, x1, vec], cot)

        unit, units, dt = "edges/s", E, "f32"
        alg = {"fwd": (E * (2944 + 3) + N * (2048 + 12672)) * 4 + 2 * E * 4,
               "bwd": (2 * E * (2944 + 3) + N * (2 * 2048 + 12672)) * 4 + 2 * E * 4}
        flops = {k: E * n_ * 128 for k, n_ in zip(("fwd", "bwd"), VALU_INSTS_PER_ELEMENT["cfg2"])}
        flop_roof, flop_peak = "valu", VALU_PEAK_F32
        desc = ("configs[1] with the spherical harmonics (l <= 3, normalised vectors) evaluated inside the edge kernels: 5000 nodes, "
                "100000 edges, inputs node features / edge vectors / per-edge weights, fwd + bwd (dw, dx1, d vectors)")
    elif wl == "fcconv":
        # the product inside FullyConnectedTensorProductConv: a weight row per edge, x1 gathered by source, output summed by
        # destination (no BASELINE config; sizes chosen here)
        E, N = 20_000, 2_000
        i1, i2 = cue.Irreps("O3", "64x0e+64x1o"), cue.Irreps("O3", "0e+1o+2e")
        m = cuet.FullyConnectedTensorProduct(i1, i2, i1, layout=cue.ir_mul, shared_weights=False, internal_weights=False,
                                             device=dev, dtype=torch.float32)
        g = torch.Generator(device=dev).manual_seed(0)
        x1 = torch.randn(N, i1.dim, device=dev, generator=g, requires_grad=True)
        x2 = torch.randn(E, i2.dim, device=dev, generator=g, requires_grad=True)
        w = torch.randn(E, m.weight_numel, device=dev, generator=g, requires_grad=True)
        snd = torch.randint(0, N, (E,), device=dev, generator=g, dtype=torch.int32)
        rcv = torch.sort(torch.randint(0, N, (E,), device=dev, generator=g, dtype=torch.int32))[0]
        cot = torch.randn(N, i1.dim, device=dev, generator=g)

        def step():
            return torch.autograd.grad(m(x1, x2, w, indices_1=snd, indices_out=rcv, size_out=N), [x1, x2, w], cot)

        unit, units, dt = "edges/s", E, "f32"
        W = m.weight_numel
        # every distinct element once: fwd reads w, x2, x1, two index arrays and writes out; bwd reads w, x2, x1, g and writes dw, dx2, dx1
        alg = {"fwd": (E * (W + 9) + 2 * N * 256) * 4 + 2 * E * 4, "bwd": (2 * E * (W + 9) + 3 * N * 256) * 4 + 2 * E * 4}
        # per weight: forward 2 (2 l3 + 1) / block flops, backward twice that (weight gradient and R)
        f = 2 * E * 64 * 64 * 11
        flops = {"fwd": f, "bwd": 2 * f}
        flop_roof, flop_peak = "valu", VALU_PEAK_F32
        desc = ("next row (FullyConnectedTensorProductConv's product): 64x0e+64x1o (x) 0e+1o+2e -> 64x0e+64x1o, a weight row per edge, "
                "20000 edges, 2000 nodes, x1 gathered by source, output summed by destination, fwd + bwd (dw, dx1, dx2)")
    elif wl == "cfg5":
        dtype = getattr(torch, _DTYPES[dtype_name or "bf16"])
        n, D = 512, 128
        g = torch.Generator(device=dev).manual_seed(0)

        def r(*shape, scale=1.0):
            return (torch.randn(*shape, device=dev, generator=g) * scale).to(dtype)

        x = r(1, n, n, D).requires_grad_(True)
        kw = dict(mask=(torch.rand(1, n, n, device=dev, generator=g) < 0.9).to(dtype),
                  norm_in_weight=torch.ones(D, device=dev, dtype=dtype), norm_in_bias=torch.zeros(D, device=dev, dtype=dtype),
                  p_in_weight=r(2 * D, D, scale=D ** -0.5), g_in_weight=r(2 * D, D, scale=D ** -0.5),
                  norm_out_weight=torch.ones(D, device=dev, dtype=dtype), norm_out_bias=torch.zeros(D, device=dev, dtype=dtype),
                  p_out_weight=r(D, D, scale=D ** -0.5), g_out_weight=r(D, D, scale=D ** -0.5))
        cot = r(1, n, n, D)

        def step():
            return torch.autograd.grad(cuet.triangle_multiplicative_update(x, "outgoing", **kw), [x], cot)

        unit, units, dt = "pair rows/s", n * n, _DT_NAME[str(dtype).replace("torch.", "")]
        es = 4 if dtype == torch.float32 else 2
        f = 2 * n * n * D * 4 * D + 2 * D * n ** 3 + 2 * n * n * D * 2 * D  # projections in, contraction, projections out
        flops = {"fwd": f, "bwd": 2 * f}
        # fwd reads z and the mask, writes the update; bwd reads z, the mask and the cotangent, writes dz
        alg = {"fwd": (2 * n * n * D + n * n) * es, "bwd": (3 * n * n * D + n * n) * es}
        flop_roof, flop_peak = "mfma", MFMA_PEAK[dt]
        desc = "configs[4]: triangle multiplicative update, outgoing, z [1,512,512,128], mask Bernoulli(0.9), fwd + bwd w.r.t. z"
        # What the stages of this decomposition move at the least (the normalised input, a, b, t, y and their cotangents live
        # in HBM between the launches): per pair row and channel, in elements - forward: x read, x-hat written, a|b (2)
        # written and read, t written and read, y written, x-hat and y read, out written = 12; backward: dout, x-hat, y read,
        # dx-hat and dy written, dy and t read, dt written, dt read twice with a and b, da|db (2) written and read, x and
        # x-hat and dx-hat read, dx written = 20.
        extra = {"decomposition_traffic_bytes": (12 + 20) * n * n * D * es}
    else:
        raise ValueError(wl)
    if graph:
        # the step as one HIP graph: same kernels, no launch gaps (per-kernel events cannot be recorded inside a graph)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(warmup, 3)):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        cuda_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cuda_graph):
            step()
        run = cuda_graph.replay
    else:
        run = step
    # calling_thread_autograd: PyTorch hands the backward of GPU tensors to a worker thread of the device and waits for it;
    # torch.autograd.set_multithreading_enabled(False) runs it on the calling thread (a process-wide setting a single-GPU
    # user may choose).  The hand-over is most of the host's time in the launch-bound workloads.
    with torch.autograd.set_multithreading_enabled(not calling_thread_autograd):
        for _ in range(warmup):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            run()
        torch.cuda.synchronize()
        elapsed = (time.perf_counter() - t0) / steps
    # per-kernel durations from a second pass of the same steps with HIP events around the library's kernels: the events cost
    # a few microseconds per kernel on the device (0.09 ms on the eleven launches of the triangle update), so they stay out
    # of the timed region of these workloads
    kernels = {}
    if not graph:
        _lib.timing_begin()
        for _ in range(steps):
            run()
        torch.cuda.synchronize()
        kernels = {n_: {"launches": l, "avg_ms": t / max(l, 1), "ms_per_step": t / steps} for n_, (l, t) in _lib.timing_end().items()}
    if graph:
        desc += "; the step replayed as one HIP graph"
    if calling_thread_autograd:
        desc += "; backward on the calling thread (torch.autograd.set_multithreading_enabled(False))"
    roofs = _roofs(alg["fwd"] + alg["bwd"], flops["fwd"] + flops["bwd"], elapsed, flop_peak, flop_roof)
    more = dict(extra) if wl == "cfg5" else {}
    if more:  # the step against 8 TB/s on the bytes its own stages must move (the binding roof of the 2-byte step as decomposed)
        more["hbm_frac_of_decomposition_traffic"] = more["decomposition_traffic_bytes"] / elapsed / 1e9 / HBM_PEAK_GBS
    if wl in ("cfg4fc", "cfg4fcmi") and dt == "f32":
        # `flops` counts the four contractions of the step (forward, dx1, dx2, dw); the matrix instructions executed are fewer
        more["executed_matrix_flops"] = fc_executed_flops
        more["mfma_frac_executed"] = fc_executed_flops / elapsed / 1e12 / flop_peak
    achieved = ((alg["fwd"] + alg["bwd"]) / elapsed / 1e9) if roofs["bound"] == "hbm" else ((flops["fwd"] + flops["bwd"]) / elapsed / 1e12)
    return {
        "metric": f"{unit.split('/')[0]}/sec, {wl} fwd+bwd (secondary workload)", "value": units / elapsed, "unit": unit, "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": elapsed * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dt, "data": "synthetic", "config": {"workload": desc},
        "roofline": {"bound": roofs["bound"], "achieved": achieved, "peak": HBM_PEAK_GBS if roofs["bound"] == "hbm" else flop_peak,
                     "unit": "GB/s" if roofs["bound"] == "hbm" else "TFLOP/s", "frac": roofs["frac"], "traffic": None,
                     "hbm_frac": roofs["hbm_frac"], f"{flop_roof}_frac": roofs[f"{flop_roof}_frac"],
                     "algorithmic_bytes": roofs["algorithmic_bytes"], "flops": roofs["flops"], **more,
                     "scope": "whole step: algorithmic bytes and flops of forward + backward over the step time, against 8 TB/s and the "
                              f"{flop_roof} peak ({flop_peak} TFLOP/s); bound = the roof with the longer minimum time"
                              + ("; flops = 2 (2 l3 + 1) per weight, forward once and backward twice (algorithmic)" if wl == "fcconv" else
                                 "; flops = executed vector instructions x 128, " + VALU_SOURCE if flop_roof == "valu" else "")},
        "kernels": kernels,
    }


def run_cfg2(torch, cue, cuet, _lib, dev, dtype, N: int, E: int, steps: int, warmup: int, deterministic: bool, fresh_indices: bool = False):
    """The headline workload once; returns (JSON line, module, host inputs)."""
    prev = os.environ.get("CUEQ_DETERMINISTIC")
    os.environ["CUEQ_DETERMINISTIC"] = "1" if deterministic else "0"
    try:
        m = cuet.ChannelWiseTensorProduct(
            cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "0e+1o+2e+3o"), "0e+1o+2e+3o",
            layout=cue.ir_mul, shared_weights=False,
        )
        host = make_inputs(torch, cue, N, E, dtype)
        node, sh, w, senders, receivers, cot = (t.to(dev) for t in host)
        node.requires_grad_(True), sh.requires_grad_(True), w.requires_grad_(True)

        def step():
            # fresh_indices: a new receiver tensor every step (a neighbour list that changes with every MD step): the grouping
            # of edges by receiver is built again instead of taken from the cache
            rcv = receivers.clone() if fresh_indices else receivers
            out = m(node, sh, w, indices_1=senders, indices_out=rcv, size_out=N)
            return torch.autograd.grad(out, [w, node, sh], cot)

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        _lib.timing_begin()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        kernels = _lib.timing_end()
    finally:
        if prev is None:
            os.environ.pop("CUEQ_DETERMINISTIC", None)
        else:
            os.environ["CUEQ_DETERMINISTIC"] = prev
    ms_per_step = elapsed / steps * 1e3
    value = E / (elapsed / steps)

    plan = m.f.m._plan(torch.float64 if dtype == torch.float64 else torch.float32)
    specialised = bool(plan.serves(dtype) and plan.backward_plan((True, True, True)).serves(dtype))
    s = {torch.float32: 4, torch.float64: 8, torch.bfloat16: 2}[dtype]
    alg = algorithmic_bytes(E, N, 2944, 2048, 16, 12672, s)
    per_kernel = {}
    for name, (launches, total_ms) in kernels.items():
        kind = "fwd" if "_fwd_" in name else "bwd"
        avg_ms = total_ms / max(launches, 1)
        per_kernel[name] = {
            "launches": launches, "avg_ms": avg_ms, "algorithmic_bytes": alg[kind],
            "achieved_GBps": alg[kind] / (avg_ms * 1e-3) / 1e9,
        }
    dominant = max(per_kernel.items(), key=lambda kv: kv[1]["avg_ms"]) if per_kernel else None
    roofline = None
    ceiling = design_ceiling(N, E, alg) if (dtype == torch.float32 and not deterministic) else None
    if dominant is not None:
        a = dominant[1]["achieved_GBps"]
        traffic = MEASURED_TRAFFIC_BYTES.get((dominant[0], N, E)) if not deterministic else None
        roofline = {
            "bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
            "traffic": traffic, "traffic_source": TRAFFIC_SOURCE if traffic else None,
            "kernel": dominant[0], "avg_ms": dominant[1]["avg_ms"],
            "algorithmic_bytes_per_launch": dominant[1]["algorithmic_bytes"],
        }
        if ceiling is not None and traffic:
            # the fraction of the 8 TB/s roofline this kernel would reach at its least time (see design_ceiling)
            kind = "fwd" if "_fwd_" in dominant[0] else "bwd"
            roofline["design_ceiling_frac"] = dominant[1]["algorithmic_bytes"] / ceiling[kind] / 1e9 / HBM_PEAK_GBS
            roofline["design_ceiling_ms"] = ceiling[kind] * 1e3
            roofline["design_ceiling_source"] = CAL_SOURCE
    total_alg = alg["fwd"] + alg["bwd"]
    valu_flops = E * sum(VALU_INSTS_PER_ELEMENT["cfg2"]) * 128  # executed vector instructions x 128 flops
    line = {
        "metric": "edges/sec, indexed channelwise TP fwd+bwd (128ch, lmax=3); % HBM roofline",
        "value": value,
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64" if dtype == torch.float64 else "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: MACE-style indexed channel-wise TP, 5000 nodes x 128x0e+128x1o+128x2e+128x3o, "
                        "100000 edges x SH 0e+1o+2e+3o, per-edge weights [E,2944], int32 sender/receiver (receivers "
                        "sorted), scatter-sum onto 5000 nodes, fwd + bwd (dw, dx1, dx2)",
            "nodes": N, "edges": E, "specialised_kernels": specialised,
            "buffers": {torch.float32: "f32", torch.float64: "f64", torch.bfloat16: "bf16 (arithmetic in f32)"}[dtype],
            "dx1_scatter": "ordered" if deterministic else "fp-atomics",
        },
        "roofline": roofline,
        "step_roofline_frac": (total_alg / (elapsed / steps)) / 1e9 / HBM_PEAK_GBS,
        "step_design_ceiling_frac": (total_alg / (ceiling["fwd"] + ceiling["bwd"])) / 1e9 / HBM_PEAK_GBS if ceiling else None,
        "step_valu_frac": valu_flops / (elapsed / steps) / 1e12 / (78.6 if dtype == torch.float64 else VALU_PEAK_F32),
        "valu_source": VALU_SOURCE,
        "kernels": per_kernel,
    }
    return line, m, host


def setup_costs(torch, cue, cuet, _lib, dev, N: int, E: int, compile_probe: bool) -> dict:
    """What a user pays before / around the timed steps of the headline workload: building the module (descriptor and
    path tables, on the host), creating the device plans of forward and backward, grouping the edges by receiver (built once
    per index tensor in eager mode and cached; measured for sorted and for shuffled receivers), and - for a descriptor the
    library was not built for - compiling its kernels at first use."""
    import tempfile

    out = {}
    t0 = time.perf_counter()
    m = cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "0e+1o+2e+3o"), "0e+1o+2e+3o",
                                      layout=cue.ir_mul, shared_weights=False)
    out["module_build_ms"] = (time.perf_counter() - t0) * 1e3
    import importlib

    u1d = importlib.import_module("cuequivariance_amd.cuet.uniform_1d")  # (the package also exports a function of this name)
    cached = m.f.m._plan(torch.float32)
    # a plan object of its own (the module's is shared through a cache and exists since the timed steps): the tables of the
    # backward derived on the host, both sets uploaded, the generated kernels looked up
    plan = u1d.Uniform1dPlan(cached.tables, torch.float32)
    plan.polynomial, plan.origin = cached.polynomial, cached.origin
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    plan.handle(dev)
    plan.backward_plan((True, True, True)).handle(dev)
    torch.cuda.synchronize()
    out["plan_create_ms"] = (time.perf_counter() - t0) * 1e3

    g = torch.Generator().manual_seed(1)
    sorted_ids = torch.sort(torch.randint(0, N, (E,), generator=g, dtype=torch.int32))[0].to(dev)
    shuffled = sorted_ids[torch.randperm(E, generator=g).to(dev)].contiguous()
    for name, ids in (("csr_build_ms_sorted_receivers", sorted_ids), ("csr_build_ms_unsorted_receivers", shuffled)):
        times = []
        for _ in range(5):
            fresh = ids.clone()  # (a new tensor: the cache of groupings misses)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            u1d._segment_csr(fresh, N)
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
        out[name] = sorted(times)[len(times) // 2]
    if compile_probe:
        # a channel-wise product the library holds no kernels for (64 channels, l <= 3), compiled into an empty cache
        from cuequivariance_amd import jit

        prev = os.environ.get("CUEQ_AMD_JIT_CACHE")
        try:
            with tempfile.TemporaryDirectory() as tmp:
                os.environ["CUEQ_AMD_JIT_CACHE"] = tmp
                if jit.enabled():
                    mm = cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "64x0e+64x1o+64x2e+64x3o"), cue.Irreps("O3", "0e+1o+2e+3o"),
                                                       "0e+1o+2e+3o", layout=cue.ir_mul, shared_weights=False)
                    t0 = time.perf_counter()
                    p2 = mm.f.m._plan(torch.float32)
                    p2.handle(dev)
                    p2.backward_plan((True, True, True)).handle(dev)
                    out["first_use_compile_s"] = time.perf_counter() - t0
                    out["first_use_compile_descriptor"] = "channel-wise 64x(0e+1o+2e+3o) x (0e+1o+2e+3o), forward + backward unit, hipcc -O3 for gfx950"
        except Exception as e:  # (no compiler on the box, cache not writable: the table-driven kernels would run)
            out["first_use_compile_s"] = None
            out["first_use_compile_error"] = f"{type(e).__name__}: {e}"
        finally:
            if prev is None:
                os.environ.pop("CUEQ_AMD_JIT_CACHE", None)
            else:
                os.environ["CUEQ_AMD_JIT_CACHE"] = prev
    return out


def cpu_baseline_dense(torch, cue, wl: str, threads: int) -> dict:
    """CPU baselines of the dense workloads: the oracle (plain torch on the host) on a bounded sample, fwd + bwd."""
    import statistics as st

    cores = threads if threads > 0 else min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    if wl == "cfg5":
        from oracle.triangle import triangle_multiplicative_update as oracle_trimul

        n, D = 384, 128

        def r(*shape, scale=1.0):
            return torch.randn(*shape, generator=g) * scale

        x = r(1, n, n, D).requires_grad_(True)
        kw = dict(mask=(torch.rand(1, n, n, generator=g) < 0.9).float(), norm_in_weight=torch.ones(D), norm_in_bias=torch.zeros(D),
                  p_in_weight=r(2 * D, D, scale=D ** -0.5), g_in_weight=r(2 * D, D, scale=D ** -0.5),
                  norm_out_weight=torch.ones(D), norm_out_bias=torch.zeros(D),
                  p_out_weight=r(D, D, scale=D ** -0.5), g_out_weight=r(D, D, scale=D ** -0.5))
        cot = r(1, n, n, D)

        def once():
            t0 = time.perf_counter()
            torch.autograd.grad(oracle_trimul(x, "outgoing", **kw), [x], cot)
            return time.perf_counter() - t0

        units, unit = n * n, "pair rows/s"
        sample = f"one {n} x {n} x {D} pair tensor (the workload has 512 x 512; the contraction grows with the cube), float32"
    else:  # cfg4 Linear: three 128 x 128 blocks per irrep component on ir_mul slices = the oracle's per-path einsum
        from oracle.naive import naive_segmented_polynomial, spec_from_polynomial

        Z = 200_000
        irreps = cue.Irreps("O3", "128x0e+128x1o+128x2e")
        e = cue.descriptors.linear(irreps, irreps)
        spec = spec_from_polynomial(e.polynomial)
        x = torch.randn(Z, 1152, generator=g).requires_grad_(True)
        w = torch.randn(1, e.polynomial.inputs[0].size, generator=g).requires_grad_(True)
        cot = torch.randn(Z, 1152, generator=g)

        def once():
            t0 = time.perf_counter()
            out = naive_segmented_polynomial(spec, [w, x])[0]
            torch.autograd.grad(out, [w, x], cot)
            return time.perf_counter() - t0

        units, unit = Z, "rows/s"
        sample = f"all {Z} rows, float32"
    once()
    t = st.median([once() for _ in range(3)])
    return {"value": units / t, "unit": unit, "cores": cores, "kind": "port",
            "sample": f"{sample}, fwd+bwd, median of 3 after 1 warm-up ({t:.2f} s each)"}


def _compact(line: dict) -> dict:
    r = line["roofline"]
    out = {"ms_per_step": line["ms_per_step"], "value": line["value"], "unit": line["unit"], "dtype": line["dtype"],
           "bound": r["bound"], "frac": r["frac"], "workload": line["config"]["workload"]}
    for k in ("hbm_frac", "mfma_frac", "valu_frac", "decomposition_traffic_bytes", "hbm_frac_of_decomposition_traffic",
              "executed_matrix_flops", "mfma_frac_executed"):
        if k in r:
            out[k] = r[k]
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--dtype", choices=["fp32", "fp64", "bf16", "fp16"], default=None,
                    help="cfg2: fp32 (default) or fp64; cfg3: fp32; cfg4: fp32 (default) or bf16; cfg5: bf16 (default) or fp32")
    ap.add_argument("--nodes", type=int, default=5000)
    ap.add_argument("--edges", type=int, default=100_000)
    ap.add_argument("--cpu-sample-edges", type=int, default=12000)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="headline line only (no 'secondary' object)")
    ap.add_argument("--no-setup-costs", action="store_true", help="leave out the 'setup' object (module build, plan creation, edge grouping, first-use compilation)")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads of the CPU baseline (default: the box's share, at most 16)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="only run a 1 GiB device-to-device copy a few times (to scale rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--calibrate", action="store_true",
                    help="only measure what the memory system delivers to streaming kernels of this library's shape: read, write, "
                         "copy and float atomic-add rates over 1 GiB")
    ap.add_argument("--deterministic", action="store_true",
                    help="ordered (bit-reproducible) scatter of the node-feature gradient instead of fp atomics")
    ap.add_argument("--graph", action="store_true",
                    help="secondary workloads only: capture the step into a HIP graph and time its replays")
    ap.add_argument("--calling-thread-autograd", action="store_true",
                    help="secondary workloads only: time the step with torch.autograd.set_multithreading_enabled(False)")
    ap.add_argument("--workload", choices=["cfg1", "cfg2", "cfg2sh", "cfg3", "cfg4", "cfg4mi", "cfg4fc", "cfg4fcmi", "fcgen", "fcconv", "cfg5"], default=None,
                    help="default: the headline metric (cfg2, fp32) with every other configuration in a 'secondary' object.  "
                         "Naming a workload prints one line for it alone: cfg2 the headline, cfg1 the reference's CPU-sized "
                         "channel-wise case, cfg3 symmetric contraction, cfg4 Linear 128 channels l<=2, cfg4fc fully connected "
                         "product, cfg5 triangle update")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the path would shard over receiver ranges (no exchange in the forward, one reduce-scatter of the node gradient in the backward)",
              file=sys.stderr)
        return 2

    import torch

    from cuequivariance_amd import _lib, cue, cuet

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    if args.calibrate:
        # what the memory system delivers to kernels shaped like the path-table kernels (cueq_calibrate): 1 GiB per launch
        n = 1 << 30
        a = torch.zeros(n // 4, dtype=torch.float32, device=dev)
        b = torch.zeros(n // 4, dtype=torch.float32, device=dev)
        stream = torch.cuda.current_stream(dev).cuda_stream
        out = {"calibration": "cueq_calibrate, 1 GiB per launch, 64-thread workgroups, one dword per lane and instruction, 8 wavefronts per CU",
               "published_hbm_TBps": HBM_PEAK_GBS / 1e3}
        for kind, name, moved in ((0, "read", n), (1, "write", n), (3, "copy", 2 * n), (2, "atomic_add_f32", n)):
            for _ in range(2):
                _lib.check(_lib.load().cueq_calibrate(kind, a.data_ptr(), b.data_ptr(), n, stream), "cueq_calibrate")
            torch.cuda.synchronize()
            _lib.timing_begin()
            for _ in range(5):
                _lib.check(_lib.load().cueq_calibrate(kind, a.data_ptr(), b.data_ptr(), n, stream), "cueq_calibrate")
            torch.cuda.synchronize()
            (launches, total_ms), = _lib.timing_end().values()
            out[name + "_TBps"] = moved / (total_ms / launches * 1e-3) / 1e12
        print(json.dumps(out))
        return 0
    if args.calibration_copy:
        n = 1 << 28  # 2^28 floats = 1 GiB read and 1 GiB written per copy
        a = torch.ones(n, dtype=torch.float32, device=dev)
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "copy", "bytes_read": n * 4, "bytes_written": n * 4, "launches": 5}))
        return 0
    if args.workload not in (None, "cfg2"):
        print(json.dumps(secondary(torch, cue, cuet, _lib, dev, args.workload, args.dtype, args.steps, args.warmup, args.graph,
                                   args.calling_thread_autograd)))
        return 0
    # (bf16: buffers of bfloat16, arithmetic in float32 - a secondary measurement, the headline is float32 throughout)
    dtype = {"fp64": torch.float64, "bf16": torch.bfloat16}.get(args.dtype, torch.float32)
    N, E = args.nodes, args.edges
    line, m, host = run_cfg2(torch, cue, cuet, _lib, dev, dtype, N, E, args.steps, args.warmup, args.deterministic)
    full = args.workload is None and not args.no_secondary
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch, cue, m, host, min(args.cpu_sample_edges, E), min(200, N), args.cpu_threads)
    if full:
        # every other configuration in the same run: fewer steps each, same discipline (warm-up, synchronise, wall clock)
        del m, host
        sec = {}
        ssteps, swarm = 20, 5

        def add(key, fn):
            torch.cuda.empty_cache()
            try:
                sec[key] = fn()
            except Exception as e:  # a secondary workload must not take the headline down with it
                sec[key] = {"error": f"{type(e).__name__}: {e}"}

        add("cfg2_fp32_ordered_dx1", lambda: _cfg2_compact(run_cfg2(torch, cue, cuet, _lib, dev, torch.float32, N, E, ssteps, swarm, True)[0]))
        add("cfg2_fp64", lambda: _cfg2_compact(run_cfg2(torch, cue, cuet, _lib, dev, torch.float64, N, E, ssteps, swarm, False)[0]))
        add("cfg2_bf16_io", lambda: _cfg2_compact(run_cfg2(torch, cue, cuet, _lib, dev, torch.bfloat16, N, E, ssteps, swarm, False)[0]))
        add("cfg2_fp32_grouping_rebuilt_every_step",
            lambda: _cfg2_compact(run_cfg2(torch, cue, cuet, _lib, dev, torch.float32, N, E, ssteps, swarm, False, fresh_indices=True)[0]))
        for key, wl, dn in (("cfg1_fp32", "cfg1", None), ("cfg3_fp32", "cfg3", None), ("cfg3_bf16_io", "cfg3", "bf16"), ("cfg4_linear_fp32", "cfg4", "fp32"),
                            ("cfg4_linear_bf16", "cfg4", "bf16"), ("cfg4_linear_fp32_mul_ir", "cfg4mi", "fp32"),
                            ("cfg4_linear_bf16_mul_ir", "cfg4mi", "bf16"), ("cfg4_fc_fp32", "cfg4fc", "fp32"), ("cfg4_fc_bf16", "cfg4fc", "bf16"), ("cfg4_fc_fp32_mul_ir", "cfg4fcmi", "fp32"),
                            ("cfg4_fc_bf16_mul_ir", "cfg4fcmi", "bf16"), ("fc_general_fp32", "fcgen", "fp32"), ("fc_general_bf16", "fcgen", "bf16"), ("fc_conv_rows_fp32", "fcconv", "fp32"), ("cfg2_fp32_harmonics_in_kernels", "cfg2sh", "fp32"),
                            ("cfg5_bf16", "cfg5", "bf16"), ("cfg5_fp16", "cfg5", "fp16"), ("cfg5_fp32", "cfg5", "fp32"),
                            ("cfg4_linear_fp16", "cfg4", "fp16"), ("cfg4_fc_fp16", "cfg4fc", "fp16")):
            add(key, lambda wl=wl, dn=dn: _compact(secondary(torch, cue, cuet, _lib, dev, wl, dn, ssteps, swarm)))
            if key in ("cfg1_fp32", "cfg4_fc_bf16", "cfg4_fc_bf16_mul_ir") and "error" not in sec[key]:
                # workloads whose eager step is bound by the host's launch path: the same step replayed as one HIP graph, and
                # the eager step with the backward on the calling thread instead of PyTorch's device worker thread
                try:
                    sec[key]["graph_ms_per_step"] = secondary(torch, cue, cuet, _lib, dev, wl, dn, ssteps, swarm, graph=True)["ms_per_step"]
                except Exception as e:
                    sec[key]["graph_ms_per_step"] = None
                    sec[key]["graph_error"] = f"{type(e).__name__}: {e}"
                try:
                    sec[key]["calling_thread_autograd_ms_per_step"] = secondary(torch, cue, cuet, _lib, dev, wl, dn, ssteps, swarm,
                                                                                calling_thread_autograd=True)["ms_per_step"]
                except Exception as e:
                    sec[key]["calling_thread_autograd_ms_per_step"] = None
                    sec[key]["calling_thread_autograd_error"] = f"{type(e).__name__}: {e}"
        if not args.no_cpu_baseline:
            # more CPU baselines (the oracle on this box's host cores, bounded samples): the headline workload on one
            # thread, the dense workloads on the box's share of cores
            h1 = make_inputs(torch, cue, N, E, torch.float32)
            m1 = cuet.ChannelWiseTensorProduct(cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o"), cue.Irreps("O3", "0e+1o+2e+3o"),
                                               "0e+1o+2e+3o", layout=cue.ir_mul, shared_weights=False)
            sec["cpu_baselines"] = {
                "cfg2_fp32_1_thread": cpu_baseline(torch, cue, m1, h1, 2000, 200, 1),
                "cfg4_linear_fp32": cpu_baseline_dense(torch, cue, "cfg4", args.cpu_threads),
                "cfg5_fp32": cpu_baseline_dense(torch, cue, "cfg5", args.cpu_threads),
            }
        line["secondary"] = sec
    if args.workload is None and not args.no_setup_costs:
        try:
            line["setup"] = setup_costs(torch, cue, cuet, _lib, dev, N, E, compile_probe=full)
        except Exception as e:
            line["setup"] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(line))
    return 0


def _cfg2_compact(line: dict) -> dict:
    return {"ms_per_step": line["ms_per_step"], "value": line["value"], "unit": line["unit"], "dtype": line["dtype"],
            "bound": "hbm", "frac": line["step_roofline_frac"], "hbm_frac": line["step_roofline_frac"],
            "valu_frac": line["step_valu_frac"], "dx1_scatter": line["config"]["dx1_scatter"], "buffers": line["config"]["buffers"],
            "specialised_kernels": line["config"]["specialised_kernels"],
            "kernels_avg_ms": {k: v["avg_ms"] for k, v in line["kernels"].items()}, "workload": line["config"]["workload"]}


if __name__ == "__main__":
    sys.exit(main())
