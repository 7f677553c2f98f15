"""Descriptors for which specialised kernels are generated when the library is built.

Each entry yields one translation unit per math type in ``csrc/generated`` holding a forward kernel and a fused
backward kernel.  Anything not listed runs on the table-driven kernels.
"""

from __future__ import annotations

from pathlib import Path

from .. import cue
from ..tables import U1dTables
from . import channelwise as cw
from . import fullyconnected_rows as fcr
from . import symmetric as sc

GENERATED_DIR = Path(__file__).resolve().parent.parent / "csrc" / "generated"

# (name, irreps_in1, irreps_in2, filter, tuning)
CHANNELWISE = [
    # float64 needs the whole register file of a SIMD lane (one wavefront per SIMD): with two, both kernels spill
    ("c128_l3", "128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o", {"double": {"fwd_waves": 1, "bwd_waves": 1}}),
    ("c32_l2", "32x0e+32x1o+32x2e", "0e+1o+2e", "0e+1o+2e", {}),
]

# Channel-wise entries that are also generated for operands in the mul_ir layout (x1, the output and their gradients
# addressed channel-major inside every irrep block: no transposition pass before or after the kernels); unit "<name>_mulir".
CHANNELWISE_MUL_IR = ["c128_l3", "c32_l2"]

# Channel-wise entries also generated with the second operand computed in the kernels as the spherical harmonics of a
# 3-vector (the degrees of the entry's second irreps); unit "<name>_sh".
CHANNELWISE_HARMONICS = ["c128_l3"]

# (name, irreps_in, irreps_out, contraction degree)
SYMMETRIC = [
    ("s128_l3", "128x0e+128x1o+128x2e+128x3o", "128x0e+128x1o", 3),
    ("s32_l2", "32x0e+32x1o+32x2e", "32x0e+32x1o", 3),
]

# Symmetric contractions also generated for x and the output in the mul_ir layout; unit "<name>_mulir".
SYMMETRIC_MUL_IR = ["s128_l3"]

# Fully connected products (shared weights) whose fused kernels are compiled when the library is built, into
# cuequivariance_amd/prebuilt/: (irreps_in1, irreps_in2, irreps_out), float and bfloat16.  Others are compiled at first use.
FULLY_CONNECTED = [
    ("64x0e+64x1o", "0e+1o+2e", "64x0e+64x1o"),
]

MATH = (("float", 0), ("double", 1))

# Units (by name, the "_mulir" ones included) also generated for buffers of 16-bit elements with float arithmetic:
# {unit name: ("bf16", ...)}.  Other units and element types are compiled at first use.
IO_16BIT = {"c128_l3": ("bf16",), "c128_l3_mulir": ("bf16",), "s128_l3": ("bf16",), "s128_l3_mulir": ("bf16",)}


def channelwise_tables(irreps1: str, irreps2: str, filt) -> U1dTables:
    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", irreps1), cue.Irreps("O3", irreps2), filt)
    return U1dTables.from_polynomial(e.polynomial.flatten_coefficient_modes().squeeze_modes())


def channelwise_mul_ir_groups(irreps1: str, irreps2: str, filt):
    """{buffer: group sizes} of the flattened channel-wise tables when x1 (buffer 1) and the output (buffer 3) are stored
    mul_ir: one group of ``ir.dim`` segments per ``(mul, ir)`` block."""
    e = cue.descriptors.channelwise_tensor_product(cue.Irreps("O3", irreps1), cue.Irreps("O3", irreps2), filt)
    return {1: [ir.dim for _, ir in e.inputs[1].irreps], 3: [ir.dim for _, ir in e.outputs[0].irreps]}


def symmetric_polynomial(irreps_in: str, irreps_out: str, degree: int):
    e = cue.descriptors.symmetric_contraction(cue.Irreps("O3", irreps_in), cue.Irreps("O3", irreps_out), range(1, degree + 1))
    return e.polynomial.flatten_coefficient_modes().squeeze_modes()


def flattened_fully_connected_tables(polynomial) -> U1dTables:
    """The uniform-1d tables of a fully connected product with a weight row per batch row: every mode but the output's
    multiplicity flattened away (what ``cuet.operations._FlattenedUniform`` builds at first use)."""
    q = polynomial.flatten_coefficient_modes()
    stp = q.operations[0][1]
    keep = stp.subscripts.operands[-1][-1]
    return U1dTables.from_polynomial(q.flatten_modes([m for m in stp.subscripts.modes() if m != keep]))


def _write(path: Path, src: str, written: list) -> None:
    if not path.exists() or path.read_text() != src:
        path.write_text(src)
    written.append(path)


def generate(verbose: bool = False) -> list[Path]:
    GENERATED_DIR.mkdir(parents=True, exist_ok=True)
    written = []
    for name, irreps_in, irreps_out, degree in SYMMETRIC:
        poly = symmetric_polynomial(irreps_in, irreps_out, degree)
        variants = [(name, U1dTables.from_polynomial(poly))]
        if name in SYMMETRIC_MUL_IR:  # buffers: w, x | out
            groups = {1: [ir.dim for _, ir in cue.Irreps("O3", irreps_in)], 2: [ir.dim for _, ir in cue.Irreps("O3", irreps_out)]}
            variants.append((name + "_mulir", variants[0][1].with_layouts(groups)))
        for vname, t in variants:
            st = sc.analyze(poly, t.layout(1), t.layout(2))
            for T, code in MATH:
                bwd = {(dw, dx): t.backward((dw, dx)).content_hash(code) for dw, dx in ((True, True), (True, False), (False, True))}
                _write(GENERATED_DIR / f"sc_{vname}_{T}.hip", sc.emit_unit(st, T, vname, t.content_hash(code), bwd), written)
                if verbose:
                    print(f"generated sc_{vname}_{T}.hip: {len(st.terms)} folded terms")
                for io in (IO_16BIT.get(vname, ()) if T == "float" else ()):
                    _write(GENERATED_DIR / f"sc_{vname}_{io}.hip", sc.emit_unit(st, T, vname, t.content_hash(code), bwd, io=io), written)
    for ir1, ir2, ir3 in FULLY_CONNECTED:
        # the same products with a weight row per batch row (the convolution layer's per-edge weights)
        poly = cue.descriptors.fully_connected_tensor_product(cue.Irreps("O3", ir1), cue.Irreps("O3", ir2), cue.Irreps("O3", ir3)).polynomial
        st = fcr.analyze(poly)
        if st is None:
            continue
        t = flattened_fully_connected_tables(poly)
        lmax = [max(ir.l for _, ir in cue.Irreps("O3", x)) for x in (ir1, ir2, ir3)]
        name = f"fcr_{st.U}l{lmax[0]}_l{lmax[1]}_{st.Wd}l{lmax[2]}"
        for T, code in MATH:
            _write(GENERATED_DIR / f"{name}_{T}.hip",
                   fcr.emit_unit(st, T, name, t.content_hash(code), t.backward((True, True, True)).content_hash(code)), written)
            if verbose:
                print(f"generated {name}_{T}.hip: {len(st.blocks)} blocks")
    for name, ir1, ir2, filt, tuning in CHANNELWISE:
        t = channelwise_tables(ir1, ir2, filt)
        assert t.operations == (0, 1, 2, 3) and t.buffer_dim == (1, 1, 0, 1)
        _, paths = t.operation(0)
        st = cw.analyze(t.operand_extent, t.buffer_num_segments, [(*idx, c) for idx, c in paths])
        tb = t.backward((True, True, True))
        variants = [(name, st, t, tb)]
        if name in CHANNELWISE_MUL_IR:
            tl = t.with_layouts(channelwise_mul_ir_groups(ir1, ir2, filt))
            stl = cw.analyze(t.operand_extent, t.buffer_num_segments, [(*idx, c) for idx, c in paths], tl.layout(1), tl.layout(3))
            variants.append((name + "_mulir", stl, tl, tl.backward((True, True, True))))
        if name in CHANNELWISE_HARMONICS:
            from ..cue import fused

            ls = [ir.l for _, ir in cue.Irreps("O3", ir2)]
            poly, info, _ = fused.channelwise_spherical(cue.Irreps("O3", ir1), ls, filt)
            tf = U1dTables.from_polynomial(poly)
            sth = cw.analyze(t.operand_extent, t.buffer_num_segments, [(*idx, c) for idx, c in paths], harmonics=info.terms)
            variants.append((name + "_sh", sth, tf, tf.backward((True, True, True))))
        for vname, vst, vt, vtb in variants:
            for T, code in MATH:
                src = cw.emit_unit(vst, T, vname, vt.content_hash(code), vtb.content_hash(code), **tuning.get(T, {}))
                _write(GENERATED_DIR / f"cw_{vname}_{T}.hip", src, written)
                if verbose:
                    print(f"generated cw_{vname}_{T}.hip: {vst.num_paths} paths")
                for io in (IO_16BIT.get(vname, ()) if T == "float" else ()):
                    _write(GENERATED_DIR / f"cw_{vname}_{io}.hip",
                           cw.emit_unit(vst, T, vname, vt.content_hash(code), vtb.content_hash(code), io=io, **tuning.get(T, {})), written)
    return written


if __name__ == "__main__":
    generate(verbose=True)
