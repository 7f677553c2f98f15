"""Fused kernels for a fully connected tensor product whose second operand has multiplicity one and whose weights are
shared over the batch (``uvw,iu,jv,kw`` with ``v = 1``; reference module ``FusedTensorProductOp4``,
``cuequivariance_torch/primitives/segmented_polynomial_fused_tp.py:40-48``), generated for one descriptor and compiled at
first use by ``cuequivariance_amd/cuet/dense.py``.

With the flattened paths ``(weight block b: K x N at w_off, x1 segment at a_off, x2 column j, output segment at c_off,
coefficient c)`` the three kernels compute, without the intermediates of the table-driven path,

* forward:     ``out[z, c_off + n] += c x2[z, j] sum_k x1[z, a_off + k] W_b[k, n]``
* gradient 1:  ``dx1[z, a_off + k] += c x2[z, j] sum_n g[z, c_off + n] W_b[k, n]``
* gradient 2:  ``dx2[z, j]         += c sum_n g[z, c_off + n] sum_k x1[z, a_off + k] W_b[k, n]``

The weights stay resident in LDS (one persistent block per CU; rows padded by 16 bytes), every wavefront walks 32-row
tiles of the batch on its own: the MFMA result of a (block, operand segment) product holds one batch row per lane and 16
result rows per lane, so the per-row factor ``c x2[z, j]`` is a per-lane scalar and the uses of one product are 16 fused
multiply-adds each into accumulators that never leave registers.  The weight gradient keeps the chunked contraction-major
GEMM.
"""

from __future__ import annotations

from collections import OrderedDict

MAX_WIDTH = 256   # output / input columns held in accumulators (8 tiles of 32)
MAX_LDS = 150 * 1024


def supported(paths, n2: int, width_in: int, width_out: int, es: int) -> bool:
    if not paths or n2 > 16 or width_in > MAX_WIDTH or width_out > MAX_WIDTH or width_in % 32 or width_out % 32:
        return False
    blocks = {(p.w_off, p.K, p.N) for p in paths}
    if any(K % 32 or N % 32 or K > 128 or N > 128 for _, K, N in blocks):
        return False
    if any(p.a_off % 32 or p.c_off % 32 for p in paths):
        return False
    lds = max(sum(N * (K * es + 16) for _, K, N in blocks), sum(K * (N * es + 16) for _, K, N in blocks))
    return lds <= MAX_LDS


PRELUDE = r'''
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef short shortx4_t __attribute__((ext_vector_type(4)));

// 2-byte element types: uint16_t = bfloat16 as its bits, f16bits = IEEE half as its bits
struct f16bits { uint16_t bits; };
template <typename TI> struct is_half { static constexpr bool value = false; };
template <> struct is_half<f16bits> { static constexpr bool value = true; };

template <typename TI>
__device__ __forceinline__ void mma_step(floatx16& acc, const uint4& a, const uint4& b) {
  if constexpr (is_half<TI>::value) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), acc, 0, 0, 0);
  } else if constexpr (sizeof(TI) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
  } else {
    const float* pa = reinterpret_cast<const float*>(&a);
    const float* pb = reinterpret_cast<const float*>(&b);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[e], pb[e], acc, 0, 0, 0);
  }
}
// two floats rounded to nearest even into one word of the 2-byte format, and the halves of such a word as floats
template <typename TI>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const floatx2_t f = {lo, hi};
  if constexpr (is_half<TI>::value) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2_t));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
template <typename TI>
__device__ __forceinline__ float lo2(uint32_t w) {
  if constexpr (is_half<TI>::value) return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w & 0xffffu)));
  else return __uint_as_float(w << 16);
}
template <typename TI>
__device__ __forceinline__ float hi2(uint32_t w) {
  if constexpr (is_half<TI>::value) return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w >> 16)));
  else return __uint_as_float(w & 0xffff0000u);
}
__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(uint16_t v) { return lo2<uint16_t>(v); }
__device__ __forceinline__ float to_f(f16bits v) { return lo2<f16bits>(v.bits); }
// four adjacent elements of a row
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <typename TI>
__device__ __forceinline__ void load4(const TI* p, float (&v)[4]) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  v[0] = lo2<TI>(t.x); v[1] = hi2<TI>(t.x);
  v[2] = lo2<TI>(t.y); v[3] = hi2<TI>(t.y);
}
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) { *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d); }
template <typename TI>
__device__ __forceinline__ void store4(TI* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack2<TI>(a, b), pack2<TI>(c, d));
}
__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
template <typename TI>
__device__ __forceinline__ void store1(TI* p, float v) { *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(pack2<TI>(v, 0.f) & 0xffffu); }

constexpr int kWaves = 8;
'''


def _mul_ir_blocks(blocks):
    """``[(start, mul, d)]`` of the blocks of an operand whose rows keep the component index contiguous (``mul_ir``:
    element (channel u, component i) of the block at ``start + u * d + i``; the kernels' own order is ``start + i * mul +
    u``).  Blocks of one component or one channel are the same in both orders and are left out."""
    return [(s0, mul, d) for s0, mul, d in (blocks or []) if d > 1 and mul > 1]


def _block_at(col: int, blocks, segment_start: bool = True):
    """The block ``(start, mul, d, component)`` that holds column ``col`` (in the kernels' own order), or None;
    ``segment_start``: ``col`` is the first column of an operand segment."""
    for s0, mul, d in blocks:
        if s0 <= col < s0 + mul * d:
            assert not segment_start or (col - s0) % mul == 0, "a path operand is one whole segment of a block"
            return s0, mul, d, (col - s0) // mul
    return None


def _products(paths, transposed: bool):
    """Group the paths by product.  Forward orientation (``transposed``): product = (block, x1 segment), result rows n,
    contraction k, uses = (j, coeff, output offset).  Otherwise: product = (block, output segment), result rows k,
    contraction n, uses = (j, coeff, x1 offset)."""
    prods = OrderedDict()
    for p in paths:
        if transposed:
            key, use = (p.w_off, p.K, p.N, p.a_off), (p.j, p.coeff, p.c_off)
        else:
            key, use = (p.w_off, p.K, p.N, p.c_off), (p.j, p.coeff, p.a_off)
        prods.setdefault(key, []).append(use)
    return prods


def _emit_staging(A, T: str, blocks, lds_off, transposed: bool, threads: int):
    """The weight blocks from memory into LDS (``lds_off[w_off] = (offset, rows, columns, row stride in bytes)``): every
    thread requests all its 16-byte pieces before it writes the first one, so the block starts after one trip to memory
    instead of one per weight block.  ``transposed``: element (k, n) of a block goes to row n, column k."""
    es = 4 if T == "float" else 2
    epv = 16 // es
    plan, total = [], 0
    for w_off, K, N in blocks:
        nvec = K * N // epv
        cnt = (nvec + threads - 1) // threads
        plan.append((w_off, K, N, nvec, cnt, total))
        total += cnt
    A("  {")
    A(f"    uint4 stg[{total}];")
    for w_off, K, N, nvec, cnt, base in plan:
        for i in range(cnt):
            guard = "" if (i + 1) * threads <= nvec else f"(tid + {i * threads} >= {nvec}) ? make_uint4(0, 0, 0, 0) : "
            A(f"    stg[{base + i}] = {guard}*reinterpret_cast<const uint4*>(W + {w_off} + (tid + {i * threads}) * {epv});")
    for w_off, K, N, nvec, cnt, base in plan:
        o, R, C, RS = lds_off[w_off]
        for i in range(cnt):
            guard = "" if (i + 1) * threads <= nvec else f"if (tid + {i * threads} < {nvec}) "
            A(f"    {guard}{{ const int e = (tid + {i * threads}) * {epv}, k = e / {N}, n = e % {N};")
            if not transposed:
                A(f"      *reinterpret_cast<uint4*>(smem + {o} + k * {RS} + n * {es}) = stg[{base + i}]; }}")
            elif es == 4:
                A(f"      char* q = smem + {o} + n * {RS} + k * 4;")
                A(f"      *reinterpret_cast<uint32_t*>(q) = stg[{base + i}].x; *reinterpret_cast<uint32_t*>(q + {RS}) = stg[{base + i}].y;")
                A(f"      *reinterpret_cast<uint32_t*>(q + {2 * RS}) = stg[{base + i}].z; *reinterpret_cast<uint32_t*>(q + {3 * RS}) = stg[{base + i}].w; }}")
            else:
                A(f"      char* q = smem + {o} + n * {RS} + k * 2;")
                for c, comp in enumerate("xyzw"):
                    A(f"      *reinterpret_cast<uint16_t*>(q + {2 * c * RS}) = static_cast<uint16_t>(stg[{base + i}].{comp} & 0xffffu); "
                      f"*reinterpret_cast<uint16_t*>(q + {(2 * c + 1) * RS}) = static_cast<uint16_t>(stg[{base + i}].{comp} >> 16);")
                A("    }")
    A("  }")


def _operand_groups(A, prods, transposed: bool, in_blocks, es: int, single: bool = False):
    """Declares the operand registers of a kernel and returns ``(groups, contraction, request, fragment)``: the products
    grouped by the segment of the row operand ``IN`` they contract with, ``request(gi)`` emits the loads of group ``gi``
    (into one of two register sets, so that a group can be requested while the previous one is worked on) and
    ``fragment(gi, comp, s2, q)`` is the expression of one 16-byte MFMA operand.  ``single``: one register set only - a
    group is requested when the last product of the previous one has read its operands."""
    # products grouped by operand segment so that its fragments are loaded once
    by_seg = OrderedDict()
    for (w_off, K, N, in_off), uses in prods.items():
        by_seg.setdefault(in_off, []).append((w_off, K, N, uses))
    segs = list(by_seg.items())
    if in_blocks:
        segs.sort(key=lambda it: it[0])  # the segments of a block next to each other
    contraction = {in_off: (pl[0][1] if transposed else pl[0][2]) for in_off, pl in segs}
    for in_off, pl in segs:
        assert all((p[1] if transposed else p[2]) == contraction[in_off] for p in pl), "one operand segment, one contraction length"
    # Operand groups: a segment on its own, or the segments of one mul_ir block together - the lane's channels of such a
    # block with all their components are one contiguous run of the row, loaded once and taken apart in registers.
    groups = []
    for in_off, pl in segs:
        blk = _block_at(in_off, in_blocks)
        if blk is not None and groups and groups[-1][0] is not None and groups[-1][0][:3] == blk[:3]:
            groups[-1][1].append((in_off, pl, blk[3]))
        else:
            groups.append((blk, [(in_off, pl, blk[3] if blk else 0)]))
    def nraw(g):  # 16-byte vectors a lane holds for the group
        blk, members = g
        C = contraction[members[0][0]]
        return (C * es // 64) * 2 * (blk[2] if blk else 1)
    if single:
        A(f"    uint4 rawa[{max(nraw(g) for g in groups)}];")
    else:
        A(f"    uint4 rawa[{max(nraw(g) for g in groups[0::2])}], rawb[{max([nraw(g) for g in groups[1::2]] or [1])}];")

    def request(gi):
        blk, members = groups[gi]
        C = contraction[members[0][0]]
        name = "rawa" if (gi % 2 == 0 or single) else "rawb"
        if blk is None:
            in_off = members[0][0]
            for s2 in range(C * es // 64):
                for q in range(2):
                    A(f"    {name}[{2 * s2 + q}] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(IN + z * ldi + {in_off}) + {s2 * 64} + h * 32 + {q * 16});")
        else:
            s0, mul, d, _ = blk
            for s2 in range(C * es // 64):
                for m in range(2 * d):
                    A(f"    {name}[{2 * d * s2 + m}] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(IN + z * ldi + {s0}) + ({s2 * 64} + h * 32) * {d} + {16 * m});")

    def fragment(gi, comp, s2, q):
        """Expression of the MFMA operand (s2, q) of component ``comp`` of group ``gi``: 16 bytes of consecutive channels."""
        blk, members = groups[gi]
        name = "rawa" if (gi % 2 == 0 or single) else "rawb"
        if blk is None:
            return f"{name}[{2 * s2 + q}]"
        d = blk[2]
        word = lambda e: f"{name}[{2 * d * s2 + (e // (4 if es == 4 else 8))}].{'xyzw'[(e // (1 if es == 4 else 2)) % 4]}"
        if es == 4:  # elements (4 q + e) * d + comp of the run, e < 4
            return "make_uint4(" + ", ".join(word((4 * q + e) * d + comp) for e in range(4)) + ")"
        parts = []
        for j in range(4):  # dword j: elements (8 q + 2 j) * d + comp (low half) and the next channel's (high half)
            e0 = (8 * q + 2 * j) * d + comp
            e1 = e0 + d
            sel = (0x0302 if e0 & 1 else 0x0100) | ((0x0706 if e1 & 1 else 0x0504) << 16)
            parts.append(f"__builtin_amdgcn_perm({word(e1)}, {word(e0)}, 0x{sel:08x}u)")
        return "make_uint4(" + ", ".join(parts) + ")"

    return groups, contraction, request, fragment


def _emit_kernel(A, name: str, T: str, paths, transposed: bool, rowdot: bool, width_res: int, n2: int, in_blocks=None, res_blocks=None):
    """One kernel.  ``transposed``: the blocks sit in LDS as W^T (rows n, contraction k).  ``rowdot``: instead of
    accumulating the scaled products into result columns, they are multiplied element-wise with G and summed per row.
    ``in_blocks`` / ``res_blocks``: blocks of the row operand ``IN`` / of the result (``G`` for ``rowdot``) that lie in
    ``mul_ir`` order in memory - see ``_mul_ir_blocks``; column numbers everywhere else are in the kernels' own order."""
    es = 4 if T == "float" else 2
    in_blocks, res_blocks = _mul_ir_blocks(in_blocks), _mul_ir_blocks(res_blocks)
    blocks = sorted({(p.w_off, p.K, p.N) for p in paths})
    lds_off, off = {}, 0
    for w_off, K, N in blocks:
        R, C = (N, K) if transposed else (K, N)
        lds_off[w_off] = (off, R, C, C * es + 16)
        off += R * (C * es + 16)
    prods = _products(paths, transposed)
    ntiles = width_res // 32
    js = sorted({u[0] for us in prods.values() for u in us})
    A(f"// {name}: {len(prods)} products, {sum(len(u) for u in prods.values())} uses, {off} bytes of weights in LDS")
    A(f"constexpr int k{name}Lds = {off};")
    args = (f"const {T}* __restrict__ W, const {T}* __restrict__ IN, int64_t ldi, const {T}* __restrict__ S, int64_t lds_, "
            + (f"const {T}* __restrict__ G, int64_t ldg, " if rowdot else "") + f"{T}* __restrict__ OUT, int64_t ldo, int Z")
    A(f"__global__ void __launch_bounds__(64 * kWaves, 1) {name}_kernel({args}) {{")
    A("  extern __shared__ __align__(16) char smem[];")
    A("  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;")
    _emit_staging(A, T, blocks, lds_off, transposed, 64 * 8)
    A("  __syncthreads();")
    A("  const int ntiles = (Z + 31) / 32;")
    A("  // tile t goes to block t mod grid, wavefront (t / grid) mod 8: a short batch spreads over every CU first")
    A("  for (int tile = blockIdx.x + gridDim.x * wave; tile < ntiles; tile += gridDim.x * kWaves) {")
    A("    const int zrow = tile * 32 + c;")
    A("    const int64_t z = zrow < Z ? zrow : Z - 1;  // (lanes past the end repeat the last row)")
    for j in js:
        A(f"    const float s{j} = to_f(S[z * lds_ + {j}]);")
    if rowdot:
        for j in js:
            A(f"    float d{j} = 0.f;")
        # this lane's 16 columns of every 32-column tile of the second row operand, held for the whole tile
        used_tiles = sorted({u[2] // 32 + t for (w_off, K, N, _), us in prods.items() for u in us for t in range((N if transposed else K) // 32)})
        for gt in used_tiles:
            A(f"    float g{gt}[16];")
        done = set()
        for gt in used_tiles:
            blk = _block_at(32 * gt, res_blocks, False)
            if blk is None:
                A("#pragma unroll")
                A(f"    for (int a = 0; a < 4; ++a) {{ float gv[4]; load4(G + z * ldg + {32 * gt} + 4 * h + 8 * a, gv); "
                  f"g{gt}[4 * a] = gv[0]; g{gt}[4 * a + 1] = gv[1]; g{gt}[4 * a + 2] = gv[2]; g{gt}[4 * a + 3] = gv[3]; }}")
                continue
            # mul_ir block: the lane's columns 8 a + 4 h + r of tile t with all d components are 4 d consecutive elements
            s0, mul, d, _ = blk
            t = ((32 * gt - s0) % mul) // 32
            if (s0, t) in done:
                continue
            done.add((s0, t))
            for a in range(4):
                A(f"    {{ float gv[{4 * d}];")
                for m in range(d):
                    A(f"      {{ float q4[4]; load4(G + z * ldg + {s0} + ({32 * t + 8 * a} + 4 * h) * {d} + {4 * m}, q4); "
                      f"gv[{4 * m}] = q4[0]; gv[{4 * m + 1}] = q4[1]; gv[{4 * m + 2}] = q4[2]; gv[{4 * m + 3}] = q4[3]; }}")
                for kc in range(d):
                    tile = (s0 + kc * mul) // 32 + t
                    if tile in used_tiles:
                        for r in range(4):
                            A(f"      g{tile}[{4 * a + r}] = gv[{r * d + kc}];")
                A("    }")
    else:
        for t in range(ntiles):
            A(f"    floatx16 o{t} = floatx16{{0}};")
    groups, contraction, request, fragment = _operand_groups(A, prods, transposed, in_blocks, es)
    request(0)
    for gi, (blk, members) in enumerate(groups):
        # the operands of the next group are requested before the products of the current one are worked on
        if gi + 1 < len(groups):
            request(gi + 1)
        for in_off, plist, comp in members:
            ns = contraction[in_off] * es // 64
            A("    {")
            for s2 in range(ns):
                for q in range(2):
                    A(f"      const uint4 xf_{s2}_{q} = {fragment(gi, comp, s2, q)};")
            for w_off, K, N, uses in plist:
                o, R, Cc, RS = lds_off[w_off]
                for t in range(R // 32):
                    A("      {")
                    A("        floatx16 T = floatx16{0};")
                    A(f"        const char* wr = smem + {o} + ({32 * t} + c) * {RS} + h * 32;")
                    for s2 in range(ns):
                        for q in range(2):
                            A(f"        mma_step<{T}>(T, *reinterpret_cast<const uint4*>(wr + {s2 * 64 + q * 16}), xf_{s2}_{q});")
                    for j, coeff, res_off in uses:
                        if rowdot:
                            A("        {")
                            A("          float p = 0.f;")
                            A("#pragma unroll")
                            A(f"          for (int v = 0; v < 16; ++v) p = fmaf(T[v], g{res_off // 32 + t}[v], p);")
                            A(f"          d{j} = fmaf({coeff!r}f, p, d{j});")
                            A(f'          asm volatile("" : "+v"(d{j}));  // finish this use here: a product\'s result is not kept for later')
                            A("        }")
                        else:
                            A(f"        {{ const float sc = {coeff!r}f * s{j};")
                            A("#pragma unroll")
                            A(f"          for (int v = 0; v < 16; ++v) o{res_off // 32 + t}[v] = fmaf(sc, T[v], o{res_off // 32 + t}[v]); }}")
                    A("      }")
                    A("      __builtin_amdgcn_sched_barrier(0);  // keep the loads of later products from piling up ahead of this one")
            A("    }")
    # rows past the end were clamped to the last row: those lanes hold its values and store them again (the same
    # bits to the same place) - a store under a condition would let the compiler sink every use of a product down
    # to it, past all the other products, and keep their results alive in scratch memory
    if rowdot:
        A("    {")
        for j in range(n2):
            if j in js:
                A(f"      {{ const float tot = d{j} + __shfl_xor(d{j}, 32, 64); if (h == 0) store1(OUT + z * ldo + {j}, tot); }}")
            else:
                A(f"      if (h == 0) store1(OUT + z * ldo + {j}, 0.f);")
        A("    }")
    else:
        A("    {")
        A(f"      {T}* op = OUT + z * ldo + 4 * h;")
        done = set()
        for t in range(ntiles):
            blk = _block_at(32 * t, res_blocks, False)
            if blk is None:
                A("#pragma unroll")
                A(f"      for (int a = 0; a < 4; ++a) store4(op + {32 * t} + 8 * a, o{t}[4 * a], o{t}[4 * a + 1], o{t}[4 * a + 2], o{t}[4 * a + 3]);")
                continue
            # mul_ir block: the lane's channels 8 a + 4 h + r of tile tb with their d components are 4 d consecutive elements
            s0, mul, d, _ = blk
            tb = ((32 * t - s0) % mul) // 32
            if (s0, tb) in done:
                continue
            done.add((s0, tb))
            val = lambda a, m: f"o{(s0 + (m % d) * mul) // 32 + tb}[{4 * a + m // d}]"
            for a in range(4):
                for m4 in range(d):
                    A(f"      store4(OUT + z * ldo + {s0} + ({32 * tb + 8 * a} + 4 * h) * {d} + {4 * m4}, "
                      + ", ".join(val(a, 4 * m4 + e) for e in range(4)) + ");")
        A("    }")
    A("  }")
    A("}")
    A("")


def dx12_supported(paths, width_in: int) -> bool:
    """The kernel that forms both input gradients splits the rows of every product between two wavefronts: multiplicities
    of the first operand multiples of 64, its segments covering the row exactly."""
    segs = {}
    for p in paths:
        if p.K % 64 or segs.setdefault(p.a_off, p.K) != p.K:
            return False
    pos = 0
    for a_off in sorted(segs):
        if a_off != pos:
            return False
        pos += segs[a_off]
    return pos == width_in


def _emit_dx12_kernel(A, T: str, paths, width_in: int, n2: int, g_blocks=None, x_blocks=None):
    """Both input gradients from one pass over the products ``R = W_b g_seg^T`` (result rows k = channels of the first
    operand, one batch row per lane): ``dx1[z, a_off + k] += c x2[z, j] R[k, z]`` and ``dx2[z, j] += c sum_k x1[z, a_off + k]
    R[k, z]`` - a quarter of the step's matrix products less than the two separate kernels.  The accumulators of dx1 and the
    row of x1 would not fit one wavefront's registers side by side, so a unit of work is (32-row tile, half of the channels
    of every segment): 64 + 64 registers, two wavefronts per SIMD as in the other kernels, and twice as many units to deal
    out.  The two halves of a row's dx2 go to ``PART[z][half][j]`` (float) and are added by ``dx12_fold_kernel``: no
    atomics, the same bits every run.  ``g_blocks`` / ``x_blocks``: blocks of g / of x1 and dx1 in ``mul_ir`` order."""
    es = 4 if T == "float" else 2
    g_blocks, x_blocks = _mul_ir_blocks(g_blocks), _mul_ir_blocks(x_blocks)
    blocks = sorted({(p.w_off, p.K, p.N) for p in paths})
    lds_off, off = {}, 0
    for w_off, K, N in blocks:
        lds_off[w_off] = (off, K, N, N * es + 16)
        off += K * (N * es + 16)
    prods = _products(paths, False)
    js = sorted({u[0] for us in prods.values() for u in us})
    seg_len = {p.a_off: p.K for p in paths}
    A(f"// dx12: {len(prods)} products, {sum(len(u) for u in prods.values())} uses (each twice), {off} bytes of weights in LDS")
    A(f"constexpr int kdx12Lds = {off};")
    A(f"__global__ void __launch_bounds__(64 * kWaves, 1) dx12_kernel(const {T}* __restrict__ W, const {T}* __restrict__ IN, int64_t ldi, "
      f"const {T}* __restrict__ S, int64_t lds_, const {T}* __restrict__ X, int64_t ldx, {T}* __restrict__ OUT, int64_t ldo, "
      f"float* __restrict__ PART, int Z) {{")
    A("  extern __shared__ __align__(16) char smem[];")
    A("  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 31, h = lane >> 5;")
    _emit_staging(A, T, blocks, lds_off, False, 64 * 8)
    A("  __syncthreads();")
    A("  const int nunits = 2 * ((Z + 31) / 32);")
    A("  // unit u = (tile u / 2, channel half u mod 2) goes to block u mod grid, wavefront (u / grid) mod 8")
    A("  for (int unit = blockIdx.x + gridDim.x * wave; unit < nunits; unit += gridDim.x * kWaves) {")
    A("    const int hlf = unit & 1;")
    A("    const int zrow = (unit >> 1) * 32 + c;")
    A("    const int64_t z = zrow < Z ? zrow : Z - 1;  // (lanes past the end repeat the last row)")
    for j in js:
        A(f"    const float s{j} = to_f(S[z * lds_ + {j}]);")
        A(f"    float d{j} = 0.f;")
    # this unit's channels of segment a_off: tiles tl < K / 64 at channel 32 * (hlf * K / 64 + tl); a lane holds 16 of the 32
    # (8 a + 4 h + r), as accumulator o_<a_off>_<tl> and as the row of x1 x_<a_off>_<tl>
    for a_off, K in sorted(seg_len.items()):
        for tl in range(K // 64):
            A(f"    floatx16 o_{a_off}_{tl} = floatx16{{0}};")
            A(f"    float x_{a_off}_{tl}[16];")
    done = set()
    for a_off, K in sorted(seg_len.items()):
        KH = K // 64
        blk = _block_at(a_off, x_blocks)
        for tl in range(KH):
            if blk is None:
                A("#pragma unroll")
                A(f"    for (int a = 0; a < 4; ++a) {{ float v4[4]; load4(X + z * ldx + {a_off} + 32 * (hlf * {KH} + {tl}) + 4 * h + 8 * a, v4); "
                  f"x_{a_off}_{tl}[4 * a] = v4[0]; x_{a_off}_{tl}[4 * a + 1] = v4[1]; x_{a_off}_{tl}[4 * a + 2] = v4[2]; x_{a_off}_{tl}[4 * a + 3] = v4[3]; }}")
                continue
            # mul_ir block: the lane's channels 8 a + 4 h + r of a tile with all d components are 4 d consecutive elements
            s0, mul, d, _ = blk
            if (s0, tl) in done:
                continue
            done.add((s0, tl))
            for a in range(4):
                A(f"    {{ float gv[{4 * d}];")
                for m in range(d):
                    A(f"      {{ float q4[4]; load4(X + z * ldx + {s0} + (32 * (hlf * {KH} + {tl}) + {8 * a} + 4 * h) * {d} + {4 * m}, q4); "
                      f"gv[{4 * m}] = q4[0]; gv[{4 * m + 1}] = q4[1]; gv[{4 * m + 2}] = q4[2]; gv[{4 * m + 3}] = q4[3]; }}")
                for kc in range(d):
                    for r in range(4):
                        A(f"      x_{s0 + kc * mul}_{tl}[{4 * a + r}] = gv[{r * d + kc}];")
                A("    }")
    # one set of operand registers (two do not fit beside the accumulators and the row of x1, and made no difference when
    # timed): the next group is requested as soon as the last product of the current one has issued its matrix
    # instructions, ahead of that product's uses
    groups, contraction, request, fragment = _operand_groups(A, prods, False, g_blocks, es, single=True)
    request(0)
    for gi, (blk, members) in enumerate(groups):
        for mi, (in_off, plist, comp) in enumerate(members):
            ns = contraction[in_off] * es // 64
            A("    {")
            for s2 in range(ns):
                for q in range(2):
                    A(f"      const uint4 xf_{s2}_{q} = {fragment(gi, comp, s2, q)};")
            for pi, (w_off, K, N, uses) in enumerate(plist):
                o, R, Cc, RS = lds_off[w_off]
                KH = K // 64
                for tl in range(KH):
                    A("      {")
                    A("        floatx16 T = floatx16{0};")
                    A(f"        const char* wr = smem + {o} + (32 * (hlf * {KH} + {tl}) + c) * {RS} + h * 32;")
                    for s2 in range(ns):
                        for q in range(2):
                            A(f"        mma_step<{T}>(T, *reinterpret_cast<const uint4*>(wr + {s2 * 64 + q * 16}), xf_{s2}_{q});")
                    if gi + 1 < len(groups) and mi == len(members) - 1 and pi == len(plist) - 1 and tl == KH - 1:
                        A("        __builtin_amdgcn_sched_barrier(0);")
                        request(gi + 1)
                    for j, coeff, a_off in uses:
                        A(f"        {{ const float sc = {coeff!r}f * s{j};")
                        A("#pragma unroll")
                        A(f"          for (int v = 0; v < 16; ++v) o_{a_off}_{tl}[v] = fmaf(sc, T[v], o_{a_off}_{tl}[v]);")
                        A("          float p = 0.f;")
                        A("#pragma unroll")
                        A(f"          for (int v = 0; v < 16; ++v) p = fmaf(T[v], x_{a_off}_{tl}[v], p);")
                        A(f"          d{j} = fmaf({coeff!r}f, p, d{j});")
                        A(f'          asm volatile("" : "+v"(d{j}));  // finish this use here: a product\'s result is not kept for later')
                        A("        }")
                    A("      }")
                    A("      __builtin_amdgcn_sched_barrier(0);  // keep the loads of later products from piling up ahead of this one")
            A("    }")
    # rows past the end were clamped to the last row: those lanes hold its values and store them again (the same bits to
    # the same place), see the other kernels
    A("    {")
    for j in range(n2):
        if j in js:
            A(f"      {{ const float tot = d{j} + __shfl_xor(d{j}, 32, 64); if (h == 0) PART[(z * 2 + hlf) * {n2} + {j}] = tot; }}")
        else:
            A(f"      if (h == 0) PART[(z * 2 + hlf) * {n2} + {j}] = 0.f;")
    done = set()
    for a_off, K in sorted(seg_len.items()):
        KH = K // 64
        blk = _block_at(a_off, x_blocks)
        for tl in range(KH):
            if blk is None:
                A("#pragma unroll")
                A(f"      for (int a = 0; a < 4; ++a) store4(OUT + z * ldo + {a_off} + 32 * (hlf * {KH} + {tl}) + 4 * h + 8 * a, "
                  f"o_{a_off}_{tl}[4 * a], o_{a_off}_{tl}[4 * a + 1], o_{a_off}_{tl}[4 * a + 2], o_{a_off}_{tl}[4 * a + 3]);")
                continue
            s0, mul, d, _ = blk
            if (s0, tl) in done:
                continue
            done.add((s0, tl))
            val = lambda a, m: f"o_{s0 + (m % d) * mul}_{tl}[{4 * a + m // d}]"
            for a in range(4):
                for m4 in range(d):
                    A(f"      store4(OUT + z * ldo + {s0} + (32 * (hlf * {KH} + {tl}) + {8 * a} + 4 * h) * {d} + {4 * m4}, "
                      + ", ".join(val(a, 4 * m4 + e) for e in range(4)) + ");")
    A("    }")
    A("  }")
    A("}")
    A("")
    A("// dx2[z][j] = PART[z][0][j] + PART[z][1][j]")
    A(f"__global__ void __launch_bounds__(256) dx12_fold_kernel(const float* __restrict__ PART, {T}* __restrict__ OUT2, int64_t ldo2, int Z) {{")
    A(f"  const int64_t e = blockIdx.x * 256ll + threadIdx.x;")
    A(f"  if (e >= int64_t(Z) * {n2}) return;")
    A(f"  const int64_t z = e / {n2};")
    A(f"  const int j = static_cast<int>(e % {n2});")
    A(f"  store1(OUT2 + z * ldo2 + j, PART[(z * 2) * {n2} + j] + PART[(z * 2 + 1) * {n2} + j]);")
    A("}")
    A("")


DW_ROWS = 16  # batch rows per staged tile of the weight-gradient kernel (8 and 32 measured 2 - 3 us slower in float)


def _emit_colmap(A, name: str, blocks):
    """``int name(int p)``: the column in the kernels' own order of the element at column ``p`` of a row in memory."""
    A(f"__device__ __forceinline__ int {name}(int p) {{")
    for s0, mul, d in blocks:
        A(f"  if (p >= {s0} && p < {s0 + mul * d}) {{ const int r = p - {s0}; return {s0} + (r % {d}) * {mul} + r / {d}; }}")
    A("  return p;")
    A("}")


def _emit_dw_kernel(A, T: str, paths, n2: int, width_in: int, width_out: int, x_blocks=None, g_blocks=None):
    """Weight gradient ``dW_b[k, n] = sum_z x1[z, a_off + k] H[z, n]`` with ``H = sum over the uses of (b, a_off) of
    c x2[z, j] g[z, c_off + n]`` formed in registers.  The batch is the contraction: a lane feeds the 32x32x2 MFMA one
    element of ``x1`` (row ``z0 + lane / 32``, column ``a_off + k``) and one of ``H``, no transposition.  A block owns a
    range of rows and stages them 16 at a time through LDS as floats (16-byte global loads issued one tile ahead, two
    LDS buffers, one barrier per tile); its wavefronts own disjoint sets of accumulator tiles (units ``(block, 32 columns
    n)`` dealt out by weight) and read their operands from LDS.  The per-block sums go to ``PART[block]`` for a row sum."""
    es = 4 if T == "float" else 2
    per = 16 // es  # elements per 16-byte load
    R, WX, WG, WS = DW_ROWS, width_in, width_out, 16
    # rows in mul_ir order are put into the kernels' own order while they are staged in LDS (element by element: a tile is
    # 16 rows), everything behind the staging is the same
    x_blocks, g_blocks = _mul_ir_blocks(x_blocks), _mul_ir_blocks(g_blocks)
    if x_blocks:
        _emit_colmap(A, "dw_xcol", x_blocks)
    if g_blocks:
        _emit_colmap(A, "dw_gcol", g_blocks)
    prods = _products(paths, True)  # (w_off, K, N, a_off) -> [(j, coeff, c_off)]
    units = {}  # (w_off, K, N, nt) -> [(a_off, uses)]
    for (w_off, K, N, a_off), uses in prods.items():
        for nt in range(N // 32):
            units.setdefault((w_off, K, N, nt), []).append((a_off, uses))
    weight = lambda u: len(units[u]) * (u[1] // 32)
    waves = [[] for _ in range(8)]
    load = [0] * 8
    for u in sorted(units, key=lambda u: (-weight(u), u)):
        w = min(range(8), key=lambda i: (load[i], i))
        waves[w].append(u)
        load[w] += weight(u)
    # wavefront i runs on SIMD i mod 4: pair the heaviest with the lightest
    order = sorted(range(8), key=lambda i: -load[i])
    slots = [order[0], order[1], order[2], order[3], order[7], order[6], order[5], order[4]]
    tiles_of = [[(w_off, K, N, nt, kt) for (w_off, K, N, nt) in waves[wi] for kt in range(K // 32)] for wi in slots]
    nacc = max(len(t) for t in tiles_of)
    nx, ng = -(-(R * WX // per) // 512), -(-(R * WG // per) // 512)
    # 2-byte elements: x1 stays as it is (rows of WX elements + 64 bytes, read back with the transposing LDS read as
    # bf16 MFMA operands: 16 rows are one 32x32x16 step), g and x2 become floats, x2 column-major (8 rows per read)
    fast16 = es == 2
    XSTR = WX * 2 + 64
    XB = R * XSTR if fast16 else R * WX * 4          # bytes of the x1 region
    SB = XB + R * WG * 4                             # byte offset of the x2 region
    stride = (SB + R * WS * 4) // 4                  # floats per buffer
    A(f"// dw: {len(units)} units over 8 wavefronts, MFMAs per pair of rows: {[load[i] for i in slots]}")
    A(f"constexpr int kdwLds = {2 * stride * 4};")
    A("__device__ __forceinline__ void stage(float* dst, const uint4& v, const float*) { *reinterpret_cast<uint4*>(dst) = v; }")
    A("template <typename TI>")
    A("__device__ __forceinline__ void stage(float* dst, const uint4& v, const TI*) {")
    A("  *reinterpret_cast<float4*>(dst) = make_float4(lo2<TI>(v.x), hi2<TI>(v.x), lo2<TI>(v.y), hi2<TI>(v.y));")
    A("  *reinterpret_cast<float4*>(dst + 4) = make_float4(lo2<TI>(v.z), hi2<TI>(v.z), lo2<TI>(v.w), hi2<TI>(v.w));")
    A("}")
    A(f"__global__ void __launch_bounds__(64 * kWaves, 1) dw_kernel(const {T}* __restrict__ X, int64_t ldx, const {T}* __restrict__ S, int64_t lds_, "
      f"const {T}* __restrict__ G, int64_t ldg, float* __restrict__ PART, int64_t numel, int Z, int chunk) {{")
    A("  extern __shared__ __align__(16) char smem[];")
    A("  float* const lds = reinterpret_cast<float*>(smem);")
    A("  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, c = lane & 31, h = lane >> 5;")
    A("  const int z_begin = blockIdx.x * chunk, z_end = min(Z, z_begin + chunk);")
    A("  if (z_begin >= z_end) return;")
    A("  float* __restrict__ part = PART + static_cast<int64_t>(blockIdx.x) * numel;")
    for a in range(nacc):
        A(f"  floatx16 acc{a} = floatx16{{0}};")
    A(f"  uint4 xr[{nx}], gr[{ng}]; float sr = 0.f;")
    A("  auto fetch = [&](int z0) {  // this thread's pieces of the 16 rows from z0 on (zeros past the range)")
    for name, W, n, src, ld in (("xr", WX, nx, "X", "ldx"), ("gr", WG, ng, "G", "ldg")):
        for i in range(n):
            A(f"    {{ const int s = tid + {512 * i}, row = s / {W // per}, q = s % {W // per}; {name}[{i}] = make_uint4(0, 0, 0, 0);")
            A(f"      if (s < {R * W // per} && z0 + row < z_end) {name}[{i}] = *reinterpret_cast<const uint4*>({src} + static_cast<int64_t>(z0 + row) * {ld} + q * {per}); }}")
    A(f"    {{ const int row = tid / {n2}, j = tid % {n2}; sr = (tid < {R * n2} && z0 + row < z_end) ? to_f(S[static_cast<int64_t>(z0 + row) * lds_ + j]) : 0.f; }}")
    A("  };")
    A("  auto commit = [&](float* buf) {")
    for name, W, n, base in (("xr", WX, nx, 0), ("gr", WG, ng, XB // 4)):
        for i in range(n):
            blocks, cmap = (x_blocks, "dw_xcol") if name == "xr" else (g_blocks, "dw_gcol")
            if blocks:
                A(f"    {{ const int s = tid + {512 * i}, row = s / {W // per}, q = s % {W // per};")
                A(f"      if (s < {R * W // per}) {{")
                A(f"        const uint32_t w4[4] = {{{name}[{i}].x, {name}[{i}].y, {name}[{i}].z, {name}[{i}].w}};")
                A("#pragma unroll")
                A(f"        for (int e = 0; e < {per}; ++e) {{")
                A(f"          const int col = {cmap}(q * {per} + e);")
                if es == 4:
                    A(f"          buf[{base} + row * {W} + col] = __uint_as_float(w4[e]);")
                elif fast16 and name == "xr":
                    A(f"          *reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(buf) + row * {XSTR} + col * 2) = static_cast<uint16_t>(w4[e >> 1] >> (16 * (e & 1)));")
                else:
                    A(f"          buf[{base} + row * {W} + col] = lo2<{T}>(w4[e >> 1] >> (16 * (e & 1)));")
                A("        }")
                A("      }")
                A("    }")
                continue
            if fast16 and name == "xr":
                A(f"    {{ const int s = tid + {512 * i}, row = s / {W // per}, q = s % {W // per}; "
                  f"if (s < {R * W // per}) *reinterpret_cast<uint4*>(reinterpret_cast<char*>(buf) + row * {XSTR} + q * 16) = xr[{i}]; }}")
            else:
                A(f"    {{ const int s = tid + {512 * i}, row = s / {W // per}, q = s % {W // per}; "
                  f"if (s < {R * W // per}) stage(buf + {base} + row * {W} + q * {per}, {name}[{i}], static_cast<const {T}*>(nullptr)); }}")
    if fast16:
        A(f"    if (tid < {R * n2}) buf[{SB // 4} + (tid % {n2}) * {R} + tid / {n2}] = sr;")
    else:
        A(f"    if (tid < {R * n2}) buf[{SB // 4} + (tid / {n2}) * {WS} + tid % {n2}] = sr;")
    A("  };")
    A("  fetch(z_begin);")
    A("  int which = 0;")
    A(f"  for (int z0 = z_begin; z0 < z_end; z0 += {R}, which ^= 1) {{")
    A(f"    float* const buf = lds + which * {stride};")
    A("    commit(buf);")
    A("    __syncthreads();  // (the other buffer is written next time round: everyone has left it by then)")
    A(f"    if (z0 + {R} < z_end) fetch(z0 + {R});")
    A("    switch (wave) {")
    for slot in range(8):
        tl = tiles_of[slot]
        if not tl:
            continue
        acc_of = {t: i for i, t in enumerate(tl)}
        us = waves[slots[slot]]
        js = sorted({j for u in us for _, uses in units[u] for j, _, _ in uses})
        xcols = sorted({a_off + 32 * kt for u in us for a_off, _ in units[u] for kt in range(u[1] // 32)})
        gcols = sorted({c_off + 32 * u[3] for u in us for _, uses in units[u] for _, _, c_off in uses})
        A(f"      case {slot}: {{")
        if fast16:
            A("        typedef shortx4_t __attribute__((address_space(3))) * lptr;")
            A("        const int s16 = lane & 15, g16 = (lane >> 4) & 1;")
            A(f"        const char* xp = reinterpret_cast<const char*>(buf) + (8 * h + (s16 >> 2)) * {XSTR} + (16 * g16 + 4 * (s16 & 3)) * 2;")
            A(f"        const float* gs = buf + {XB // 4} + (8 * h) * {WG} + c;")
            A(f"        const float* st = buf + {SB // 4} + 8 * h;")
            for j in js:
                A(f"        float s{j}[8]; {{ const float4 lo = *reinterpret_cast<const float4*>(st + {j * R}), hi = *reinterpret_cast<const float4*>(st + {j * R + 4}); "
                  f"s{j}[0] = lo.x; s{j}[1] = lo.y; s{j}[2] = lo.z; s{j}[3] = lo.w; s{j}[4] = hi.x; s{j}[5] = hi.y; s{j}[6] = hi.z; s{j}[7] = hi.w; }}")
            for col in gcols:
                A(f"        float g{col}[8];")
                A("#pragma unroll")
                A(f"        for (int e = 0; e < 8; ++e) g{col}[e] = gs[e * {WG} + {col}];")
            for col in xcols:
                A(f"        uint4 x{col}; {{ const uint2 lo = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(xp + {col * 2}))), "
                  f"hi = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lptr)(xp + {col * 2 + 4 * XSTR}))); x{col} = make_uint4(lo.x, lo.y, hi.x, hi.y); }}")
            for (w_off, K, N, nt) in us:
                for a_off, uses in units[(w_off, K, N, nt)]:
                    A("        {")
                    A("          float hv[8];")
                    A("#pragma unroll")
                    terms = " + ".join(f"({coeff!r}f * s{j}[e]) * g{c_off + 32 * nt}[e]" for j, coeff, c_off in uses)
                    A(f"          for (int e = 0; e < 8; ++e) hv[e] = {terms};")
                    A(f"          const uint4 hb = make_uint4(pack2<{T}>(hv[0], hv[1]), pack2<{T}>(hv[2], hv[3]), pack2<{T}>(hv[4], hv[5]), pack2<{T}>(hv[6], hv[7]));")
                    for kt in range(K // 32):
                        a = acc_of[(w_off, K, N, nt, kt)]
                        A(f"          mma_step<{T}>(acc{a}, x{a_off + 32 * kt}, hb);")
                    A("        }")
            A("      } break;")
            continue
        A("#pragma unroll 4")
        A(f"        for (int p = 0; p < {R // 2}; ++p) {{")
        A(f"          const float* xs = buf + (2 * p + h) * {WX} + c;")
        A(f"          const float* gs = buf + {XB // 4} + (2 * p + h) * {WG} + c;")
        A(f"          const float* ss = buf + {SB // 4} + (2 * p + h) * {WS};")
        for j in js:
            A(f"          const float s{j} = ss[{j}];")
        for col in xcols:
            A(f"          const float x{col} = xs[{col}];")
        for col in gcols:
            A(f"          const float g{col} = gs[{col}];")
        for (w_off, K, N, nt) in us:
            for a_off, uses in units[(w_off, K, N, nt)]:
                terms = " + ".join(f"({coeff!r}f * s{j}) * g{c_off + 32 * nt}" for j, coeff, c_off in uses)
                A(f"          {{ const float hv = {terms};")
                for kt in range(K // 32):
                    a = acc_of[(w_off, K, N, nt, kt)]
                    A(f"            acc{a} = __builtin_amdgcn_mfma_f32_32x32x2f32(x{a_off + 32 * kt}, hv, acc{a}, 0, 0, 0);")
                A("          }")
        A("        }")
        A("      } break;")
    A("      default: break;")
    A("    }")
    A("  }")
    A("  switch (wave) {")
    for slot in range(8):
        tl = tiles_of[slot]
        if not tl:
            continue
        A(f"    case {slot}:")
        for a, (w_off, K, N, nt, kt) in enumerate(tl):
            A("#pragma unroll")
            A(f"      for (int v = 0; v < 16; ++v) part[{w_off + 32 * kt * N + 32 * nt} + (8 * (v >> 2) + 4 * h + (v & 3)) * {N} + c] = acc{a}[v];")
        A("      break;")
    A("    default: break;")
    A("  }")
    A("}")
    A("")


def emit_unit(paths, n2: int, width_in: int, width_out: int, T: str, in_blocks=None, out_blocks=None) -> str:
    """``paths``: objects with ``w_off, a_off, j, c_off, K, N, coeff``; ``T``: ``float`` or ``uint16_t`` (bfloat16 bits).
    ``in_blocks`` / ``out_blocks``: ``[(start, mul, d)]`` of the first operand / the output when their rows lie in ``mul_ir``
    order in memory (the reference transposes such rows in front of and behind its kernel,
    ``cuequivariance_torch/operations/tp_fully_connected.py:118-150``); ``None``: ``ir_mul``, the kernels' own order."""
    L = []
    A = L.append
    A("// GENERATED by cuequivariance_amd/codegen/fullyconnected.py - do not edit.")
    A(PRELUDE)
    _emit_kernel(A, "fwd", T, paths, True, False, width_out, n2, in_blocks, out_blocks)
    _emit_kernel(A, "dx1", T, paths, False, False, width_in, n2, out_blocks, in_blocks)
    _emit_kernel(A, "dx2", T, paths, True, True, width_out, n2, in_blocks, out_blocks)
    # (2-byte types keep the two separate kernels: they are bound by memory latency, not by the matrix cores, and ran
    # 39 + 5 us against 22 + 18 us with the one-pass kernel on the 64-channel benchmark product)
    has_dx12 = T == "float" and dx12_supported(paths, width_in)
    if has_dx12:
        _emit_dx12_kernel(A, T, paths, width_in, n2, out_blocks, in_blocks)
    _emit_dw_kernel(A, T, paths, n2, width_in, width_out, in_blocks, out_blocks)
    A("// compute units of the current device (asked once per device: the query is slow)")
    A("int grid_for(int64_t Z) {")
    A("  static int cus_of[64] = {0};")
    A("  int dev = 0;")
    A("  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;")
    A("  int cus = __atomic_load_n(&cus_of[dev], __ATOMIC_RELAXED);")
    A("  if (cus == 0) {")
    A("    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;")
    A("    __atomic_store_n(&cus_of[dev], cus, __ATOMIC_RELAXED);")
    A("  }")
    A("  const int64_t need = (Z + 31) / 32;")
    A("  return static_cast<int>(need < cus ? (need < 1 ? 1 : need) : cus);")
    A("}")
    A("// the LDS limit of a kernel is raised once per device")
    A("template <typename F> int prepare(F fn, int lds, int* done) {")
    A("  int dev = 0;")
    A("  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;")
    A("  if (__atomic_load_n(&done[dev], __ATOMIC_ACQUIRE)) return 0;")
    A("  if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return -1;")
    A("  __atomic_store_n(&done[dev], 1, __ATOMIC_RELEASE);")
    A("  return 0;")
    A("}")
    A("int done_fwd[64], done_dx1[64], done_dx2[64], done_dx12[64], done_dw[64];")
    A("}  // namespace")
    A("")
    A(f'extern "C" int fcj_fwd(int64_t Z, const void* W, const void* X, int64_t ldx, const void* S, int64_t lds_, void* OUT, int64_t ldo, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  if (reinterpret_cast<uintptr_t>(W) % 16) return -1;  // (the weight blocks are staged in 16-byte pieces)")
    A("  if (prepare(fwd_kernel, kfwdLds, done_fwd)) return -1;")
    A(f"  hipLaunchKernelGGL(fwd_kernel, dim3(grid_for(Z)), dim3(64 * kWaves), kfwdLds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(W), "
      f"static_cast<const {T}*>(X), ldx, static_cast<const {T}*>(S), lds_, static_cast<{T}*>(OUT), ldo, static_cast<int>(Z));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    A(f'extern "C" int fcj_dx1(int64_t Z, const void* W, const void* G, int64_t ldg, const void* S, int64_t lds_, void* DX1, int64_t ldd, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  if (reinterpret_cast<uintptr_t>(W) % 16) return -1;  // (the weight blocks are staged in 16-byte pieces)")
    A("  if (prepare(dx1_kernel, kdx1Lds, done_dx1)) return -1;")
    A(f"  hipLaunchKernelGGL(dx1_kernel, dim3(grid_for(Z)), dim3(64 * kWaves), kdx1Lds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(W), "
      f"static_cast<const {T}*>(G), ldg, static_cast<const {T}*>(S), lds_, static_cast<{T}*>(DX1), ldd, static_cast<int>(Z));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    A(f'extern "C" int fcj_dx2(int64_t Z, const void* W, const void* X, int64_t ldx, const void* S, int64_t lds_, const void* G, int64_t ldg, void* DX2, int64_t ld2, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  if (reinterpret_cast<uintptr_t>(W) % 16) return -1;  // (the weight blocks are staged in 16-byte pieces)")
    A("  if (prepare(dx2_kernel, kdx2Lds, done_dx2)) return -1;")
    A(f"  hipLaunchKernelGGL(dx2_kernel, dim3(grid_for(Z)), dim3(64 * kWaves), kdx2Lds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(W), "
      f"static_cast<const {T}*>(X), ldx, static_cast<const {T}*>(S), lds_, static_cast<const {T}*>(G), ldg, static_cast<{T}*>(DX2), ld2, static_cast<int>(Z));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    A("// both input gradients in one pass; PART: 2 * n2 floats per row of scratch.  -2: this product has no such kernel")
    A(f'extern "C" int fcj_dx12(int64_t Z, const void* W, const void* G, int64_t ldg, const void* S, int64_t lds_, const void* X, int64_t ldx, '
      f'void* DX1, int64_t ldd, void* DX2, int64_t ld2, float* PART, void* stream) {{')
    if has_dx12:
        A("  if (Z <= 0) return 0;")
        A("  if (reinterpret_cast<uintptr_t>(W) % 16) return -1;  // (the weight blocks are staged in 16-byte pieces)")
        A("  if (prepare(dx12_kernel, kdx12Lds, done_dx12)) return -1;")
        A("  const int64_t units = 2 * ((Z + 31) / 32);")
        A("  const int cus = grid_for(int64_t(1) << 40);")
        A(f"  hipLaunchKernelGGL(dx12_kernel, dim3(static_cast<unsigned>(units < cus ? units : cus)), dim3(64 * kWaves), kdx12Lds, static_cast<hipStream_t>(stream), "
          f"static_cast<const {T}*>(W), static_cast<const {T}*>(G), ldg, static_cast<const {T}*>(S), lds_, static_cast<const {T}*>(X), ldx, "
          f"static_cast<{T}*>(DX1), ldd, PART, static_cast<int>(Z));")
        A(f"  hipLaunchKernelGGL(dx12_fold_kernel, dim3(static_cast<unsigned>((Z * {n2} + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream), "
          f"PART, static_cast<{T}*>(DX2), ld2, static_cast<int>(Z));")
        A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    else:
        A("  return -2;")
    A("}")
    A("// number of per-block partial sums fcj_dw writes for a batch of Z rows (the caller sizes PART with it)")
    A('extern "C" int fcj_dw_blocks(int64_t Z) {')
    A("  if (Z <= 0) return 0;")
    A("  const int g = grid_for(Z);")
    A(f"  const int64_t chunk = ((Z + g - 1) / g + {DW_ROWS - 1}) / {DW_ROWS} * {DW_ROWS};")
    A("  return static_cast<int>((Z + chunk - 1) / chunk);")
    A("}")
    A(f'extern "C" int fcj_dw(int64_t Z, const void* X, int64_t ldx, const void* S, int64_t lds_, const void* G, int64_t ldg, float* PART, int64_t numel, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  const int g = grid_for(Z);")
    A(f"  const int64_t chunk = ((Z + g - 1) / g + {DW_ROWS - 1}) / {DW_ROWS} * {DW_ROWS};")
    A("  const int blocks = static_cast<int>((Z + chunk - 1) / chunk);")
    A("  if (prepare(dw_kernel, kdwLds, done_dw)) return -1;")
    A(f"  hipLaunchKernelGGL(dw_kernel, dim3(blocks), dim3(64 * kWaves), kdwLds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(X), ldx, "
      f"static_cast<const {T}*>(S), lds_, static_cast<const {T}*>(G), ldg, PART, numel, static_cast<int>(Z), static_cast<int>(chunk));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    return "\n".join(L) + "\n"
