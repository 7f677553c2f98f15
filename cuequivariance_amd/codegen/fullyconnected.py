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

template <typename TI>
__device__ __forceinline__ void mma_step(floatx16& acc, const uint4& a, const uint4& b) {
  if constexpr (sizeof(TI) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
  } else {
    const float* pa = reinterpret_cast<const float*>(&a);
    const float* pb = reinterpret_cast<const float*>(&b);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[e], pb[e], acc, 0, 0, 0);
  }
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const floatx2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(uint16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }
// four adjacent elements of a row
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const uint16_t* p, float (&v)[4]) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
  v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) { *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d); }
__device__ __forceinline__ void store4(uint16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(a, b), pack_bf16(c, d));
}
__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
__device__ __forceinline__ void store1(uint16_t* p, float v) { *p = static_cast<uint16_t>(pack_bf16(v, 0.f) & 0xffffu); }

constexpr int kWaves = 8;
'''


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


def _emit_kernel(A, name: str, T: str, paths, transposed: bool, rowdot: bool, width_res: int, n2: int):
    """One kernel.  ``transposed``: the blocks sit in LDS as W^T (rows n, contraction k).  ``rowdot``: instead of
    accumulating the scaled products into result columns, they are multiplied element-wise with G and summed per row."""
    es = 4 if T == "float" else 2
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
    for w_off, K, N in blocks:
        o, R, C, RS = lds_off[w_off]
        if transposed:  # global block is K x N (k major): element (k, n) goes to row n, column k
            A(f"  for (int e = tid; e < {K * N}; e += 64 * kWaves) {{ const int k = e / {N}, n = e % {N}; "
              f"*reinterpret_cast<{T}*>(smem + {o} + n * {RS} + k * {es}) = W[{w_off} + e]; }}")
        else:
            A(f"  for (int e = tid; e < {K * N}; e += 64 * kWaves) {{ const int k = e / {N}, n = e % {N}; "
              f"*reinterpret_cast<{T}*>(smem + {o} + k * {RS} + n * {es}) = W[{w_off} + e]; }}")
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
            A("#pragma unroll")
            A(f"    for (int a = 0; a < 4; ++a) {{ float gv[4]; load4(G + z * ldg + {32 * gt} + 4 * h + 8 * a, gv); "
              f"g{gt}[4 * a] = gv[0]; g{gt}[4 * a + 1] = gv[1]; g{gt}[4 * a + 2] = gv[2]; g{gt}[4 * a + 3] = gv[3]; }}")
    else:
        for t in range(ntiles):
            A(f"    floatx16 o{t} = floatx16{{0}};")
    # products grouped by operand segment so that its fragments are loaded once
    by_seg = OrderedDict()
    for (w_off, K, N, in_off), uses in prods.items():
        by_seg.setdefault(in_off, []).append((w_off, K, N, uses))
    for in_off, plist in by_seg.items():
        C = (plist[0][1] if transposed else plist[0][2])
        assert all((p[1] if transposed else p[2]) == C for p in plist), "one operand segment, one contraction length"
        ns = C * es // 64
        A("    {")
        A(f"      uint4 xf[{ns}][2];")
        A(f"      const {T}* xp = IN + z * ldi + {in_off};")
        for s2 in range(ns):
            for q in range(2):
                A(f"      xf[{s2}][{q}] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(xp) + {s2 * 64} + h * 32 + {q * 16});")
        for w_off, K, N, uses in plist:
            o, R, Cc, RS = lds_off[w_off]
            for t in range(R // 32):
                A("      {")
                A("        floatx16 T = floatx16{0};")
                A(f"        const char* wr = smem + {o} + ({32 * t} + c) * {RS} + h * 32;")
                for s2 in range(ns):
                    for q in range(2):
                        A(f"        mma_step<{T}>(T, *reinterpret_cast<const uint4*>(wr + {s2 * 64 + q * 16}), xf[{s2}][{q}]);")
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
        for t in range(ntiles):
            A("#pragma unroll")
            A(f"      for (int a = 0; a < 4; ++a) store4(op + {32 * t} + 8 * a, o{t}[4 * a], o{t}[4 * a + 1], o{t}[4 * a + 2], o{t}[4 * a + 3]);")
        A("    }")
    A("  }")
    A("}")
    A("")


def emit_unit(paths, n2: int, width_in: int, width_out: int, T: str) -> str:
    """``paths``: objects with ``w_off, a_off, j, c_off, K, N, coeff``; ``T``: ``float`` or ``uint16_t`` (bfloat16 bits)."""
    L = []
    A = L.append
    A("// GENERATED by cuequivariance_amd/codegen/fullyconnected.py - do not edit.")
    A(PRELUDE)
    _emit_kernel(A, "fwd", T, paths, True, False, width_out, n2)
    _emit_kernel(A, "dx1", T, paths, False, False, width_in, n2)
    _emit_kernel(A, "dx2", T, paths, True, True, width_out, n2)
    A("int grid_for(int64_t Z) {")
    A("  int dev = 0, cus = 256; hipDeviceProp_t p;")
    A("  if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;")
    A("  const int64_t need = (Z + 31) / 32;")
    A("  return static_cast<int>(need < cus ? (need < 1 ? 1 : need) : cus);")
    A("}")
    A("template <typename F> int prepare(F fn, int lds) {")
    A("  return hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess ? 0 : -1;")
    A("}")
    A("}  // namespace")
    A("")
    A(f'extern "C" int fcj_fwd(int64_t Z, const void* W, const void* X, int64_t ldx, const void* S, int64_t lds_, void* OUT, int64_t ldo, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  if (prepare(fwd_kernel, kfwdLds)) return -1;")
    A(f"  hipLaunchKernelGGL(fwd_kernel, dim3(grid_for(Z)), dim3(64 * kWaves), kfwdLds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(W), "
      f"static_cast<const {T}*>(X), ldx, static_cast<const {T}*>(S), lds_, static_cast<{T}*>(OUT), ldo, static_cast<int>(Z));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    A(f'extern "C" int fcj_dx1(int64_t Z, const void* W, const void* G, int64_t ldg, const void* S, int64_t lds_, void* DX1, int64_t ldd, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  if (prepare(dx1_kernel, kdx1Lds)) return -1;")
    A(f"  hipLaunchKernelGGL(dx1_kernel, dim3(grid_for(Z)), dim3(64 * kWaves), kdx1Lds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(W), "
      f"static_cast<const {T}*>(G), ldg, static_cast<const {T}*>(S), lds_, static_cast<{T}*>(DX1), ldd, static_cast<int>(Z));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    A(f'extern "C" int fcj_dx2(int64_t Z, const void* W, const void* X, int64_t ldx, const void* S, int64_t lds_, const void* G, int64_t ldg, void* DX2, int64_t ld2, void* stream) {{')
    A("  if (Z <= 0) return 0;")
    A("  if (prepare(dx2_kernel, kdx2Lds)) return -1;")
    A(f"  hipLaunchKernelGGL(dx2_kernel, dim3(grid_for(Z)), dim3(64 * kWaves), kdx2Lds, static_cast<hipStream_t>(stream), static_cast<const {T}*>(W), "
      f"static_cast<const {T}*>(X), ldx, static_cast<const {T}*>(S), lds_, static_cast<const {T}*>(G), ldg, static_cast<{T}*>(DX2), ld2, static_cast<int>(Z));")
    A("  return hipGetLastError() == hipSuccess ? 0 : -1;")
    A("}")
    return "\n".join(L) + "\n"
