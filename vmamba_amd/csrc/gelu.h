// Exact (erf) GELU for 16-bit activations, shared by the kernels that fuse it.
//   * bf16: the argument is a bf16 value, so gelu(x) = 0.5 x + |x| E(|x|), E(x) = 0.5 erf(x / sqrt 2), with E read from
//     a 2176-entry fp32 table (copied into LDS by the kernel) indexed by the bf16 bit pattern clamped to [2^-14, 8)
//     (below, |x| E is under 1e-4 of 0.5 |x|; above, E is 0.5 to fp32 precision).  The table is generated in double
//     precision at build time (gen_gelu_table.py);
//   * fp16: erf from Abramowitz-Stegun 7.1.26 (absolute error 1.5e-7, far below 16-bit rounding).
#pragma once

#include "ss2d_common.h"

namespace ss2d {

#include "gelu_table.inc"

constexpr int kGeluEntries = kGeluHiBits - kGeluLoBits;

__device__ __forceinline__ float gelu_erf(float x) {
    const float z = fabsf(x) * 0.70710678118654752f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
    float poly = fmaf(1.061405429f, t, -1.453152027f);
    poly = fmaf(poly, t, 1.421413741f);
    poly = fmaf(poly, t, -0.284496736f);
    poly = fmaf(poly, t, 0.254829592f);
    const float e = __builtin_amdgcn_exp2f(z * z * -1.4426950408889634f);
    const float erf_abs = fmaf(-poly * t, e, 1.0f);                   // erf(|x| / sqrt 2)
    const float erf_x = __builtin_copysignf(erf_abs, x);
    return 0.5f * x * (1.0f + erf_x);
}

// GELU of two packed 16-bit values, result packed and rounded again; tbl: the table in LDS (bf16 only)
__device__ __forceinline__ uint32_t gelu_pair(bf16_t, uint32_t w, const float *tbl) {
    const uint32_t a0 = w & 0x7fffu, a1 = (w >> 16) & 0x7fffu;
    const uint32_t m0 = min(max(a0, (uint32_t)kGeluLoBits), (uint32_t)kGeluHiBits - 1u) - kGeluLoBits;
    const uint32_t m1 = min(max(a1, (uint32_t)kGeluLoBits), (uint32_t)kGeluHiBits - 1u) - kGeluLoBits;
    const float e0 = tbl[m0], e1 = tbl[m1];
    const float x0 = bits_to_f32(w << 16), x1 = bits_to_f32(w & 0xffff0000u);
    return pack2_from_f32<bf16_t>(fmaf(fabsf(x0), e0, 0.5f * x0), fmaf(fabsf(x1), e1, 0.5f * x1));
}
__device__ __forceinline__ uint32_t gelu_pair(f16_t, uint32_t w, const float *) {
    return pack2_from_f32<f16_t>(gelu_erf(unpack_lo<f16_t>(w)), gelu_erf(unpack_hi<f16_t>(w)));
}

}  // namespace ss2d
