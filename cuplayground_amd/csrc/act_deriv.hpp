// The derivative of the activation for 16-bit layers, as the one piece of arithmetic that the stand-alone pass
// (moe_act_backward) and the epilogue of the fused data gradient (moe_expert_gemm_act_backward) both inline: dh comes in as
// the 16-bit value the data gradient stores, the result is rounded once on store, so the two paths agree bit for bit.
// Hardware exp2 and reciprocal (about 1 ulp each in fp32, far below the 16-bit rounding of the result) in place of the
// library expf / erff / division: inside a tile's epilogue every operation is paid for by the one wavefront a SIMD holds.
// Contraction is switched off and the fused multiply-adds are spelled out: the compiler must not pair the products and
// sums differently in the two places.
#pragma once

#include "moe_internal.hpp"

namespace moe355 {

// The fp32 result as a value of its own.  Without this the compiler may merge the last product with the caller's
// narrowing to fp16 into one mixed-precision instruction (rounded once, not twice) -- and does so in the stand-alone
// pass, whose narrowing is scalar, but not in the epilogue, whose narrowing is packed: 1 result in 17000 then differs
// by a unit of the last place.
__device__ __forceinline__ float settled(float v) {
    asm volatile("" : "+v"(v));
    return v;
}

// h = silu(g) * u:  du = dh * silu(g),  dg = dh * u * s * (1 + g * (1 - s)),  s = sigmoid(g)
__device__ __forceinline__ void dswiglu16(float d, float u, float g, float& du, float& dg) {
#pragma clang fp contract(off)
    const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
    du = settled(d * (g * s));
    const float one_minus = 1.0f - s;
    dg = settled((d * u) * (s * __builtin_fmaf(g, one_minus, 1.0f)));
}

// gelu(u) = u * Phi(u):  du = dh * (Phi(u) + u * phi(u)); Phi through erfc(x) = t (a1 + t (a2 + ... t a5)) exp(-x^2),
// t = 1 / (1 + p x), x = |u| / sqrt 2 (Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7), phi from the same exponential.
__device__ __forceinline__ float dgelu16(float d, float u) {
#pragma clang fp contract(off)
    const float x = fabsf(u) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, x, 1.0f));
    float q = __builtin_fmaf(1.061405429f, t, -1.453152027f);
    q = __builtin_fmaf(q, t, 1.421413741f);
    q = __builtin_fmaf(q, t, -0.284496736f);
    q = __builtin_fmaf(q, t, 0.254829592f);
    const float e = __builtin_amdgcn_exp2f((u * u) * -0.72134752044448170368f);     // exp(-u^2 / 2)
    const float half_erfc = (0.5f * (q * t)) * e;
    const float cdf = u >= 0.0f ? 1.0f - half_erfc : half_erfc;
    const float pdf = 0.39894228040143267794f * e;
    return settled(d * __builtin_fmaf(u, pdf, cdf));
}

__device__ __forceinline__ float drelu16(float d, float u) { return u > 0.0f ? d : 0.0f; }

}  // namespace moe355
