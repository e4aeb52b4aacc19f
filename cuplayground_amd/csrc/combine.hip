// Combine stage: expert-ordered rows back to token order.
//
// The reference scatters a finished tile row t to activations[tokenIndices[t], :] by vector copy
// (CombineMode::single, top-1) or by vector atomic add (CombineMode::multithreaded, top-k)
// (combine.cuh:170-186, VAA at combine.cuh:19-93); gate weights are not applied there and the atomic order
// is not deterministic.  This kernel is the gather form of the same data movement:
//   out[t,:] = sum over ranks r (ascending) of topk_w[t,r] * y[pair_row[t,r], :]
// accumulated in fp32 and rounded once; pairs with pair_row < 0 (dropped) contribute nothing.  With k = 1
// and unit weights it is exactly the reference's single-mode copy.
#include "moe_internal.hpp"

namespace moe355 {
namespace {

__device__ __forceinline__ uint32_t pack16x2(float lo, float hi, bf16_s) {
    // round to nearest even, the rounding the oracle and torch use for bf16
    uint32_t a = __float_as_uint(lo), b = __float_as_uint(hi);
    a += 0x7FFFu + ((a >> 16) & 1u);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return (a >> 16) | (b & 0xFFFF0000u);
}
__device__ __forceinline__ uint32_t pack16x2(float lo, float hi, f16_s) {
    const uint32_t a = __builtin_bit_cast(uint16_t, (_Float16)lo), b = __builtin_bit_cast(uint16_t, (_Float16)hi);   // RNE
    return a | (b << 16);
}
__device__ __forceinline__ float lo16(uint32_t w, bf16_s) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi16(uint32_t w, bf16_s) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ __forceinline__ float lo16(uint32_t w, f16_s) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu)); }
__device__ __forceinline__ float hi16(uint32_t w, f16_s) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }

// grid = (S, ceil(H / (256*8))) for the 16-bit types; each thread owns 8 consecutive columns
template <typename T16>
__global__ __launch_bounds__(256) void combine_16_kernel(const uint16_t* __restrict__ y,
                                                         const int32_t* __restrict__ pair_row,
                                                         const float* __restrict__ topk_w, int k, int H,
                                                         uint16_t* __restrict__ out) {
    const int t = blockIdx.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (c >= H) return;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (int r = 0; r < k; ++r) {
        const int row = pair_row[(size_t)t * k + r];
        if (row < 0) continue;
        const float w = topk_w[(size_t)t * k + r];
        const uint4 v = *reinterpret_cast<const uint4*>(y + (size_t)row * H + c);
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = acc[2 * i] + w * lo16(u[i], T16{});
            acc[2 * i + 1] = acc[2 * i + 1] + w * hi16(u[i], T16{});
        }
    }
    uint4 o;
    o.x = pack16x2(acc[0], acc[1], T16{});
    o.y = pack16x2(acc[2], acc[3], T16{});
    o.z = pack16x2(acc[4], acc[5], T16{});
    o.w = pack16x2(acc[6], acc[7], T16{});
    *reinterpret_cast<uint4*>(out + (size_t)t * H + c) = o;
}

__global__ __launch_bounds__(256) void combine_f32_kernel(const float* __restrict__ y,
                                                          const int32_t* __restrict__ pair_row,
                                                          const float* __restrict__ topk_w, int k, int H,
                                                          float* __restrict__ out) {
    const int t = blockIdx.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c >= H) return;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int r = 0; r < k; ++r) {
        const int row = pair_row[(size_t)t * k + r];
        if (row < 0) continue;
        const float w = topk_w[(size_t)t * k + r];
        const float4 v = *reinterpret_cast<const float4*>(y + (size_t)row * H + c);
        acc.x = acc.x + w * v.x;
        acc.y = acc.y + w * v.y;
        acc.z = acc.z + w * v.z;
        acc.w = acc.w + w * v.w;
    }
    *reinterpret_cast<float4*>(out + (size_t)t * H + c) = acc;
}

}  // namespace

hipError_t launch_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w, int S, int k, int H,
                          int act_dtype, void* out, hipStream_t st) {
    if (S <= 0) return hipSuccess;
    if (act_dtype == MOE_DTYPE_F32) {
        const dim3 grid(S, (H + 256 * 4 - 1) / (256 * 4));
        combine_f32_kernel<<<grid, 256, 0, st>>>((const float*)y_rows, pair_row, topk_w, k, H, (float*)out);
    } else {
        const dim3 grid(S, (H + 256 * 8 - 1) / (256 * 8));
        if (act_dtype == MOE_DTYPE_FP16)
            combine_16_kernel<f16_s><<<grid, 256, 0, st>>>((const uint16_t*)y_rows, pair_row, topk_w, k, H, (uint16_t*)out);
        else
            combine_16_kernel<bf16_s><<<grid, 256, 0, st>>>((const uint16_t*)y_rows, pair_row, topk_w, k, H, (uint16_t*)out);
    }
    return hipGetLastError();
}

}  // namespace moe355
