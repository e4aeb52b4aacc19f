// Combine stage: expert-ordered rows back to token order.
//
// The reference scatters a finished tile row t to activations[tokenIndices[t], :] by vector copy
// (CombineMode::single, top-1) or by vector atomic add (CombineMode::multithreaded, top-k)
// (combine.cuh:170-186, VAA at combine.cuh:19-93); gate weights are not applied there and the atomic order
// is not deterministic.  This kernel is the gather form of the same data movement:
//   out[t,:] = sum over ranks r (ascending) of topk_w[t,r] * y[pair_row[t,r], :]
// accumulated in fp32 and rounded once; pairs with pair_row < 0 (dropped) contribute nothing.  With k = 1
// and unit weights it is exactly the reference's single-mode copy.
#include "combine_core.hpp"

namespace moe355 {
namespace {

// grid = (S, ceil(H / (256*8))) for the 16-bit types; each thread owns 8 consecutive columns
template <typename T16>
__global__ __launch_bounds__(256) void combine_16_kernel(const uint16_t* __restrict__ y,
                                                         const int32_t* __restrict__ pair_row,
                                                         const float* __restrict__ topk_w, int k, int H,
                                                         uint16_t* __restrict__ out, const int32_t* __restrict__ taken) {
    const int t = blockIdx.x;
    if (taken && taken[(size_t)blockIdx.y * gridDim.x + t]) return;   // combined inside the FFN queue kernel
    const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (c >= H) return;
    combine_token_16<T16, false>(y, pair_row, topk_w, t, k, H, c, out);
}

__global__ __launch_bounds__(256) void combine_f32_kernel(const float* __restrict__ y,
                                                          const int32_t* __restrict__ pair_row,
                                                          const float* __restrict__ topk_w, int k, int H,
                                                          float* __restrict__ out, const int32_t* __restrict__ taken) {
    const int t = blockIdx.x;
    if (taken && taken[(size_t)blockIdx.y * gridDim.x + t]) return;   // combined inside the FFN queue kernel
    const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c >= H) return;
    combine_token_f32<false>(y, pair_row, topk_w, t, k, H, c, out);
}

}  // namespace

hipError_t launch_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w, int S, int k, int H,
                          int act_dtype, void* out, const int32_t* taken, hipStream_t st) {
    if (S <= 0) return hipSuccess;
    if (act_dtype == MOE_DTYPE_F32) {
        const dim3 grid(S, (H + 256 * 4 - 1) / (256 * 4));
        combine_f32_kernel<<<grid, 256, 0, st>>>((const float*)y_rows, pair_row, topk_w, k, H, (float*)out, taken);
    } else {
        const dim3 grid(S, (H + 256 * 8 - 1) / (256 * 8));
        if (act_dtype == MOE_DTYPE_FP16)
            combine_16_kernel<f16_s><<<grid, 256, 0, st>>>((const uint16_t*)y_rows, pair_row, topk_w, k, H, (uint16_t*)out, taken);
        else
            combine_16_kernel<bf16_s><<<grid, 256, 0, st>>>((const uint16_t*)y_rows, pair_row, topk_w, k, H, (uint16_t*)out, taken);
    }
    return hipGetLastError();
}

}  // namespace moe355
