// Weight preparation for the fp8 path: OCP e4m3 values with one fp32 scale per 128x128 block.
//
// The reference has no quantised dtype (torch_dtype stops at fp16, aristos_config.schema.json:49-53); the format
// is this library's: for every 128x128 block of a row-major [N,K] matrix, scale = amax / 448 (1 for an all-zero
// block) and q = e4m3(w / scale), round to nearest even, saturating at +-448.  Scales are stored
// [N/128, K/128] row-major per matrix -- the layout the fp8 FFN kernel reads.
#include "moe_internal.hpp"

namespace moe355 {
namespace {

// fp32 -> e4m3 (1-4-3, bias 7, no infinities, 0x7F = NaN), round to nearest even, saturating.
__device__ __forceinline__ uint32_t f32_to_e4m3(float v) {
    const uint32_t u = __float_as_uint(v);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t mag = u & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return sign | 0x7Fu;
    const float a = __uint_as_float(mag);
    if (a >= 448.0f) return sign | 0x7Eu;
    if (a < 0.015625f) return sign | (uint32_t)__builtin_rintf(a * 512.0f);   // units of 2^-9; 8 = smallest normal
    int e = (int)(mag >> 23) - 127;                                           // -6 .. 8
    uint32_t m = (mag >> 20) & 7u;
    const uint32_t rem = mag & 0xFFFFFu;
    if (rem > 0x80000u || (rem == 0x80000u && (m & 1u))) ++m;
    if (m == 8u) { m = 0u; ++e; }
    uint32_t code = ((uint32_t)(e + 7) << 3) | m;
    if (code > 0x7Eu) code = 0x7Eu;
    return sign | code;
}

__device__ __forceinline__ float load_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float load_as_f32(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }

// One workgroup per 128x128 block; thread t owns the 8-element column group (t & 15) of rows (t >> 4) + 16*i.
template <typename T>
__global__ __launch_bounds__(256) void quant_block128_kernel(const T* __restrict__ w, uint8_t* __restrict__ q,
                                                             float* __restrict__ scales, int64_t N, int64_t K) {
    __shared__ float s_max[4];
    const int kb = (int)(K / 128);
    const int64_t mat = blockIdx.z;
    const int bi = blockIdx.y, bj = blockIdx.x;
    const T* src = w + mat * N * K + (int64_t)bi * 128 * K + (int64_t)bj * 128;
    uint8_t* dst = q + mat * N * K + (int64_t)bi * 128 * K + (int64_t)bj * 128;
    const int tid = threadIdx.x, cg = tid & 15, r0 = tid >> 4;
    float v[8][8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const T* row = src + (int64_t)(r0 + 16 * i) * K + cg * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[i][e] = load_as_f32(row + e);
            amax = fmaxf(amax, fabsf(v[i][e]));
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    if ((tid & 63) == 0) s_max[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    const float s = amax > 0.0f ? amax / 448.0f : 1.0f;
    if (tid == 0) scales[mat * (N / 128) * kb + (int64_t)bi * kb + bj] = s;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo |= f32_to_e4m3(v[i][e] / s) << (8 * e);
            hi |= f32_to_e4m3(v[i][e + 4] / s) << (8 * e);
        }
        uint2 o = {lo, hi};
        *reinterpret_cast<uint2*>(dst + (int64_t)(r0 + 16 * i) * K + cg * 8) = o;
    }
}

// The inverse, for layers that run the 16-bit tile GEMM on e4m3 weights: out = bf16(e4m3(q) * scale of its block), round
// to nearest even (the product of a 4-bit significand and an fp32 scale is rounded once, to 8 bits: 2^-9 relative,
// a thirty-second of the e4m3 rounding step).  A lane widens 16 consecutive codes of one row (one scale block).
__global__ __launch_bounds__(256) void widen_block128_kernel(const uint8_t* __restrict__ q, const float* __restrict__ scales,
                                                             uint16_t* __restrict__ out, int64_t rows, int64_t N,
                                                             int64_t K) {
    const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;   // 16 codes each
    const int64_t per_row = K / 16;
    if (chunk >= rows * per_row) return;
    const int64_t row = chunk / per_row, c0 = (chunk - row * per_row) * 16;
    const int64_t mat = row / N, r = row - mat * N;
    const float s = scales[(mat * (N / 128) + r / 128) * (K / 128) + c0 / 128];
    const uint4 in = *reinterpret_cast<const uint4*>(q + row * K + c0);
    const uint32_t w[4] = {in.x, in.y, in.z, in.w};
    uint32_t o[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int hi = 0; hi < 2; ++hi) {
            const auto f = hi ? __builtin_amdgcn_cvt_pk_f32_fp8(w[i], true) : __builtin_amdgcn_cvt_pk_f32_fp8(w[i], false);
            uint32_t b[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const uint32_t u = __float_as_uint(f[e] * s);
                b[e] = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
            }
            o[2 * i + hi] = b[0] | (b[1] << 16);
        }
    }
    uint4* dst = reinterpret_cast<uint4*>(out + row * K + c0);
    dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
    dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

// Activation rows for the e4m3 x e4m3 products: one fp32 scale per (row, 128 columns), scale = amax / 448 over that piece
// of the row (1 when it is all zero), q = e4m3(x / scale).  x is bf16 [rows, K], K a multiple of 128.  Sixteen lanes
// share a piece (8 values each); the maximum travels over xor 8, 4, 2, 1, which stays inside the sixteen.  limit
// (may be null): a device word holding the number of rows that matter; rows behind it are skipped.
__global__ __launch_bounds__(256) void quant_rows128_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ q,
                                                            float* __restrict__ scales, int64_t rows, int64_t K,
                                                            const int32_t* __restrict__ limit) {
    const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;   // 8 values each
    const int64_t per_row = K / 8;
    const int64_t row = chunk / per_row, c8 = chunk - row * per_row;
    if (row >= rows || (limit && row >= *limit)) return;              // K % 128 == 0: the sixteen lanes of a piece agree
    const uint4 in = *reinterpret_cast<const uint4*>(x + row * K + c8 * 8);
    const uint32_t w[4] = {in.x, in.y, in.z, in.w};
    float v[8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        amax = fmaxf(amax, fmaxf(fabsf(v[2 * i]), fabsf(v[2 * i + 1])));   // fmaxf passes over a NaN, as the comparison of the restatement does
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    const float s = amax > 0.0f ? amax / 448.0f : 1.0f;
    if ((c8 & 15) == 0) scales[row * (K / 128) + c8 / 16] = s;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        lo |= f32_to_e4m3(v[e] / s) << (8 * e);
        hi |= f32_to_e4m3(v[e + 4] / s) << (8 * e);
    }
    *reinterpret_cast<uint2*>(q + row * K + c8 * 8) = uint2{lo, hi};
}

}  // namespace

hipError_t launch_quant_rows128(const void* x, void* q, float* scales, int64_t rows, int64_t K, const int32_t* limit,
                                hipStream_t st) {
    const int64_t chunks = rows * (K / 8);
    if (chunks <= 0) return hipSuccess;
    quant_rows128_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, st>>>((const uint16_t*)x, (uint8_t*)q, scales, rows, K, limit);
    return hipGetLastError();
}

hipError_t launch_widen_block128(const void* q, const float* scales, void* out, int64_t matrices, int64_t N, int64_t K,
                                 hipStream_t st) {
    const int64_t chunks = matrices * N * (K / 16);
    widen_block128_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, st>>>((const uint8_t*)q, scales, (uint16_t*)out,
                                                                             matrices * N, N, K);
    return hipGetLastError();
}

}  // namespace moe355

using namespace moe355;

extern "C" int moe_quant_block128(const void* w, int32_t src_dtype, int64_t matrices, int64_t N, int64_t K, void* q,
                                  float* scales, void* stream) {
    if (!w || !q || !scales || matrices < 1 || N < 128 || K < 128 || (N % 128) || (K % 128)) return MOE_ERR_BAD_ARGUMENT;
    if (src_dtype != MOE_DTYPE_F32 && src_dtype != MOE_DTYPE_BF16) return MOE_ERR_UNSUPPORTED;
    if (matrices > 65535 || N / 128 > 65535) return MOE_ERR_BAD_ARGUMENT;
    const dim3 grid((unsigned)(K / 128), (unsigned)(N / 128), (unsigned)matrices);
    hipStream_t st = (hipStream_t)stream;
    if (src_dtype == MOE_DTYPE_F32)
        quant_block128_kernel<float><<<grid, 256, 0, st>>>((const float*)w, (uint8_t*)q, scales, N, K);
    else
        quant_block128_kernel<uint16_t><<<grid, 256, 0, st>>>((const uint16_t*)w, (uint8_t*)q, scales, N, K);
    return hipGetLastError() == hipSuccess ? MOE_OK : MOE_ERR_HIP;
}

extern "C" int moe_quant_rows128(const void* x, int64_t rows, int64_t K, void* q, float* scales, void* stream) {
    if (!x || !q || !scales || rows < 0 || K < 128 || (K % 128)) return MOE_ERR_BAD_ARGUMENT;
    if (rows * (K / 8) > (int64_t)0x7FFFFFFF * 256) return MOE_ERR_BAD_ARGUMENT;
    return launch_quant_rows128(x, q, scales, rows, K, nullptr, (hipStream_t)stream) == hipSuccess ? MOE_OK : MOE_ERR_HIP;
}

extern "C" int moe_dequant_block128(const void* q, const float* scales, int64_t matrices, int64_t N, int64_t K, void* out,
                                    void* stream) {
    if (!q || !out || !scales || matrices < 1 || N < 128 || K < 128 || (N % 128) || (K % 128)) return MOE_ERR_BAD_ARGUMENT;
    if (matrices * N * (K / 16) > (int64_t)0x7FFFFFFF * 256) return MOE_ERR_BAD_ARGUMENT;
    return launch_widen_block128(q, scales, out, matrices, N, K, (hipStream_t)stream) == hipSuccess ? MOE_OK : MOE_ERR_HIP;
}
