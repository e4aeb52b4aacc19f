// Building blocks of the backward pass of the expert FFN (the training knob is_training,
// aristos_config.schema.json:20-23, is parsed by the reference and never read; these are this library's).
//
// Everything works on packed expert-major rows as the forward pass lays them out: rows
// [expert_offset[e], expert_offset[e] + expert_count[e]) belong to expert e.
//   * data gradients are grouped (M,K) x (N,K)^T GEMMs with the weight in its K-major view, which a batched transpose
//     produces: dX = dY . W  ==  dY x (W^T)^T.  The forward tile kernels run them unchanged.
//   * weight gradients sum over an expert's rows: dW[e] = dY_e^T . A_e.  Both operands are transposed into buffers whose
//     columns are the packed rows, each expert's window padded with zeros to a multiple of 128 columns, and every
//     expert is then one tile GEMM over its window.
#include <algorithm>

#include <type_traits>

#include "moe_internal.hpp"
#include "act_deriv.hpp"

namespace moe355 {

bool grouped_gemm_takes_large_tile(int64_t A, int E, int N, int K);
hipError_t launch_grouped_gemm_16(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                  const int32_t* num_mtiles, const int32_t* count, int max_mtiles, int tile, int64_t A,
                                  int N, int K, int act, bool f16, hipStream_t st);
hipError_t launch_wgrad_16(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K,
                           int64_t ld, bool f16, hipStream_t st);

hipError_t launch_grouped_gemm_deriv_16(const void* a_rows, const void* w, const void* u, const void* g, void* du, void* dg,
                                        const MTile* mtiles, const int32_t* num_mtiles, const int32_t* count, int max_mtiles,
                                        int tile, int64_t A, int N, int K, int hidden_act, bool f16, hipStream_t st);
hipError_t launch_grouped_gemm_f32(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                   const int32_t* num_mtiles, int max_mtiles, int N, int K, int act, hipStream_t st);
hipError_t launch_wgrad_f32(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K, int64_t ld,
                            hipStream_t st);
bool grouped_gemm_f32_takes_tile(int64_t A, int N, int K);
hipError_t launch_grouped_gemm_f32_tile(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                        const int32_t* num_mtiles, int max_mtiles, int N, int K, int act, hipStream_t st);
bool wgrad_f32_takes_tile(int E, int N, int K);
hipError_t launch_wgrad_f32_tile(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K,
                                 int64_t ld, hipStream_t st);

namespace {

constexpr int kWindowAlign = 128;   // columns an expert's window of a transposed operand is padded to

// One workgroup: row blocks of `block_m` rows per expert (for the grouped GEMM) and the padded window offsets (for the
// weight gradient).  Either table may be null.
__global__ __launch_bounds__(kMaxExperts) void backward_tables_kernel(const int32_t* __restrict__ count,
                                                                      const int32_t* __restrict__ offset, int E,
                                                                      int block_m, MTile* mtiles, int32_t* num_mtiles,
                                                                      int32_t* poff) {
    __shared__ int s_mt0[kMaxExperts + 1];
    const int e = threadIdx.x;
    if (e == 0) {
        int mt = 0, po = 0;
        for (int i = 0; i < E; ++i) {
            const int n = max(count[i], 0);
            s_mt0[i] = mt;
            mt += (n + block_m - 1) / block_m;
            if (poff) poff[i] = po;
            po += (n + kWindowAlign - 1) / kWindowAlign * kWindowAlign;
        }
        s_mt0[E] = mt;
        if (num_mtiles) *num_mtiles = mt;
        if (poff) poff[E] = po;
    }
    __syncthreads();
    if (e < E && mtiles) {
        const int n = max(count[e], 0), off = offset[e];
        for (int i = 0, mt = s_mt0[e]; mt < s_mt0[e + 1]; ++i, ++mt) {
            MTile t;
            t.expert = e;
            t.row0 = off + i * block_m;
            t.rows = min(block_m, n - i * block_m);
            t.pad = s_mt0[e];        // first row block of this expert (the grouped GEMM orders its tiles by it)
            mtiles[mt] = t;
        }
    }
}

// dst[b][c][r] = src[b][r][c] for 16-bit elements; 64 x 64 tiles through LDS.  grid = (ceil(C/64), ceil(R/64), B).
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                          int64_t R, int64_t C) {
    __shared__ uint16_t tile[64][66];
    const uint16_t* s = src + (size_t)blockIdx.z * R * C;
    uint16_t* d = dst + (size_t)blockIdx.z * R * C;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int r = i >> 6, c = i & 63;
        tile[r][c] = (r0 + r < R && c0 + c < C) ? s[(r0 + r) * C + c0 + c] : (uint16_t)0;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int c = i >> 6, r = i & 63;
        if (r0 + r < R && c0 + c < C) d[(c0 + c) * R + r0 + r] = tile[r][c];
    }
}
__global__ __launch_bounds__(256) void transpose32_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                          int64_t R, int64_t C) {
    __shared__ uint32_t tile[64][65];
    const uint32_t* s = src + (size_t)blockIdx.z * R * C;
    uint32_t* d = dst + (size_t)blockIdx.z * R * C;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int r = i >> 6, c = i & 63;
        tile[r][c] = (r0 + r < R && c0 + c < C) ? s[(r0 + r) * C + c0 + c] : 0u;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int c = i >> 6, r = i & 63;
        if (r0 + r < R && c0 + c < C) d[(c0 + c) * R + r0 + r] = tile[r][c];
    }
}

// The same for 16-bit elements when R and C are multiples of 8: every global access is 16 bytes per lane.  A 64 x 64
// tile goes into LDS as rows of 32 dwords + 1 (the odd pitch spreads a column over the banks) and comes out as
// columns, eight 2-byte reads per lane packed into one 16-byte store.
__device__ __forceinline__ void tile64_store_row(uint32_t* tile, int r, int ch, uint4 v) {
    uint32_t* p = tile + r * 33 + ch * 4;
    p[0] = v.x; p[1] = v.y; p[2] = v.z; p[3] = v.w;
}
__device__ __forceinline__ uint4 tile64_load_column(const uint32_t* tile, int col, int row8) {
    const uint16_t* t = reinterpret_cast<const uint16_t*>(tile);
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t lo = t[(row8 * 8 + 2 * j) * 66 + col], hi = t[(row8 * 8 + 2 * j + 1) * 66 + col];
        w[j] = lo | (hi << 16);
    }
    return uint4{w[0], w[1], w[2], w[3]};
}

__global__ __launch_bounds__(256) void transpose16_vec_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                              int64_t R, int64_t C) {
    __shared__ uint32_t tile[64 * 33];
    const uint16_t* s = src + (size_t)blockIdx.z * R * C;
    uint16_t* d = dst + (size_t)blockIdx.z * R * C;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int sub = threadIdx.x >> 3, ch = threadIdx.x & 7;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int r = sub + 32 * pass;
        uint4 v = {0u, 0u, 0u, 0u};
        if (r0 + r < R && c0 + ch * 8 < C) v = *reinterpret_cast<const uint4*>(s + (r0 + r) * C + c0 + ch * 8);
        tile64_store_row(tile, r, ch, v);
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int c = sub + 32 * pass;
        if (c0 + c < C && r0 + ch * 8 < R)
            *reinterpret_cast<uint4*>(d + (c0 + c) * R + r0 + ch * 8) = tile64_load_column(tile, c, ch);
    }
}

// Packed rows [*, C] -> dst [C, ld]: column poff[e] + s holds row offset[e] + s of expert e (s < count[e]); the rest
// of each window is zero.  A 64-column tile of dst never straddles two windows (they are multiples of 128 wide).
// C is a multiple of 8.  grid = (ld / 64, ceil(C / 64)).
__global__ __launch_bounds__(256) void transpose_rows_padded_kernel(const uint16_t* __restrict__ rows, int C,
                                                                    const int32_t* __restrict__ count,
                                                                    const int32_t* __restrict__ offset,
                                                                    const int32_t* __restrict__ poff, int E, int64_t ld,
                                                                    uint16_t* __restrict__ dst) {
    __shared__ uint32_t tile[64 * 33];
    const int p0 = blockIdx.x * 64;
    if (p0 >= poff[E]) return;                 // behind the last window: never read
    int lo = 0, hi = E - 1;
    while (lo < hi) {                          // last expert whose window starts at or before p0 (empty windows skipped)
        const int mid = (lo + hi + 1) >> 1;
        if (poff[mid] <= p0) lo = mid; else hi = mid - 1;
    }
    const int e = lo, s0 = p0 - poff[e], n = count[e], off = offset[e];
    const int c0 = blockIdx.y * 64;
    const int sub = threadIdx.x >> 3, ch = threadIdx.x & 7;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int r = sub + 32 * pass;
        uint4 v = {0u, 0u, 0u, 0u};
        if (s0 + r < n && c0 + ch * 8 < C)
            v = *reinterpret_cast<const uint4*>(rows + (size_t)(off + s0 + r) * C + c0 + ch * 8);
        tile64_store_row(tile, r, ch, v);
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int c = sub + 32 * pass;
        if (c0 + c < C)
            *reinterpret_cast<uint4*>(dst + (size_t)(c0 + c) * ld + p0 + ch * 8) = tile64_load_column(tile, c, ch);
    }
}

// The same for 4-byte elements (fp32 layers): any C.  grid = (ld / 64, ceil(C / 64)).
__global__ __launch_bounds__(256) void transpose_rows_padded32_kernel(const uint32_t* __restrict__ rows, int C,
                                                                      const int32_t* __restrict__ count,
                                                                      const int32_t* __restrict__ offset,
                                                                      const int32_t* __restrict__ poff, int E, int64_t ld,
                                                                      uint32_t* __restrict__ dst) {
    __shared__ uint32_t tile[64][65];
    const int p0 = blockIdx.x * 64;
    if (p0 >= poff[E]) return;                 // behind the last window: never read
    int lo = 0, hi = E - 1;
    while (lo < hi) {                          // last expert whose window starts at or before p0 (empty windows skipped)
        const int mid = (lo + hi + 1) >> 1;
        if (poff[mid] <= p0) lo = mid; else hi = mid - 1;
    }
    const int e = lo, s0 = p0 - poff[e], n = count[e], off = offset[e];
    const int c0 = blockIdx.y * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int r = i >> 6, c = i & 63;
        tile[r][c] = (s0 + r < n && c0 + c < C) ? rows[(size_t)(off + s0 + r) * C + c0 + c] : 0u;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int c = i >> 6, r = i & 63;
        if (c0 + c < C) dst[(size_t)(c0 + c) * ld + p0 + r] = tile[r][c];
    }
}

// ---- elementwise and reduction steps of a backward pass ----
struct f32_s {};
template <class T> struct RawOf { typedef uint16_t type; };
template <> struct RawOf<f32_s> { typedef float type; };
template <class T16> __device__ __forceinline__ float ld16(const typename RawOf<T16>::type* p, size_t i);
template <> __device__ __forceinline__ float ld16<bf16_s>(const uint16_t* p, size_t i) { return __uint_as_float((uint32_t)p[i] << 16); }
template <> __device__ __forceinline__ float ld16<f16_s>(const uint16_t* p, size_t i) { return (float)__builtin_bit_cast(_Float16, p[i]); }
template <> __device__ __forceinline__ float ld16<f32_s>(const float* p, size_t i) { return p[i]; }
template <class T16> __device__ __forceinline__ typename RawOf<T16>::type st16(float v);
template <> __device__ __forceinline__ uint16_t st16<bf16_s>(float v) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t x = {v, 0.0f};
    return (uint16_t)(__builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2_t)) & 0xFFFFu);
}
template <> __device__ __forceinline__ uint16_t st16<f16_s>(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
template <> __device__ __forceinline__ float st16<f32_s>(float v) { return v; }

// du = dh * act'(u); SwiGLU (h = silu(g) u): du = dh silu(g), dg = dh u s (1 + g (1 - s)), s = sigmoid(g).
// fp32 layers use the library functions; 16-bit layers the forms of act_deriv.hpp, which the fused data gradient's
// epilogue inlines as well (same bits on both paths).
template <class T16>
__device__ __forceinline__ void act_backward_one(float d, float uv, float gv, int act, float& a, float& b) {
    constexpr bool kF32 = std::is_same<T16, f32_s>::value;
    b = 0.0f;
    if (act == MOE_ACT_SWIGLU) {
        if constexpr (kF32) {
            const float sg = 1.0f / (1.0f + expf(-gv));
            a = d * (gv * sg);
            b = d * uv * (sg * (1.0f + gv * (1.0f - sg)));
        } else {
            dswiglu16(d, uv, gv, a, b);
        }
    } else if (act == MOE_ACT_GELU) {
        if constexpr (kF32) {
            const float cdf = 0.5f * (1.0f + erff(uv * 0.70710678118654752440f));
            const float pdf = 0.39894228040143267794f * expf(-0.5f * uv * uv);
            a = d * (cdf + uv * pdf);
        } else {
            a = dgelu16(d, uv);
        }
    } else {
        a = drelu16(d, uv);
    }
}

// 16 bytes of every operand per thread and step (8 or 4 elements): the pass is a stream over five arrays at most and
// has nothing else to wait for.  n is a multiple of the intermediate size, which is a multiple of 64; all pointers
// 16-byte aligned (the launcher checks both).
template <class T16, class RAW = typename RawOf<T16>::type>
__global__ __launch_bounds__(256) void act_backward_kernel(const RAW* __restrict__ dh, const RAW* __restrict__ u,
                                                           const RAW* __restrict__ g, size_t n, int act,
                                                           RAW* __restrict__ du, RAW* __restrict__ dg) {
    constexpr int VEC = 16 / (int)sizeof(RAW);
    union Pack { uint4 q; RAW e[VEC]; };
    const size_t nv = n / VEC, id = (size_t)blockIdx.x * 256 + threadIdx.x;
    const bool gated = act == MOE_ACT_SWIGLU;
    for (size_t i = id; i < nv; i += (size_t)gridDim.x * 256) {
        Pack d, uu, gg, oa, ob;
        d.q = reinterpret_cast<const uint4*>(dh)[i];
        uu.q = reinterpret_cast<const uint4*>(u)[i];
        gg.q = gated ? reinterpret_cast<const uint4*>(g)[i] : uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            float a, b;
            act_backward_one<T16>(ld16<T16>(d.e, k), ld16<T16>(uu.e, k), ld16<T16>(gg.e, k), act, a, b);
            oa.e[k] = st16<T16>(a);
            ob.e[k] = st16<T16>(b);
        }
        reinterpret_cast<uint4*>(du)[i] = oa.q;
        if (gated) reinterpret_cast<uint4*>(dg)[i] = ob.q;
    }
}

// The same one element at a time, for operands that are not 16-byte aligned.
template <class T16, class RAW = typename RawOf<T16>::type>
__global__ __launch_bounds__(256) void act_backward_unaligned_kernel(const RAW* __restrict__ dh, const RAW* __restrict__ u,
                                                                     const RAW* __restrict__ g, size_t n, int act,
                                                                     RAW* __restrict__ du, RAW* __restrict__ dg) {
    const bool gated = act == MOE_ACT_SWIGLU;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float a, b;
        act_backward_one<T16>(ld16<T16>(dh, i), ld16<T16>(u, i), gated ? ld16<T16>(g, i) : 0.0f, act, a, b);
        du[i] = st16<T16>(a);
        if (gated) dg[i] = st16<T16>(b);
    }
}

// db[e, n] = sum over expert e's rows, ascending, of dy[r, n]: one thread per column, so the order is fixed.
// grid = (ceil(N / 256), E).
template <class T16, class RAW = typename RawOf<T16>::type>
__global__ __launch_bounds__(256) void bias_grad_kernel(const RAW* __restrict__ dy, const int32_t* __restrict__ count,
                                                        const int32_t* __restrict__ offset, int N, RAW* __restrict__ db) {
    const int n = blockIdx.x * 256 + threadIdx.x, e = blockIdx.y;
    if (n >= N) return;
    const int r0 = offset[e], r1 = r0 + max(count[e], 0);
    float acc = 0.0f;
    for (int r = r0; r < r1; ++r) acc = acc + ld16<T16>(dy, (size_t)r * N + n);
    db[(size_t)e * N + n] = st16<T16>(acc);
}

// One workgroup per token: dy[row(t,r), :] = w[t,r] * dout[t, :]; dw[t,r] = <dout[t, :], y[row(t,r), :]>.
template <class T16, class RAW = typename RawOf<T16>::type>
__global__ __launch_bounds__(256) void combine_backward_kernel(const RAW* __restrict__ dout, const RAW* __restrict__ y,
                                                               const int32_t* __restrict__ pair_row,
                                                               const float* __restrict__ topk_w, int k, int H,
                                                               RAW* __restrict__ dy, float* __restrict__ dw) {
    __shared__ float part[4];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int r = 0; r < k; ++r) {
        const int row = pair_row[(size_t)t * k + r];
        float acc = 0.0f;
        if (row >= 0) {
            const float w = topk_w[(size_t)t * k + r];
            for (int j = threadIdx.x; j < H; j += 256) {
                const float d = ld16<T16>(dout, (size_t)t * H + j);
                dy[(size_t)row * H + j] = st16<T16>(w * d);
                acc = fmaf(d, ld16<T16>(y, (size_t)row * H + j), acc);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        __syncthreads();                       // part may still be read for the previous rank
        if (lane == 0) part[wave] = acc;
        __syncthreads();
        if (threadIdx.x == 0) dw[(size_t)t * k + r] = row >= 0 ? (part[0] + part[1]) + (part[2] + part[3]) : 0.0f;
    }
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

int64_t wgrad_ld(int64_t A, int E) { return (A + (int64_t)kWindowAlign * E + 127) / 128 * 128; }

size_t backward_scratch_bytes(int64_t A, int E, int H, int I, int elem_bytes) {
    const size_t tables = align256(sizeof(int32_t)) + align256((size_t)(A / 64 + E + 1) * sizeof(MTile)) + align256((size_t)(E + 1) * 4);
    const size_t operands = align256((size_t)H * wgrad_ld(A, E) * elem_bytes) + align256((size_t)I * wgrad_ld(A, E) * elem_bytes);
    return tables + operands;
}

hipError_t launch_transpose(const void* src, void* dst, int64_t batch, int64_t rows, int64_t cols, int elem_bytes,
                            hipStream_t st) {
    if (batch < 1 || rows < 1 || cols < 1) return hipSuccess;
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64), (unsigned)batch);
    if (elem_bytes == 2 && rows % 8 == 0 && cols % 8 == 0 && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0))
        transpose16_vec_kernel<<<grid, 256, 0, st>>>((const uint16_t*)src, (uint16_t*)dst, rows, cols);
    else if (elem_bytes == 2) transpose16_kernel<<<grid, 256, 0, st>>>((const uint16_t*)src, (uint16_t*)dst, rows, cols);
    else transpose32_kernel<<<grid, 256, 0, st>>>((const uint32_t*)src, (uint32_t*)dst, rows, cols);
    return hipGetLastError();
}

namespace {
// The table region at the head of the scratch buffer: the number of row blocks, the row blocks (64 rows is the
// smallest block any kernel here uses), the window offsets.
struct ScratchTables {
    int32_t* num_mtiles;
    MTile* mtiles;
    int32_t* poff;
    char* operands;
};
ScratchTables scratch_tables(void* scratch, int64_t A, int E) {
    char* s = static_cast<char*>(scratch);
    ScratchTables t;
    t.num_mtiles = reinterpret_cast<int32_t*>(s);
    t.mtiles = reinterpret_cast<MTile*>(s + align256(sizeof(int32_t)));
    const size_t tables = align256(sizeof(int32_t)) + align256((size_t)(A / 64 + E + 1) * sizeof(MTile));
    t.poff = reinterpret_cast<int32_t*>(s + tables);
    t.operands = s + tables + align256((size_t)(E + 1) * 4);
    return t;
}
}  // namespace

// out_rows[r,:] = act(a_rows[r,:] . w[e(r)]^T + bias[e(r)]); scratch holds the row-block table.
// dtype: the storage type of every operand (MOE_DTYPE_F32, _BF16 or _FP16).
hipError_t launch_expert_gemm(const void* a_rows, const void* w, const void* bias, const int32_t* count,
                              const int32_t* offset, int64_t A, int E, int N, int K, int act, int dtype,
                              const moe_options& opt, void* out_rows, void* scratch, hipStream_t st) {
    const ScratchTables t = scratch_tables(scratch, A, E);
    if (dtype == MOE_DTYPE_F32) {
        bool mfma = grouped_gemm_f32_takes_tile(A, N, K);
        if (opt.f32_tile == 0) mfma = false;   // option: keep the vector-ALU kernel
        const int block_m = mfma ? 128 : 64;
        const int max_mtiles = (int)(A / block_m + E);
        backward_tables_kernel<<<1, kMaxExperts, 0, st>>>(count, offset, E, block_m, t.mtiles, t.num_mtiles, nullptr);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        return (mfma ? launch_grouped_gemm_f32_tile : launch_grouped_gemm_f32)(a_rows, w, bias, out_rows, t.mtiles,
                                                                               t.num_mtiles, max_mtiles, N, K, act, st);
    }
    int tile = grouped_gemm_takes_large_tile(A, E, N, K) ? 1 : 0;     // 1: 256 x 256, 0: 128 x 128
    if (opt.grouped_tile != MOE_OPT_AUTO) {                            // option; 2: 128 x 256 (hand-ordered)
        const int v = opt.grouped_tile;
        const int64_t lim = (int64_t)1 << 32;
        if ((v == 1 || v == 2) && N % 256 == 0 && K % 128 == 0 && A * K * 2 < lim && (int64_t)N * K * 2 < lim) tile = v;
        if (v == 0) tile = 0;
    }
    const int block_m = tile == 1 ? 256 : 128;
    const int max_mtiles = (int)(A / block_m + E);
    backward_tables_kernel<<<1, kMaxExperts, 0, st>>>(count, offset, E, block_m, t.mtiles, t.num_mtiles, nullptr);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_grouped_gemm_16(a_rows, w, bias, out_rows, t.mtiles, t.num_mtiles, count, max_mtiles, tile, A, N, K, act,
                                  dtype == MOE_DTYPE_FP16, st);
}

// The tile the fused data gradient (product + activation derivative) would run on: 1 or 2 (the hand-ordered tiles), or 0
// when the shape or the options leave only the 128 x 128 tile, which has no such epilogue.
int expert_gemm_dact_tile(int64_t A, int E, int N, int K, int dtype, const moe_options& opt) {
    if (dtype != MOE_DTYPE_BF16 && dtype != MOE_DTYPE_FP16) return 0;
    int tile = grouped_gemm_takes_large_tile(A, E, N, K) ? 1 : 0;
    const int64_t lim = (int64_t)1 << 32;
    const bool hand_ok = N % 256 == 0 && K % 128 == 0 && A * K * 2 < lim && (int64_t)N * K * 2 < lim;
    if (opt.grouped_tile != MOE_OPT_AUTO) {
        const int v = opt.grouped_tile;
        if ((v == 1 || v == 2) && hand_ok) tile = v;
        if (v == 0) tile = 0;
    } else if (tile == 0 && hand_ok) {
        tile = 2;      // few rows per expert: the 128-row hand-ordered tile rather than no fusion at all
    }
    return tile;
}

// du_rows = (dy_rows . w[e(r)]^T) * act'(u_rows) (and dg_rows for SwiGLU): launch_expert_gemm with act NONE and
// launch_act_backward in one kernel; the product is rounded to the storage type before the derivative, as the two-call
// chain does when it stores dh, so both give the same bits.  16-bit layers on the hand-ordered tiles only.
hipError_t launch_expert_gemm_dact(const void* dy_rows, const void* w, const void* u_rows, const void* g_rows,
                                   const int32_t* count, const int32_t* offset, int64_t A, int E, int N, int K, int hidden_act,
                                   int dtype, const moe_options& opt, void* du_rows, void* dg_rows, void* scratch,
                                   hipStream_t st) {
    const int tile = expert_gemm_dact_tile(A, E, N, K, dtype, opt);
    if (tile == 0) return hipErrorNotSupported;
    const ScratchTables t = scratch_tables(scratch, A, E);
    const int block_m = tile == 1 ? 256 : 128;
    const int max_mtiles = (int)(A / block_m + E);
    backward_tables_kernel<<<1, kMaxExperts, 0, st>>>(count, offset, E, block_m, t.mtiles, t.num_mtiles, nullptr);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_grouped_gemm_deriv_16(dy_rows, w, u_rows, g_rows, du_rows, dg_rows, t.mtiles, t.num_mtiles, count, max_mtiles,
                                        tile, A, N, K, hidden_act, dtype == MOE_DTYPE_FP16, st);
}

// dw[e] [N,K] = dy_e^T . a_e; scratch holds the window offsets and the two transposed operands.
hipError_t launch_expert_wgrad(const void* dy_rows, const void* a_rows, const int32_t* count, const int32_t* offset,
                               int64_t A, int E, int N, int K, int dtype, const moe_options& opt, void* dw, void* scratch,
                               hipStream_t st) {
    const ScratchTables t = scratch_tables(scratch, A, E);
    const int64_t ld = wgrad_ld(A, E);
    const size_t eb = dtype == MOE_DTYPE_F32 ? 4 : 2;
    void* dyT = t.operands;
    void* aT = t.operands + align256((size_t)N * ld * eb);
    backward_tables_kernel<<<1, kMaxExperts, 0, st>>>(count, offset, E, 128, nullptr, nullptr, t.poff);
    const dim3 g1((unsigned)(ld / 64), (unsigned)((N + 63) / 64)), g2((unsigned)(ld / 64), (unsigned)((K + 63) / 64));
    if (dtype == MOE_DTYPE_F32) {
        transpose_rows_padded32_kernel<<<g1, 256, 0, st>>>((const uint32_t*)dy_rows, N, count, offset, t.poff, E, ld, (uint32_t*)dyT);
        transpose_rows_padded32_kernel<<<g2, 256, 0, st>>>((const uint32_t*)a_rows, K, count, offset, t.poff, E, ld, (uint32_t*)aT);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        bool mfma = wgrad_f32_takes_tile(E, N, K);
        if (opt.f32_tile == 0) mfma = false;   // option: keep the vector-ALU kernel
        return (mfma ? launch_wgrad_f32_tile : launch_wgrad_f32)(dyT, aT, dw, t.poff, E, N, K, ld, st);
    }
    transpose_rows_padded_kernel<<<g1, 256, 0, st>>>((const uint16_t*)dy_rows, N, count, offset, t.poff, E, ld, (uint16_t*)dyT);
    transpose_rows_padded_kernel<<<g2, 256, 0, st>>>((const uint16_t*)a_rows, K, count, offset, t.poff, E, ld, (uint16_t*)aT);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_wgrad_16(dyT, aT, dw, t.poff, E, N, K, ld, dtype == MOE_DTYPE_FP16, st);
}

template <class T16, class RAW>
static void launch_act_backward_t(const void* dh, const void* u, const void* g, int64_t n, int act, void* du, void* dg,
                                  hipStream_t st) {
    constexpr int VEC = 16 / (int)sizeof(RAW);
    const uintptr_t bits = (uintptr_t)dh | (uintptr_t)u | (uintptr_t)g | (uintptr_t)du | (uintptr_t)dg;
    if (bits % 16 == 0 && n % VEC == 0) {
        const int grid = (int)std::min<int64_t>((n / VEC + 255) / 256, 65536);
        act_backward_kernel<T16><<<grid, 256, 0, st>>>((const RAW*)dh, (const RAW*)u, (const RAW*)g, (size_t)n, act, (RAW*)du, (RAW*)dg);
    } else {
        const int grid = (int)std::min<int64_t>((n + 255) / 256, 65536);
        act_backward_unaligned_kernel<T16><<<grid, 256, 0, st>>>((const RAW*)dh, (const RAW*)u, (const RAW*)g, (size_t)n, act, (RAW*)du, (RAW*)dg);
    }
}

hipError_t launch_act_backward(const void* dh, const void* u, const void* g, int64_t n, int act, int dtype, void* du,
                               void* dg, hipStream_t st) {
    if (n <= 0) return hipSuccess;
    if (dtype == MOE_DTYPE_F32) launch_act_backward_t<f32_s, float>(dh, u, g, n, act, du, dg, st);
    else if (dtype == MOE_DTYPE_FP16) launch_act_backward_t<f16_s, uint16_t>(dh, u, g, n, act, du, dg, st);
    else launch_act_backward_t<bf16_s, uint16_t>(dh, u, g, n, act, du, dg, st);
    return hipGetLastError();
}

hipError_t launch_bias_grad(const void* dy, const int32_t* count, const int32_t* offset, int E, int N, int dtype, void* db,
                            hipStream_t st) {
    const dim3 grid((unsigned)((N + 255) / 256), (unsigned)E);
    if (dtype == MOE_DTYPE_F32) bias_grad_kernel<f32_s><<<grid, 256, 0, st>>>((const float*)dy, count, offset, N, (float*)db);
    else if (dtype == MOE_DTYPE_FP16) bias_grad_kernel<f16_s><<<grid, 256, 0, st>>>((const uint16_t*)dy, count, offset, N, (uint16_t*)db);
    else bias_grad_kernel<bf16_s><<<grid, 256, 0, st>>>((const uint16_t*)dy, count, offset, N, (uint16_t*)db);
    return hipGetLastError();
}

hipError_t launch_combine_backward(const void* dout, const void* y, const int32_t* pair_row, const float* topk_w, int S,
                                   int k, int H, int dtype, void* dy, float* dw, hipStream_t st) {
    if (S <= 0) return hipSuccess;
    if (dtype == MOE_DTYPE_F32) combine_backward_kernel<f32_s><<<S, 256, 0, st>>>((const float*)dout, (const float*)y, pair_row, topk_w, k, H, (float*)dy, dw);
    else if (dtype == MOE_DTYPE_FP16) combine_backward_kernel<f16_s><<<S, 256, 0, st>>>((const uint16_t*)dout, (const uint16_t*)y, pair_row, topk_w, k, H, (uint16_t*)dy, dw);
    else combine_backward_kernel<bf16_s><<<S, 256, 0, st>>>((const uint16_t*)dout, (const uint16_t*)y, pair_row, topk_w, k, H, (uint16_t*)dy, dw);
    return hipGetLastError();
}

}  // namespace moe355
