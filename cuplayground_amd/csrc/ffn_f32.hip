// Expert FFN in fp32 (torch_dtype 0): the reference's tile GEMM contract, C = act(A.B^T + bias)
// (mma.cuh:46-179; its only instantiated case is fp32 + ReLU, mma.cuh:378-384), on the vector ALUs.
// This is the kernel of small and ragged fp32 layers (large ones take ffn_f32_tile.hip): a plain LDS-tiled FMA kernel, 64x64 output tile,
// 16-wide K slabs, 256 threads with a 4x4 register block each.  Task decoding, dispatch-by-gather and the
// phase dependency protocol are shared with the bf16 path.
#include "ffn_common.hpp"

namespace moe355 {
namespace {

constexpr int FBM = 64, FBN = 64, FBK = 16, FPAD = 4;

struct TaskPtrsF {
    const float* a_base;
    const int32_t* gather;
    int64_t a_row0;
    int a_ld;
    int b_ld;          // row pitch of b0 / b1 (K, except for windows of a wider matrix)
    const float* b0;
    const float* b1;
    const float* bias0;
    const float* bias1;
    float* c_base;
    int N, K, rows, n0, act;
    bool swiglu;
    bool publish;   // rows are read by other workgroups of the same launch
};

__device__ __forceinline__ void gemm_tile_f32(const TaskPtrsF& p, float (*As)[FBM + FPAD], float (*Bs)[FBN + FPAD]) {
    const int tid = threadIdx.x;
    const int ty = tid >> 4, tx = tid & 15;
    const int lrow = tid >> 2, lk = (tid & 3) * 4;

    int ar = lrow < p.rows ? lrow : 0;
    const int64_t src_row = p.gather ? (int64_t)p.gather[ar] : p.a_row0 + ar;
    const float* a_src = p.a_base + src_row * p.a_ld + lk;

    int col;
    const float* bbase = p.b0;
    if (p.swiglu) {
        col = p.n0 + (lrow & 31);
        bbase = (lrow >> 5) ? p.b0 : p.b1;      // tile rows 0..31 gate, 32..63 up
    } else {
        col = p.n0 + lrow;
    }
    if (col >= p.N) col = p.N - 1;
    const float* b_src = bbase + (int64_t)col * p.b_ld + lk;

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[i][q] = 0.0f;

    for (int k0 = 0; k0 < p.K; k0 += FBK) {
        const float4 av = *reinterpret_cast<const float4*>(a_src + k0);
        const float4 bv = *reinterpret_cast<const float4*>(b_src + k0);
        __syncthreads();
        As[lk + 0][lrow] = av.x; As[lk + 1][lrow] = av.y; As[lk + 2][lrow] = av.z; As[lk + 3][lrow] = av.w;
        Bs[lk + 0][lrow] = bv.x; Bs[lk + 1][lrow] = bv.y; Bs[lk + 2][lrow] = bv.z; Bs[lk + 3][lrow] = bv.w;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < FBK; ++kk) {
            const float4 a4 = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);
            const float2 b01 = *reinterpret_cast<const float2*>(&Bs[kk][tx * 2]);
            const float2 b23 = *reinterpret_cast<const float2*>(&Bs[kk][32 + tx * 2]);
            const float a[4] = {a4.x, a4.y, a4.z, a4.w};
            const float b[4] = {b01.x, b01.y, b23.x, b23.y};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[i][q] = __builtin_fmaf(a[i], b[q], acc[i][q]);
        }
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = ty * 4 + i;
        if (m >= p.rows) continue;
        float* crow = p.c_base + (int64_t)m * p.N;
        if (p.swiglu) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int c = p.n0 + tx * 2 + q;
                if (c >= p.N) continue;
                float g = acc[i][q], u = acc[i][q + 2];
                if (p.bias1) g = g + p.bias1[c];
                if (p.bias0) u = u + p.bias0[c];
                const float v = silu(g) * u;
                if (p.publish) publish4(crow + c, __float_as_uint(v)); else crow[c] = v;
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = p.n0 + (q >> 1) * 32 + tx * 2 + (q & 1);
                if (c >= p.N) continue;
                float u = acc[i][q];
                if (p.bias0) u = u + p.bias0[c];
                const float v = act_apply(u, p.act);
                if (p.publish) publish4(crow + c, __float_as_uint(v)); else crow[c] = v;
            }
        }
    }
}

__device__ __forceinline__ TaskPtrsF resolve_f32(const FfnArgs& a, const Task& t, bool publish) {
    TaskPtrsF p;
    const int64_t HI = (int64_t)a.H * a.I;
    const bool sw = a.act == MOE_ACT_SWIGLU;
    if (t.phase == 0) {
        p.a_base = (const float*)a.x;
        p.gather = a.token_indices + t.row0;
        p.a_row0 = 0;
        p.a_ld = a.H;
        p.b_ld = a.H;
        p.b0 = (const float*)a.w_up + t.expert * HI;
        p.b1 = sw ? (const float*)a.w_gate + t.expert * HI : nullptr;
        p.bias0 = a.b_up ? (const float*)a.b_up + (int64_t)t.expert * a.I : nullptr;
        p.bias1 = (sw && a.b_gate) ? (const float*)a.b_gate + (int64_t)t.expert * a.I : nullptr;
        p.c_base = (float*)a.h + (int64_t)t.row0 * a.I;
        p.N = a.I;
        p.K = a.H;
        p.n0 = t.ntile * (sw ? FBN / 2 : FBN);
        p.act = a.act;
        p.swiglu = sw;
        p.publish = publish;
    } else {
        p.a_base = (const float*)a.h;
        p.gather = nullptr;
        p.a_row0 = t.row0;
        p.a_ld = a.I;
        p.b_ld = a.I;
        p.b0 = (const float*)a.w_down + t.expert * HI;
        p.b1 = nullptr;
        p.bias0 = a.b_down ? (const float*)a.b_down + (int64_t)t.expert * a.H : nullptr;
        p.bias1 = nullptr;
        p.c_base = (float*)a.y + (int64_t)t.row0 * a.H;
        p.N = a.H;
        p.K = a.I;
        p.n0 = t.ntile * FBN;
        p.act = MOE_ACT_NONE;
        p.swiglu = false;
        p.publish = publish;
    }
    p.rows = t.rows;
    return p;
}

__global__ __launch_bounds__(256) void ffn_tiled_f32_kernel(FfnArgs a, int phase) {
    __shared__ __align__(16) float As[FBK][FBM + FPAD];
    __shared__ __align__(16) float Bs[FBK][FBN + FPAD];
    Task t;
    __shared__ int s_list[1 + FBM];
    if (phase == 0) zero_unrouted_rows(a, 4);
    if (!tiled_task(a, phase, blockIdx.x, t)) return;
    const TaskPtrsF p = resolve_f32(a, t, phase == 1 && a.arrive);
    gemm_tile_f32(p, As, Bs);
    if (phase == 1 && a.arrive) combine_arrivals<float>(combine_args(a), t.row0, t.rows, t.ntile, p.n0, FBN, s_list);
}

__global__ __launch_bounds__(256) void ffn_persistent_f32_kernel(FfnArgs a) {
    __shared__ __align__(16) float As[FBK][FBM + FPAD];
    __shared__ __align__(16) float Bs[FBK][FBN + FPAD];
    __shared__ int s_task, s_ok;
    __shared__ int s_cmb[kCombineLds];
    __shared__ int s_list[1 + FBM];
    queue_kernel_entry();
    queue_clock_stamp(a.wg_clock, 0);
    zero_unrouted_rows(a, 4);
    const int ids = a.q->ids_queue;
    const int nseg = a.q->nseg;
    const int nnt0 = a.seg_phase0[0].nnt;
    QueueCursor cur = queue_cursor(a.groups);
    Task t;
    while (next_task(a, cur, &s_task, ids, nseg, nnt0, t)) {
        int ok = 1;
        if (t.phase == 1) ok = wait_phase0_done(a.done0, t.mtile, nnt0, a.spin_limit, a.q, a.host_stall, &s_ok);
        const TaskPtrsF p = resolve_f32(a, t, t.phase == 0 || publish_y(a));
        const long long started = trace_clock(a.task_trace);
        if (ok) gemm_tile_f32(p, As, Bs);
        else poison_tile(p.c_base, p.rows, p.N, p.n0, FBN, 4);
        if (a.task_trace) trace_task(a.task_trace, a.task_trace_cap, t.phase, t.expert, t.mtile, t.ntile, t.rows, started);
        if (t.phase == 0) signal_phase0_done(a.done0, t.mtile);
        else after_down_tile<float>(a, t.row0, t.rows, t.mtile, t.ntile, p.n0, FBN, s_list);
    }
    if (a.combined) combine_while_idle_narrow<float>(sweep_args(a), &s_task, s_cmb);
    queue_clock_stamp(a.wg_clock, 1);
}

__global__ __launch_bounds__(256) void gemm_dense_f32_kernel(const float* A, const float* B, const float* bias,
                                                             float* C, int M, int N, int K, int act) {
    __shared__ __align__(16) float As[FBK][FBM + FPAD];
    __shared__ __align__(16) float Bs[FBK][FBN + FPAD];
    TaskPtrsF p;
    const int row0 = blockIdx.y * FBM;
    p.a_base = A; p.gather = nullptr; p.a_row0 = row0; p.a_ld = K; p.b_ld = K;
    p.b0 = B; p.b1 = nullptr; p.bias0 = bias; p.bias1 = nullptr;
    p.c_base = C + (int64_t)row0 * N;
    p.N = N; p.K = K; p.rows = min(FBM, M - row0); p.n0 = blockIdx.x * FBN; p.act = act; p.swiglu = false; p.publish = false;
    gemm_tile_f32(p, As, Bs);
}

// Grouped product over packed expert-major rows (backward.hip): out[r,:] = act(a_rows[r,:] . w[e(r)]^T + bias[e(r)]),
// one workgroup per (row block of 64 from `mtiles`, 64 output columns).
__global__ __launch_bounds__(256) void grouped_gemm_f32_kernel(const float* a_rows, const float* w, const float* bias,
                                                               float* out, const MTile* mtiles, const int32_t* num_mtiles,
                                                               int nnt, int N, int K, int act) {
    __shared__ __align__(16) float As[FBK][FBM + FPAD];
    __shared__ __align__(16) float Bs[FBK][FBN + FPAD];
    const int mt = blockIdx.x / nnt, nt = blockIdx.x % nnt;
    if (mt >= *num_mtiles) return;
    const MTile m = mtiles[mt];
    TaskPtrsF p;
    p.a_base = a_rows; p.gather = nullptr; p.a_row0 = m.row0; p.a_ld = K; p.b_ld = K;
    p.b0 = w + (int64_t)m.expert * N * K; p.b1 = nullptr;
    p.bias0 = bias ? bias + (int64_t)m.expert * N : nullptr; p.bias1 = nullptr;
    p.c_base = out + (int64_t)m.row0 * N;
    p.N = N; p.K = K; p.rows = m.rows; p.n0 = nt * FBN; p.act = act; p.swiglu = false; p.publish = false;
    gemm_tile_f32(p, As, Bs);
}

// Weight gradient of one expert: dw[e] [N,K] = dyT[:, window e] . aT[:, window e]^T, the windows being the expert's
// packed rows as columns of the transposed operands (zero padded to a multiple of 128, pitch ld).
// grid = (ceil(K / 64), ceil(N / 64), E).
__global__ __launch_bounds__(256) void wgrad_f32_kernel(const float* dyT, const float* aT, float* dw, const int32_t* poff,
                                                        int N, int K, int64_t ld) {
    __shared__ __align__(16) float As[FBK][FBM + FPAD];
    __shared__ __align__(16) float Bs[FBK][FBN + FPAD];
    const int e = blockIdx.z, row0 = blockIdx.y * FBM;
    TaskPtrsF p;
    p.a_base = dyT + poff[e]; p.gather = nullptr; p.a_row0 = row0; p.a_ld = (int)ld; p.b_ld = (int)ld;
    p.b0 = aT + poff[e]; p.b1 = nullptr; p.bias0 = nullptr; p.bias1 = nullptr;
    p.c_base = dw + (int64_t)e * N * K + (int64_t)row0 * K;
    p.N = K; p.K = poff[e + 1] - poff[e]; p.rows = min(FBM, N - row0); p.n0 = blockIdx.x * FBN; p.act = MOE_ACT_NONE;
    p.swiglu = false; p.publish = false;
    gemm_tile_f32(p, As, Bs);
}

}  // namespace

int f32_block_m() { return FBM; }
int f32_block_n() { return FBN; }

hipError_t launch_ffn_tiled_f32(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, hipStream_t st) {
    ffn_tiled_f32_kernel<<<tiled_grid(max_mtiles, nnt0, a.groups), 256, 0, st>>>(a, 0);
    ffn_tiled_f32_kernel<<<tiled_grid(max_mtiles, nnt1, a.groups), 256, 0, st>>>(a, 1);
    return hipGetLastError();
}

hipError_t launch_ffn_persistent_f32(const FfnArgs& a, int blocks, hipStream_t st) {
    ffn_persistent_f32_kernel<<<blocks, 256, 0, st>>>(a);
    return hipGetLastError();
}

hipError_t launch_gemm_dense_f32(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                 int64_t K, int act, hipStream_t st) {
    const dim3 grid((unsigned)((N + FBN - 1) / FBN), (unsigned)((M + FBM - 1) / FBM));
    gemm_dense_f32_kernel<<<grid, 256, 0, st>>>((const float*)A, (const float*)B, (const float*)bias, (float*)C,
                                                (int)M, (int)N, (int)K, act);
    return hipGetLastError();
}

hipError_t launch_grouped_gemm_f32(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                   const int32_t* num_mtiles, int max_mtiles, int N, int K, int act, hipStream_t st) {
    const int nnt = (N + FBN - 1) / FBN;
    grouped_gemm_f32_kernel<<<(unsigned)max_mtiles * nnt, 256, 0, st>>>((const float*)a_rows, (const float*)w,
                                                                        (const float*)bias, (float*)out, mtiles,
                                                                        num_mtiles, nnt, N, K, act);
    return hipGetLastError();
}

hipError_t launch_wgrad_f32(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K, int64_t ld,
                            hipStream_t st) {
    const dim3 grid((unsigned)((K + FBN - 1) / FBN), (unsigned)((N + FBM - 1) / FBM), (unsigned)E);
    wgrad_f32_kernel<<<grid, 256, 0, st>>>((const float*)dyT, (const float*)aT, (float*)dw, poff, N, K, ld);
    return hipGetLastError();
}

}  // namespace moe355
