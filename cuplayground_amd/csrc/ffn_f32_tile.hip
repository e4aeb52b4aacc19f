// Expert FFN in fp32 (torch_dtype 0, and 1: tf32 is stored and computed as fp32) on the matrix cores, for layers whose
// experts see enough rows to fill 128-row blocks -- the reference's own knob file is such a layer (aristos_config.json:
// fp32, 8192 tokens, one expert, H 1024, I 4096).  ffn_f32.hip multiplies on the vector ALUs, whose unpacked fp32 rate
// is half of what v_mfma_f32_32x32x2_f32 reaches; small or ragged layers stay there.
// The contract is the reference's tile GEMM (mma.cuh:46-179: C = act(A.B^T + bias), A (M,K), B (N,K) row-major, fp32
// accumulation) with its only instantiated element type (mma.cuh:378-384).
//
// A task is (expert, 128-token row block, 128 weight rows): 64 gate + 64 up rows for a SwiGLU up projection (pairs stay
// inside a lane), 128 rows of w_up or w_down otherwise.
//   * four wavefronts of 64 x 64 outputs = 2 x 2 blocks of v_mfma_f32_32x32x2_f32, weights as the "A" operand, so a
//     lane ends up with 4 consecutive output columns of one token row (16-byte stores);
//   * K slabs of 32: token rows and weight rows both go from global memory straight into LDS (global_load ... lds) as
//     128-byte rows with xor-swizzled 16-byte chunks; a lane reads 4 consecutive k of its row at a time
//     (ds_read_b128) and feeds them to 4 MFMAs -- the k order inside a slab is permuted the same way for both
//     operands, which only changes the order of the fp32 sum;
//   * two 32 KiB LDS stages per workgroup, two workgroups per compute unit.
#include "ffn_common.hpp"

namespace moe355 {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

constexpr int GBM = 128;          // token rows per row block
constexpr int GBN = 128;          // weight rows per tile
constexpr int GN0 = 64;           // intermediate columns per SwiGLU up-projection task (64 gate + 64 up rows)
constexpr int GN1 = 128;          // output columns of every other task
constexpr int GBK = 32;           // k per slab
constexpr int GROW = 128;         // bytes per LDS row (32 floats)
constexpr int GSTAGE = (GBM + GBN) * GROW;
constexpr int GLDS = 2 * GSTAGE;
constexpr int GTHREADS = 256;
constexpr int GTM = 2, GTN = 2;   // 32 x 32 blocks per wavefront: tokens, weight rows
constexpr int GLOADS = GBM * 8 / GTHREADS;     // 16-byte loads per thread per slab and operand

struct TileTaskF {
    const float* a_base;        // x or h
    const int32_t* gather;      // token_indices + row0, or null
    int64_t a_row0;
    const float* w[2];          // SwiGLU up projection: {w_gate, w_up} of the expert; otherwise the same matrix twice
    const float* bias[2];
    float* c_base;              // h or y at the first row of the block
    int K, N, rows, c0;
    int a_ld, b_ld;             // row pitch of the operands in elements (K, except for windows of a wider matrix)
    int act;                    // activation of the epilogue (MOE_ACT_NONE for SwiGLU pairs and the down projection)
    bool paired;
    bool publish;               // rows are read by other workgroups of the same launch
};

// PARTIAL: the row block holds fewer than 128 rows; 32-row blocks that lie entirely in the padding are skipped.
template <bool PARTIAL>
__device__ __forceinline__ void tile_mainloop_f32(const TileTaskF& p, unsigned char* smem, f32x16 (&acc)[GTM][GTN]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // 8 threads per row, LDS slot (row, c) holds global chunk c ^ ((row >> 1) & 7); a wavefront fills 8 consecutive rows
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ ((prow >> 1) & 7);
    const float* a_src[GLOADS];
    const float* b_src[GLOADS];
#pragma unroll
    for (int i = 0; i < GLOADS; ++i) {
        int r = prow + i * 32;
        if (r >= p.rows) r = 0;                                   // padding rows re-read row 0; never stored
        const int64_t src_row = p.gather ? (int64_t)p.gather[r] : p.a_row0 + r;
        a_src[i] = p.a_base + src_row * p.a_ld + chunk * 4;
        const int j = prow + i * 32;                              // row of the weight tile
        const float* base = p.w[0];
        int col;
        if (p.paired) {       // wavefront column w owns tile rows [64 w, 64 w + 64): 32 gate rows, then 32 up rows
            const int w = j >> 6, jj = j & 63;
            col = p.c0 + w * 32 + (jj & 31);
            base = (jj >> 5) ? p.w[1] : p.w[0];
        } else {
            col = p.c0 + j;
        }
        b_src[i] = base + (int64_t)col * p.b_ld + chunk * 4;
    }
    const int wrow = __builtin_amdgcn_readfirstlane(prow & ~7);
    auto issue = [&](int kt) {
        unsigned char* st = smem + (kt & 1) * GSTAGE;
#pragma unroll
        for (int i = 0; i < GLOADS; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(a_src[i] + kt * GBK), (lds_void*)(st + (wrow + i * 32) * GROW), 16,
                                             0, 0);
#pragma unroll
        for (int i = 0; i < GLOADS; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(b_src[i] + kt * GBK),
                                             (lds_void*)(st + (GBM + wrow + i * 32) * GROW), 16, 0, 0);
    };

    const int frow = lane & 31, fk = lane >> 5;
    const int sw = (frow >> 1) & 7;
    const int ta = PARTIAL ? min(GTM, max(0, (p.rows - wm * 32 * GTM + 31) >> 5)) : GTM;
    const int a_off = (wm * 32 * GTM + frow) * GROW;
    const int b_off = GBM * GROW + (wn * 32 * GTN + frow) * GROW;

#pragma unroll
    for (int i = 0; i < GTM; ++i)
#pragma unroll
        for (int j = 0; j < GTN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // eight k of a slab: lane (row, k half) reads k = 8 q + 4 (k half) .. + 3 of its rows; MFMA e takes element e of
    // both k halves
    auto quarter_slab = [&](const unsigned char* st, int q) {
        const int c = ((2 * q + fk) ^ sw) << 4;
        f32x4 af[GTM], bf[GTN];
#pragma unroll
        for (int j = 0; j < GTN; ++j) bf[j] = *reinterpret_cast<const f32x4*>(st + b_off + j * 32 * GROW + c);
#pragma unroll
        for (int i = 0; i < GTM; ++i)
            if (!PARTIAL || i < ta) af[i] = *reinterpret_cast<const f32x4*>(st + a_off + i * 32 * GROW + c);
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < GTM; ++i) {
                if (PARTIAL && i >= ta) continue;
#pragma unroll
                for (int j = 0; j < GTN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j][e], af[i][e], acc[i][j], 0, 0, 0);
            }
    };
    // every load of this wavefront has landed, its LDS reads are done; then the workgroup meets
    auto end_slab = [&]() {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    const int nk = p.K / GBK;               // 0 for the empty window of an expert without rows (weight gradient)
    __syncthreads();                        // the previous task may still be reading the stages
    if (nk > 0) issue(0);
    end_slab();
    for (int kt = 0; kt < nk; ++kt) {
        // slab kt sits in stage kt & 1; the other stage is free: every wavefront is past the barrier that ended slab kt - 1
        if (kt + 1 < nk) issue(kt + 1);
        const unsigned char* st = smem + (kt & 1) * GSTAGE;
#pragma unroll
        for (int q = 0; q < 4; ++q) quarter_slab(st, q);
        end_slab();
    }
}

// acc[i][j][v]: token row = 64 wm + 32 i + (lane & 31); weight row inside block j = 8 (v >> 2) + 4 (lane >> 5) + (v & 3).
__device__ __forceinline__ void store4(float* dst, const float (&o)[4], bool publish) {
    if (publish) {
        publish8(dst, __float_as_uint(o[0]), __float_as_uint(o[1]));
        publish8(dst + 2, __float_as_uint(o[2]), __float_as_uint(o[3]));
    } else {
        *reinterpret_cast<f32x4*>(dst) = f32x4{o[0], o[1], o[2], o[3]};
    }
}

__device__ __forceinline__ void tile_epilogue_f32(const TileTaskF& p, f32x16 (&acc)[GTM][GTN]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 31, fk = lane >> 5;
#pragma unroll
    for (int i = 0; i < GTM; ++i) {
        const int m = wm * 32 * GTM + i * 32 + frow;
        if (m >= p.rows) continue;
        float* crow = p.c_base + (int64_t)m * p.N;
        if (p.paired) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = p.c0 + wn * 32 + 8 * g + 4 * fk;
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float gt = acc[i][0][4 * g + r], u = acc[i][1][4 * g + r];
                    if (p.bias[0]) gt = gt + p.bias[0][col + r];
                    if (p.bias[1]) u = u + p.bias[1][col + r];
                    o[r] = silu(gt) * u;
                }
                store4(crow + col, o, p.publish);
            }
        } else {
#pragma unroll
            for (int j = 0; j < GTN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int col = p.c0 + wn * 64 + j * 32 + 8 * g + 4 * fk;
                    float o[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        o[r] = acc[i][j][4 * g + r];
                        if (p.bias[0]) o[r] = o[r] + p.bias[0][col + r];
                        o[r] = act_apply(o[r], p.act);
                    }
                    store4(crow + col, o, p.publish);
                }
        }
    }
}

__device__ __forceinline__ void f32_gemm_tile(const TileTaskF& p, unsigned char* smem) {
    f32x16 acc[GTM][GTN];
    if (p.rows < GBM) tile_mainloop_f32<true>(p, smem, acc);
    else tile_mainloop_f32<false>(p, smem, acc);
    tile_epilogue_f32(p, acc);
}

__device__ __forceinline__ TileTaskF resolve_tile_f32(const FfnArgs& a, const Task& t, bool publish) {
    TileTaskF p;
    p.publish = publish;
    const int64_t HI = (int64_t)a.H * a.I;
    p.rows = t.rows;
    p.act = MOE_ACT_NONE;
    p.paired = t.phase == 0 && a.act == MOE_ACT_SWIGLU;
    p.bias[1] = nullptr;
    if (t.phase == 0) {
        p.c0 = t.ntile * (p.paired ? GN0 : GN1);
        p.K = p.a_ld = p.b_ld = a.H;
        p.N = a.I;
        if (p.paired) {
            p.w[0] = (const float*)a.w_gate + t.expert * HI;
            p.w[1] = (const float*)a.w_up + t.expert * HI;
            p.bias[0] = a.b_gate ? (const float*)a.b_gate + (int64_t)t.expert * a.I : nullptr;
            p.bias[1] = a.b_up ? (const float*)a.b_up + (int64_t)t.expert * a.I : nullptr;
        } else {
            p.w[0] = p.w[1] = (const float*)a.w_up + t.expert * HI;
            p.bias[0] = a.b_up ? (const float*)a.b_up + (int64_t)t.expert * a.I : nullptr;
            p.act = a.act;
        }
        p.a_base = (const float*)a.x;
        p.gather = a.token_indices + t.row0;
        p.a_row0 = 0;
        p.c_base = (float*)a.h + (int64_t)t.row0 * a.I;
    } else {
        p.c0 = t.ntile * GN1;
        p.K = p.a_ld = p.b_ld = a.I;
        p.N = a.H;
        p.w[0] = p.w[1] = (const float*)a.w_down + t.expert * HI;
        p.bias[0] = a.b_down ? (const float*)a.b_down + (int64_t)t.expert * a.H : nullptr;
        p.a_base = (const float*)a.h;
        p.gather = nullptr;
        p.a_row0 = t.row0;
        p.c_base = (float*)a.y + (int64_t)t.row0 * a.H;
    }
    return p;
}

__global__ __launch_bounds__(GTHREADS) void ffn_tiled_f32_tile_kernel(FfnArgs a, int phase) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_list[1 + GBM];
    if (phase == 0) zero_unrouted_rows(a, 4);
    Task t;
    if (!tiled_task(a, phase, blockIdx.x, t)) return;
    const TileTaskF p = resolve_tile_f32(a, t, phase == 1 && a.arrive);
    f32_gemm_tile(p, smem);
    if (phase == 1 && a.arrive) combine_arrivals<float>(combine_args(a), t.row0, t.rows, t.ntile, p.c0, GN1, s_list);
}

__global__ __launch_bounds__(GTHREADS) void ffn_persistent_f32_tile_kernel(FfnArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_task, s_ok;
    __shared__ int s_cmb[kCombineLds];
    __shared__ int s_list[1 + GBM];
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
        const TileTaskF p = resolve_tile_f32(a, t, t.phase == 0 || publish_y(a));
        const long long started = trace_clock(a.task_trace);
        if (ok) f32_gemm_tile(p, smem);
        else poison_tile(p.c_base, p.rows, p.N, p.c0, p.paired ? GN0 : GN1, 4);
        if (a.task_trace) trace_task(a.task_trace, a.task_trace_cap, t.phase, t.expert, t.mtile, t.ntile, t.rows, started);
        if (t.phase == 0) signal_phase0_done(a.done0, t.mtile);
        else after_down_tile<float>(a, t.row0, t.rows, t.mtile, t.ntile, p.c0, GN1, s_list);
    }
    if (a.combined) combine_while_idle_narrow<float>(sweep_args(a), &s_task, s_cmb);
    queue_clock_stamp(a.wg_clock, 1);
}

// The same tile on dense operands (moe_gemm_bias_act): C[M,N] = act(A[M,K] . B[N,K]^T + bias), N % 128 = 0, K % 32 = 0.
__global__ __launch_bounds__(GTHREADS) void gemm_dense_f32_tile_kernel(const float* A, const float* B, const float* bias,
                                                                       float* C, int M, int N, int K, int act) {
    extern __shared__ __align__(16) unsigned char smem[];
    TileTaskF p;
    const int row0 = blockIdx.y * GBM;
    p.a_base = A; p.gather = nullptr; p.a_row0 = row0;
    p.w[0] = p.w[1] = B; p.bias[0] = bias; p.bias[1] = nullptr;
    p.c_base = C + (int64_t)row0 * N;
    p.K = p.a_ld = p.b_ld = K; p.N = N; p.rows = min(GBM, M - row0); p.c0 = blockIdx.x * GN1; p.act = act;
    p.paired = false; p.publish = false;
    f32_gemm_tile(p, smem);
}

// Grouped product over packed expert-major rows (backward.hip): out[r,:] = act(a_rows[r,:] . w[e(r)]^T + bias[e(r)]),
// one workgroup per (row block of 128 from `mtiles`, 128 output columns).  N % 128 = 0, K % 32 = 0.
__global__ __launch_bounds__(GTHREADS) void grouped_gemm_f32_tile_kernel(const float* a_rows, const float* w,
                                                                         const float* bias, float* out, const MTile* mtiles,
                                                                         const int32_t* num_mtiles, int nnt, int N, int K,
                                                                         int act) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int mt = blockIdx.x / nnt, nt = blockIdx.x % nnt;
    if (mt >= *num_mtiles) return;
    const MTile m = mtiles[mt];
    TileTaskF p;
    p.a_base = a_rows; p.gather = nullptr; p.a_row0 = m.row0;
    p.w[0] = p.w[1] = w + (int64_t)m.expert * N * K;
    p.bias[0] = bias ? bias + (int64_t)m.expert * N : nullptr; p.bias[1] = nullptr;
    p.c_base = out + (int64_t)m.row0 * N;
    p.K = p.a_ld = p.b_ld = K; p.N = N; p.rows = m.rows; p.c0 = nt * GN1; p.act = act;
    p.paired = false; p.publish = false;
    f32_gemm_tile(p, smem);
}

// Weight gradient of one expert: dw[e] [N,K] = dyT[:, window e] . aT[:, window e]^T over the expert's zero-padded
// window of packed rows (a multiple of 128 columns of the transposed operands, pitch ld).  K % 128 = 0.
// grid = (K / 128, ceil(N / 128), E).
__global__ __launch_bounds__(GTHREADS) void wgrad_f32_tile_kernel(const float* dyT, const float* aT, float* dw,
                                                                  const int32_t* poff, int N, int K, int64_t ld) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int e = blockIdx.z, row0 = blockIdx.y * GBM;
    TileTaskF p;
    p.a_base = dyT + poff[e]; p.gather = nullptr; p.a_row0 = row0;
    p.w[0] = p.w[1] = aT + poff[e]; p.bias[0] = p.bias[1] = nullptr;
    p.c_base = dw + (int64_t)e * N * K + (int64_t)row0 * K;
    p.K = poff[e + 1] - poff[e]; p.a_ld = p.b_ld = (int)ld; p.N = K; p.rows = min(GBM, N - row0); p.c0 = blockIdx.x * GN1;
    p.act = MOE_ACT_NONE; p.paired = false; p.publish = false;
    f32_gemm_tile(p, smem);
}

template <class K>
hipError_t allow_lds(K kernel) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, GLDS);
}

}  // namespace

int f32_tile_block_m() { return GBM; }
int f32_tile_block_n0(int swiglu) { return swiglu ? GN0 : GN1; }
int f32_tile_block_n1() { return GN1; }

int ffn_persistent_occupancy_f32_tile() {
    int n = 0;
    if (allow_lds(&ffn_persistent_f32_tile_kernel) != hipSuccess) return 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(&ffn_persistent_f32_tile_kernel),
                                                     GTHREADS, GLDS) != hipSuccess || n < 1)
        n = 1;
    return n;
}

bool gemm_dense_f32_takes_tile(int64_t M, int64_t N, int64_t K) {
    // full tiles only, and enough of them to occupy the chip (the 64 x 64 vector-ALU tiles spread small products wider)
    return N % GBN == 0 && K % GBK == 0 && M >= GBM && (M / GBM) * (N / GBN) >= 256;
}

hipError_t launch_gemm_dense_f32_tile(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                      int64_t K, int act, hipStream_t st) {
    hipError_t e = allow_lds(&gemm_dense_f32_tile_kernel);
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)(N / GBN), (unsigned)((M + GBM - 1) / GBM));
    gemm_dense_f32_tile_kernel<<<grid, GTHREADS, GLDS, st>>>((const float*)A, (const float*)B, (const float*)bias, (float*)C,
                                                             (int)M, (int)N, (int)K, act);
    return hipGetLastError();
}

bool grouped_gemm_f32_takes_tile(int64_t A, int N, int K) {
    return N % GBN == 0 && K % GBK == 0 && (A / GBM) * (N / GBN) >= 256;
}

hipError_t launch_grouped_gemm_f32_tile(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                        const int32_t* num_mtiles, int max_mtiles, int N, int K, int act, hipStream_t st) {
    hipError_t e = allow_lds(&grouped_gemm_f32_tile_kernel);
    if (e != hipSuccess) return e;
    const int nnt = N / GBN;
    grouped_gemm_f32_tile_kernel<<<(unsigned)max_mtiles * nnt, GTHREADS, GLDS, st>>>(
        (const float*)a_rows, (const float*)w, (const float*)bias, (float*)out, mtiles, num_mtiles, nnt, N, K, act);
    return hipGetLastError();
}

bool wgrad_f32_takes_tile(int E, int N, int K) { return K % GBN == 0 && (int64_t)E * (N / GBM) * (K / GBN) >= 128; }

hipError_t launch_wgrad_f32_tile(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K,
                                 int64_t ld, hipStream_t st) {
    hipError_t e = allow_lds(&wgrad_f32_tile_kernel);
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)(K / GBN), (unsigned)((N + GBM - 1) / GBM), (unsigned)E);
    wgrad_f32_tile_kernel<<<grid, GTHREADS, GLDS, st>>>((const float*)dyT, (const float*)aT, (float*)dw, poff, N, K, ld);
    return hipGetLastError();
}

hipError_t launch_ffn_f32_tile(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, int blocks, hipStream_t st) {
    if (blocks > 0) {
        hipError_t e = allow_lds(&ffn_persistent_f32_tile_kernel);
        if (e != hipSuccess) return e;
        ffn_persistent_f32_tile_kernel<<<blocks, GTHREADS, GLDS, st>>>(a);
    } else {
        hipError_t e = allow_lds(&ffn_tiled_f32_tile_kernel);
        if (e != hipSuccess) return e;
        ffn_tiled_f32_tile_kernel<<<tiled_grid(max_mtiles, nnt0, a.groups), GTHREADS, GLDS, st>>>(a, 0);
        ffn_tiled_f32_tile_kernel<<<tiled_grid(max_mtiles, nnt1, a.groups), GTHREADS, GLDS, st>>>(a, 1);
    }
    return hipGetLastError();
}

}  // namespace moe355
