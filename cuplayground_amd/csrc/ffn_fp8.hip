// Expert FFN for e4m3 weights with one fp32 scale per 128x128 block and bf16 activations (torch_dtype 4).
//
// The reference excludes fp8 (combine.cuh:129-131) and has no block-scaled GEMM, so the numerics are this
// library's: y[n] = sum over 128-wide k blocks of scale[n/128][kb] * (fp32 dot product of that block).  The
// data contract is still the reference GEMM's: weights (N,K) row-major, fp32 accumulation, one cast on store
// (mma.cuh:59,108-111,415-427).
//
// This shape is decode-like: a handful of token rows per expert against tens of megabytes of weights, so
// the kernel is a weight streamer.  A task is (expert, 16-token row block, chunk of weight rows -- 64 gate + 64 up rows
// per sub-tile of a SwiGLU up projection, 128 rows of one matrix otherwise):
//   * v_mfma_f32_16x16x32_bf16 with the weights as the "A" operand (16 weight rows) and up to 16 token rows
//     as "B"; e4m3 bytes are widened to bf16 in registers (exact) right before the MFMA;
//   * each lane fetches 16 contiguous weight bytes per 64-wide k slab, so a wavefront load covers 64
//     contiguous bytes of 16 rows and the four wavefronts of a workgroup, which interleave 128-wide k
//     blocks, together sweep 512 contiguous bytes of each row;
//   * each wavefront multiplies its k blocks against all 8 row groups of the task (activation fragments are
//     reused 8 times), scales the 128-deep partial sums by the block scale in fp32, and the four
//     wavefronts' sums meet in LDS for the epilogue (bias, SwiGLU, bf16 store).
#include "ffn_common.hpp"

namespace moe355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int QBM = 16;      // token rows per task
constexpr int QN0 = 64;      // intermediate columns per phase-0 sub-tile (64 gate rows + 64 up rows)
constexpr int QN1 = 128;     // output columns per phase-1 sub-tile
// Sub-tiles per task.  An up-projection task streams four (64 gate + 64 up rows x H bytes each): fewer pops, decodes
// and dependency counts per byte.  A down-projection task takes one: those are the last tasks of the queue, and the
// smaller they are the shorter the tail in which workgroups run dry.  Measured on the decode shape (H 7168, I 2048,
// 219 experts hit; kernel time, same box): (2, 2) 1.638 ms, (2, 4) 1.646, (2, 1) 1.621, (1, 1) 1.636, (4, 1) 1.606,
// (8, 1) 1.618, (16, 1) 1.93.
constexpr int QSUB = 4;
constexpr int QSUB1 = 1;
constexpr int QGROUPS = 8;   // 16-row weight groups per task
constexpr int QWAVES = 4;

union Frag {
    bf16x8 v;
    uint32_t u[4];
    uint4 q;
};

// 8 e4m3 bytes -> 8 bf16.  Every e4m3 value is exactly representable in bf16, so truncating the fp32
// conversion result is exact.
__device__ __forceinline__ bf16x8 widen8(uint32_t lo, uint32_t hi) {
    Frag f;
    const uint32_t w[2] = {lo, hi};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
        f.u[2 * i] = (__float_as_uint(a[0]) >> 16) | (__float_as_uint(a[1]) & 0xFFFF0000u);
        f.u[2 * i + 1] = (__float_as_uint(b[0]) >> 16) | (__float_as_uint(b[1]) & 0xFFFF0000u);
    }
    return f.v;
}

struct Fp8Task {
    const uint8_t* w[2];        // phase 0: {w_gate, w_up} of the expert; phase 1: {w_down, w_down}
    const float* s[2];          // matching scale rows: &scale[expert][n/128][0]
    const uint16_t* bias[2];
    const uint16_t* a_base;     // x or h
    const int32_t* gather;      // token_indices + row0, or null
    int64_t a_row0;
    uint16_t* c_base;           // h or y at the first row of the block
    int K, N, rows, c0, phase;
    int act;        // up projection without SwiGLU: the activation of the epilogue (else MOE_ACT_NONE)
    bool paired;    // up projection with SwiGLU: 64 gate rows + 64 up rows per sub-tile; otherwise 128 rows of one matrix
    bool publish;   // rows are read by other workgroups of the same launch
};

__device__ __forceinline__ void fp8_tile(const Fp8Task& t, float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int idx = lane & 15, kg = lane >> 4;

    // activation row of this lane (B operand column); rows past the block re-read row 0 and are never stored
    const int ar = idx < t.rows ? idx : 0;
    const int64_t src_row = t.gather ? (int64_t)t.gather[ar] : t.a_row0 + ar;
    const uint16_t* xp = t.a_base + src_row * t.K + 16 * kg;

    // weight rows of this lane, one per group
    const uint8_t* wp[QGROUPS];
#pragma unroll
    for (int g = 0; g < QGROUPS; ++g) {
        int n;
        const uint8_t* base;
        if (t.paired) {
            n = t.c0 + (g & 3) * 16 + idx;
            base = t.w[g >> 2];
        } else {
            n = t.c0 + g * 16 + idx;
            base = t.w[0];
        }
        wp[g] = base + (int64_t)n * t.K + 16 * kg;
    }

    f32x4 acc[QGROUPS];
#pragma unroll
    for (int g = 0; g < QGROUPS; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int KB = t.K >> 7;
    for (int kb = wave; kb < KB; kb += QWAVES) {
        const int k0 = kb << 7;
        uint4 wv[QGROUPS][2];
#pragma unroll
        for (int g = 0; g < QGROUPS; ++g)
#pragma unroll
            for (int s = 0; s < 2; ++s) wv[g][s] = *reinterpret_cast<const uint4*>(wp[g] + k0 + 64 * s);
        Frag xa[2][2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            xa[s][0].q = *reinterpret_cast<const uint4*>(xp + k0 + 64 * s);
            xa[s][1].q = *reinterpret_cast<const uint4*>(xp + k0 + 64 * s + 8);
        }
        const float sc0 = t.s[0][kb], sc1 = t.s[1][kb];
#pragma unroll
        for (int g = 0; g < QGROUPS; ++g) {
            f32x4 part = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(widen8(wv[g][s].x, wv[g][s].y), xa[s][0].v, part, 0, 0, 0);
                part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(widen8(wv[g][s].z, wv[g][s].w), xa[s][1].v, part, 0, 0, 0);
            }
            const float sc = (t.paired && g >= 4) ? sc1 : sc0;
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[g][r] = __builtin_fmaf(sc, part[r], acc[g][r]);
        }
    }

    // ---- cross-wave sum in LDS: red[wave][group][r][lane] ----
    __syncthreads();   // a previous task's epilogue may still be reading red
#pragma unroll
    for (int g = 0; g < QGROUPS; ++g)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((wave * QGROUPS + g) * 4 + r) * 64 + lane] = acc[g][r];
    __syncthreads();

    // wave w finishes groups w and w+4: acc layout gives this lane token row `idx` and weight rows 4*kg + r
    float v[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < QWAVES; ++w) s = s + red[((w * QGROUPS + wave + 4 * h) * 4 + r) * 64 + lane];
            v[h][r] = s;
        }
    if (idx >= t.rows) return;
    uint16_t* crow = t.c_base + (int64_t)idx * t.N;
    if (t.paired) {
        const int col = t.c0 + wave * 16 + 4 * kg;
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float g = v[0][r], u = v[1][r];
            if (t.bias[0]) g = g + bf16_bits_to_f32(t.bias[0][col + r]);
            if (t.bias[1]) u = u + bf16_bits_to_f32(t.bias[1][col + r]);
            o[r] = silu(g) * u;
        }
        uint2 st;
        st.x = pack2_bf16(o[0], o[1]);
        st.y = pack2_bf16(o[2], o[3]);
        if (t.publish) publish8(crow + col, st.x, st.y);
        else *reinterpret_cast<uint2*>(crow + col) = st;
    } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int col = t.c0 + (wave + 4 * h) * 16 + 4 * kg;
            float o[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                o[r] = v[h][r];
                if (t.bias[0]) o[r] = o[r] + bf16_bits_to_f32(t.bias[0][col + r]);
                o[r] = act_apply(o[r], t.act);
            }
            uint2 st;
            st.x = pack2_bf16(o[0], o[1]);
            st.y = pack2_bf16(o[2], o[3]);
            if (t.publish) publish8(crow + col, st.x, st.y);
            else *reinterpret_cast<uint2*>(crow + col) = st;
        }
    }
}

__device__ __forceinline__ Fp8Task resolve_fp8(const FfnArgs& a, const Task& t, int sub, bool publish) {
    Fp8Task p;
    p.publish = publish;
    const int64_t HI = (int64_t)a.H * a.I;
    const int kbH = a.H >> 7, kbI = a.I >> 7;
    p.phase = t.phase;
    p.rows = t.rows;
    p.act = MOE_ACT_NONE;
    p.paired = t.phase == 0 && a.act == MOE_ACT_SWIGLU;
    if (t.phase == 0) {
        p.c0 = (t.ntile * QSUB + sub) * (p.paired ? QN0 : QN1);
        p.K = a.H;
        p.N = a.I;
        const int64_t srow = ((int64_t)t.expert * (a.I >> 7) + (p.c0 >> 7)) * kbH;
        if (p.paired) {
            p.w[0] = (const uint8_t*)a.w_gate + t.expert * HI;
            p.w[1] = (const uint8_t*)a.w_up + t.expert * HI;
            p.s[0] = a.s_gate + srow;
            p.s[1] = a.s_up + srow;
            p.bias[0] = a.b_gate ? (const uint16_t*)a.b_gate + (int64_t)t.expert * a.I : nullptr;
            p.bias[1] = a.b_up ? (const uint16_t*)a.b_up + (int64_t)t.expert * a.I : nullptr;
        } else {
            p.w[0] = p.w[1] = (const uint8_t*)a.w_up + t.expert * HI;
            p.s[0] = p.s[1] = a.s_up + srow;
            p.bias[0] = a.b_up ? (const uint16_t*)a.b_up + (int64_t)t.expert * a.I : nullptr;
            p.bias[1] = nullptr;
            p.act = a.act;
        }
        p.a_base = (const uint16_t*)a.x;
        p.gather = a.token_indices + t.row0;
        p.a_row0 = 0;
        p.c_base = (uint16_t*)a.h + (int64_t)t.row0 * a.I;
    } else {
        p.c0 = (t.ntile * QSUB1 + sub) * QN1;
        p.K = a.I;
        p.N = a.H;
        p.w[0] = p.w[1] = (const uint8_t*)a.w_down + t.expert * HI;
        const int64_t srow = ((int64_t)t.expert * (a.H >> 7) + (p.c0 >> 7)) * kbI;
        p.s[0] = p.s[1] = a.s_down + srow;
        p.bias[0] = a.b_down ? (const uint16_t*)a.b_down + (int64_t)t.expert * a.H : nullptr;
        p.bias[1] = nullptr;
        p.a_base = (const uint16_t*)a.h;
        p.gather = nullptr;
        p.a_row0 = t.row0;
        p.c_base = (uint16_t*)a.y + (int64_t)t.row0 * a.H;
    }
    return p;
}

__global__ __launch_bounds__(256) void ffn_tiled_fp8_kernel(FfnArgs a, int phase) {
    __shared__ float red[QWAVES * QGROUPS * 4 * 64];
    __shared__ int s_list[1 + QBM];
    if (phase == 0) zero_unrouted_rows(a, 2);
    Task t;
    if (!tiled_task(a, phase, blockIdx.x, t)) return;
    for (int sub = 0; sub < (phase ? QSUB1 : QSUB); ++sub) {
        const Fp8Task p = resolve_fp8(a, t, sub, phase == 1 && a.arrive);
        if (p.c0 < p.N) fp8_tile(p, red);
    }
    if (phase == 1 && a.arrive) combine_arrivals<bf16_s>(combine_args(a), t.row0, t.rows, t.ntile, t.ntile * QSUB1 * QN1, QSUB1 * QN1, s_list);
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void ffn_persistent_fp8_kernel(FfnArgs a) {
    __shared__ float red[QWAVES * QGROUPS * 4 * 64];
    __shared__ int s_task, s_ok;
    __shared__ int s_cmb[kCombineLds];
    __shared__ int s_list[1 + QBM];
    queue_kernel_entry();
    queue_clock_stamp(a.wg_clock, 0);
    zero_unrouted_rows(a, 2);
    const int ids = a.q->ids_queue;
    const int nseg = a.q->nseg;
    const int nnt0 = a.seg_phase0[0].nnt;
    QueueCursor cur = queue_cursor(a.groups);
    Task t;
    while (next_task(a, cur, &s_task, ids, nseg, nnt0, t)) {
        int ok = 1;
        if (t.phase == 1) ok = wait_phase0_done(a.done0, t.mtile, nnt0, a.spin_limit, a.q, a.host_stall, &s_ok);
        const long long started = trace_clock(a.task_trace);
        for (int sub = 0; sub < (t.phase ? QSUB1 : QSUB); ++sub) {
            const Fp8Task p = resolve_fp8(a, t, sub, t.phase == 0 || publish_y(a));
            if (p.c0 >= p.N) continue;
            if (ok) fp8_tile(p, red);
            else poison_tile(p.c_base, p.rows, p.N, p.c0, QN1, 2);
        }
        if (a.task_trace) trace_task(a.task_trace, a.task_trace_cap, t.phase, t.expert, t.mtile, t.ntile, t.rows, started);
        if (t.phase == 0) signal_phase0_done(a.done0, t.mtile);
        else after_down_tile<bf16_s>(a, t.row0, t.rows, t.mtile, t.ntile, t.ntile * QSUB1 * QN1, QSUB1 * QN1, s_list);
    }
    if (a.combined) combine_while_idle_narrow<bf16_s>(sweep_args(a), &s_task, s_cmb);
    queue_clock_stamp(a.wg_clock, 1);
}

}  // namespace

int fp8_block_m() { return QBM; }
int fp8_block_n0(int swiglu) { return (swiglu ? QN0 : QN1) * QSUB; }
int fp8_block_n1() { return QN1 * QSUB1; }

int ffn_persistent_occupancy_fp8() {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(&ffn_persistent_fp8_kernel), 256,
                                                     0) != hipSuccess || n < 1)
        n = 1;
    return n;
}

hipError_t launch_ffn_fp8(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, int blocks, hipStream_t st) {
    if (blocks > 0) {
        ffn_persistent_fp8_kernel<<<blocks, 256, 0, st>>>(a);
    } else {
        ffn_tiled_fp8_kernel<<<tiled_grid(max_mtiles, nnt0, a.groups), 256, 0, st>>>(a, 0);
        ffn_tiled_fp8_kernel<<<tiled_grid(max_mtiles, nnt1, a.groups), 256, 0, st>>>(a, 1);
    }
    return hipGetLastError();
}

}  // namespace moe355
