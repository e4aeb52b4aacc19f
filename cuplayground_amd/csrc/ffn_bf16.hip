// Expert FFN on bf16 MFMA: the tile GEMM "processor" of the reference, rebuilt for gfx950.
//
// Contract kept from the reference (mma.cuh:46-179, processor/tiling.cuh:273-323): C = act(A.B^T + bias)
// with A (M,K) and B (N,K) row-major, fp32 accumulation, one cast to the storage type on store, epilogue
// order add-then-activate (processor/tiling.cuh:29-38).  Everything else is designed for CDNA4:
//   * v_mfma_f32_32x32x16_bf16; the weight tile is the MFMA "A" operand and the token tile the "B" operand,
//     so each lane ends up with 4 consecutive output columns of one token row and stores 8 bytes at a time;
//   * tiles are staged through LDS in 128-byte rows (64 bf16 of K) whose 16-byte chunks are xor-swizzled
//     with the row number, which makes both the ds_write_b128 and the ds_read_b128 patterns conflict free;
//   * LDS is double buffered and the next K slab is fetched into registers while the current one feeds the
//     matrix cores: one barrier per slab;
//   * dispatch is fused into the A-tile load: phase 0 gathers token rows through token_indices[];
//   * SwiGLU pairs gate and up columns inside one wavefront (first half of its columns from w_gate, second
//     half from w_up), so silu(g)*u happens in registers.
#include "ffn_common.hpp"

namespace moe355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

constexpr int kBK = 64;               // bf16 elements of K per slab = one 128-byte LDS row
constexpr int kRowBytes = kBK * 2;

template <int BM_, int BN_, int WM_, int WN_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int THREADS = WM * WN * kWave;
    static constexpr int TM = BM / WM / 32;       // 32x32 MFMA tiles per wavefront along tokens
    static constexpr int TN = BN / WN / 32;       // ... along weight rows
    static constexpr int ROWS_PER_PASS = THREADS / 8;
    static constexpr int RA = BM / ROWS_PER_PASS; // 16-byte loads per thread per slab, token tile
    static constexpr int RB = BN / ROWS_PER_PASS; // ... weight tile
    static constexpr int STAGE_BYTES = (BM + BN) * kRowBytes;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static_assert(TM >= 1 && TN >= 1 && RA >= 1 && RB >= 1, "tile too small for the wave grid");
    static_assert(TN % 2 == 0, "SwiGLU pairs column tiles inside a wavefront");
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * kRowBytes + ((chunk ^ (row & 7)) << 4); }

// What one task needs, resolved to pointers.
struct TaskPtrs {
    const uint16_t* a_base;      // phase 0: x; phase 1: h
    const int32_t* gather;       // phase 0: token_indices + row0; phase 1: null
    int64_t a_row0;              // phase 1: first row of h
    int a_ld;                    // K
    const uint16_t* b0;          // weight matrix of this expert (w_up or w_down)
    const uint16_t* b1;          // SwiGLU: w_gate of this expert, else null
    const uint16_t* bias0;
    const uint16_t* bias1;
    uint16_t* c_base;            // h or y, first row of the block
    int N;                       // output columns (I for phase 0, H for phase 1)
    int K;
    int rows;
    int n0;                      // first output column of this tile
    int act;                     // epilogue
    bool swiglu;
};

template <class T>
__device__ __forceinline__ void gemm_tile(const TaskPtrs& p, unsigned char* smem) {
    constexpr int BM = T::BM, BN = T::BN, TM = T::TM, TN = T::TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / T::WN, wn = wave % T::WN;
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ (prow & 7);   // LDS slot (row, c) holds global chunk c ^ (row & 7)

    // ---- per-thread source rows ----
    const uint16_t* a_src[T::RA];
    const uint16_t* b_src[T::RB];
#pragma unroll
    for (int i = 0; i < T::RA; ++i) {
        int r = prow + i * T::ROWS_PER_PASS;
        if (r >= p.rows) r = 0;                                   // padding rows re-read row 0; never stored
        const int64_t src_row = p.gather ? (int64_t)p.gather[r] : p.a_row0 + r;
        a_src[i] = p.a_base + src_row * p.a_ld + chunk * 8;
    }
#pragma unroll
    for (int i = 0; i < T::RB; ++i) {
        const int j = prow + i * T::ROWS_PER_PASS;                // row of the weight tile
        const uint16_t* base = p.b0;
        int col;
        if (p.swiglu) {
            constexpr int WCOLS = BN / T::WN;                     // tile rows owned by one wavefront column
            const int w = j / WCOLS, jj = j % WCOLS;
            const int half = jj / (WCOLS / 2);
            col = p.n0 + w * (WCOLS / 2) + (jj % (WCOLS / 2));
            base = half ? p.b0 : p.b1;                            // first half gate, second half up
        } else {
            col = p.n0 + j;
        }
        if (col >= p.N) col = p.N - 1;                            // ragged last tile; never stored
        b_src[i] = base + (int64_t)col * p.K + chunk * 8;
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // Slab kt of both tiles goes from global memory straight into LDS stage kt % 2 (no VGPR staging): one
    // global_load_lds_dwordx4 per 8 rows and wavefront writes 1 KiB of consecutive LDS, lane l landing in
    // row (l >> 3), chunk slot (l & 7); the xor swizzle is applied on the global side (see a_src / b_src).
    const int wrow = __builtin_amdgcn_readfirstlane(prow & ~7);
    const int KT = p.K / kBK;
    auto issue = [&](int kt, int stage) {
        unsigned char* sa = smem + stage * T::STAGE_BYTES;
        unsigned char* sb = sa + BM * kRowBytes;
        const int koff = kt * kBK;
#pragma unroll
        for (int i = 0; i < T::RA; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(a_src[i] + koff),
                                             (lds_void*)(sa + (wrow + i * T::ROWS_PER_PASS) * kRowBytes), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < T::RB; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(b_src[i] + koff),
                                             (lds_void*)(sb + (wrow + i * T::ROWS_PER_PASS) * kRowBytes), 16, 0, 0);
    };
    __syncthreads();                        // the previous task's last slab may still be being read
    issue(0, 0);
    const int frow = lane & 31, fk = lane >> 5;
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's share of slab kt has landed
        __syncthreads();                                    // ... and everyone else's; stage cur^1 is free again
        if (kt + 1 < KT) issue(kt + 1, cur ^ 1);
        const unsigned char* sa = smem + cur * T::STAGE_BYTES;
        const unsigned char* sb = sa + BM * kRowBytes;
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            bf16x8 af[TM], bfr[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[i] = *reinterpret_cast<const bf16x8*>(sa + swz(wm * 32 * TM + i * 32 + frow, ks * 2 + fk));
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bfr[j] = *reinterpret_cast<const bf16x8*>(sb + swz(wn * 32 * TN + j * 32 + frow, ks * 2 + fk));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
        }
    }

    // ---- epilogue ----
    // acc[i][j][r]: token row = wm*32*TM + i*32 + (lane & 31);
    //               weight row inside the 32-wide MFMA tile = 8*(r/4) + 4*(lane >> 5) + (r % 4)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = wm * 32 * TM + i * 32 + frow;
        if (m >= p.rows) continue;
        uint16_t* crow = p.c_base + (int64_t)m * p.N;
        if (p.swiglu) {
#pragma unroll
            for (int j = 0; j < TN / 2; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int col = p.n0 + wn * 16 * TN + j * 32 + 8 * q + 4 * fk;
                    if (col >= p.N) continue;
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float g = acc[i][j][4 * q + r], u = acc[i][j + TN / 2][4 * q + r];
                        if (p.bias1) g = g + bf16_bits_to_f32(p.bias1[col + r]);
                        if (p.bias0) u = u + bf16_bits_to_f32(p.bias0[col + r]);
                        v[r] = silu(g) * u;
                    }
                    uint2 o;
                    o.x = pack2_bf16(v[0], v[1]);
                    o.y = pack2_bf16(v[2], v[3]);
                    *reinterpret_cast<uint2*>(crow + col) = o;
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int col = p.n0 + wn * 32 * TN + j * 32 + 8 * q + 4 * fk;
                    if (col >= p.N) continue;
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float u = acc[i][j][4 * q + r];
                        if (p.bias0) u = u + bf16_bits_to_f32(p.bias0[col + r]);
                        v[r] = act_apply(u, p.act);
                    }
                    uint2 o;
                    o.x = pack2_bf16(v[0], v[1]);
                    o.y = pack2_bf16(v[2], v[3]);
                    *reinterpret_cast<uint2*>(crow + col) = o;
                }
            }
        }
    }
}

template <class T>
__device__ __forceinline__ TaskPtrs resolve(const FfnArgs& a, const Task& t) {
    TaskPtrs p;
    const int64_t HI = (int64_t)a.H * a.I;
    const bool sw = a.act == MOE_ACT_SWIGLU;
    if (t.phase == 0) {
        p.a_base = (const uint16_t*)a.x;
        p.gather = a.token_indices + t.row0;
        p.a_row0 = 0;
        p.a_ld = a.H;
        p.b0 = (const uint16_t*)a.w_up + t.expert * HI;
        p.b1 = sw ? (const uint16_t*)a.w_gate + t.expert * HI : nullptr;
        p.bias0 = a.b_up ? (const uint16_t*)a.b_up + (int64_t)t.expert * a.I : nullptr;
        p.bias1 = (sw && a.b_gate) ? (const uint16_t*)a.b_gate + (int64_t)t.expert * a.I : nullptr;
        p.c_base = (uint16_t*)a.h + (int64_t)t.row0 * a.I;
        p.N = a.I;
        p.K = a.H;
        p.n0 = t.ntile * (sw ? T::BN / 2 : T::BN);
        p.act = a.act;
        p.swiglu = sw;
    } else {
        p.a_base = (const uint16_t*)a.h;
        p.gather = nullptr;
        p.a_row0 = t.row0;
        p.a_ld = a.I;
        p.b0 = (const uint16_t*)a.w_down + t.expert * HI;
        p.b1 = nullptr;
        p.bias0 = a.b_down ? (const uint16_t*)a.b_down + (int64_t)t.expert * a.H : nullptr;
        p.bias1 = nullptr;
        p.c_base = (uint16_t*)a.y + (int64_t)t.row0 * a.H;
        p.N = a.H;
        p.K = a.I;
        p.n0 = t.ntile * T::BN;
        p.act = MOE_ACT_NONE;
        p.swiglu = false;
    }
    p.rows = t.rows;
    return p;
}

// One launch per phase; workgroup b runs task b of that phase.
template <class T>
__global__ __launch_bounds__(T::THREADS) void ffn_tiled_kernel(FfnArgs a, int phase) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int ntasks = phase ? a.q->tasks_phase1 : a.q->tasks_phase0;
    const int id = blockIdx.x;
    if (id >= ntasks) return;
    const int nnt0 = a.seg_phase0[0].nnt;
    const Task t = decode_task(phase ? a.seg_phase1 : a.seg_phase0, a.E, a.mtiles, id, nnt0);
    const TaskPtrs p = resolve<T>(a, t);
    gemm_tile<T>(p, smem);
}

// Persistent workgroups popping (expert, tile) tasks from one global atomic counter.
template <class T>
__global__ __launch_bounds__(T::THREADS) void ffn_persistent_kernel(FfnArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_task;
    const int total = a.q->total_tasks;
    const int nseg = a.q->nseg;
    const int nnt0 = a.seg_phase0[0].nnt;
    for (;;) {
        const int id = __builtin_amdgcn_readfirstlane(pop_task(&a.q->head, &s_task));
        if (id >= total) break;             // uniform exit: every wavefront leaves here
        const Task t = decode_task(a.seg_queue, nseg, a.mtiles, id, nnt0);
        if (t.phase == 1) wait_phase0_done(a.done0, t.mtile, nnt0, a.spin_limit, a.q);
        const TaskPtrs p = resolve<T>(a, t);
        gemm_tile<T>(p, smem);
        if (t.phase == 0) signal_phase0_done(a.done0, t.mtile);
    }
}

// The bare reference contract on dense operands: rows [b*BM, ...) of A, one "expert".
template <class T>
__global__ __launch_bounds__(T::THREADS) void gemm_dense_kernel(const uint16_t* A, const uint16_t* B,
                                                                const uint16_t* bias, uint16_t* C, int M, int N, int K,
                                                                int act) {
    extern __shared__ __align__(16) unsigned char smem[];
    TaskPtrs p;
    const int row0 = blockIdx.y * T::BM;
    p.a_base = A;
    p.gather = nullptr;
    p.a_row0 = row0;
    p.a_ld = K;
    p.b0 = B;
    p.b1 = nullptr;
    p.bias0 = bias;
    p.bias1 = nullptr;
    p.c_base = C + (int64_t)row0 * N;
    p.N = N;
    p.K = K;
    p.rows = min(T::BM, M - row0);
    p.n0 = blockIdx.x * T::BN;
    p.act = act;
    p.swiglu = false;
    gemm_tile<T>(p, smem);
}

using TileA = Tile<128, 128, 2, 2>;   // 256 threads, 64x64 per wavefront, 64 KiB LDS

template <class K>
hipError_t allow_lds(K kernel, int bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               bytes);
}

}  // namespace

int bf16_block_m() { return TileA::BM; }
int bf16_block_n() { return TileA::BN; }

hipError_t launch_ffn_tiled_bf16(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, hipStream_t st) {
    using T = TileA;
    hipError_t e = allow_lds(&ffn_tiled_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    ffn_tiled_kernel<T><<<max_mtiles * nnt0, T::THREADS, T::LDS_BYTES, st>>>(a, 0);
    ffn_tiled_kernel<T><<<max_mtiles * nnt1, T::THREADS, T::LDS_BYTES, st>>>(a, 1);
    return hipGetLastError();
}

hipError_t launch_ffn_persistent_bf16(const FfnArgs& a, int blocks, hipStream_t st) {
    using T = TileA;
    hipError_t e = allow_lds(&ffn_persistent_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    ffn_persistent_kernel<T><<<blocks, T::THREADS, T::LDS_BYTES, st>>>(a);
    return hipGetLastError();
}

int ffn_persistent_occupancy_bf16() {
    using T = TileA;
    int n = 0;
    if (allow_lds(&ffn_persistent_kernel<T>, T::LDS_BYTES) != hipSuccess) return 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(&ffn_persistent_kernel<T>),
                                                     T::THREADS, T::LDS_BYTES) != hipSuccess || n < 1)
        n = 1;
    return n;
}

hipError_t launch_gemm_dense_bf16(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                  int64_t K, int act, hipStream_t st) {
    using T = TileA;
    hipError_t e = allow_lds(&gemm_dense_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)((N + T::BN - 1) / T::BN), (unsigned)((M + T::BM - 1) / T::BM));
    gemm_dense_kernel<T><<<grid, T::THREADS, T::LDS_BYTES, st>>>((const uint16_t*)A, (const uint16_t*)B,
                                                                 (const uint16_t*)bias, (uint16_t*)C, (int)M, (int)N,
                                                                 (int)K, act);
    return hipGetLastError();
}

}  // namespace moe355
