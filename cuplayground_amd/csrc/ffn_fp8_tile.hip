// Expert FFN for e4m3 weights with 128x128 block scales when every expert sees many token rows (prefill-sized
// batches of torch_dtype 4).  ffn_fp8.hip streams the weights once per 16-token row block, which is right for
// decode and wrong here: with hundreds of rows per expert each weight byte would be fetched again for every 16 rows.
// This file is the tile GEMM of the reference (mma.cuh:46-179: C = act(A.B^T + bias), A (M,K), B (N,K) row-major,
// fp32 accumulation, one cast on store) for that operand pair, with the numerics of ffn_fp8.hip:
//   y[n] = sum over 128-wide k blocks of scale[n/128][kb] * (fp32 dot product of that block).
//
// A task is (expert, 128-token row block, 128 weight rows): 64 gate + 64 up rows for a SwiGLU up projection (the pairs
// stay inside a lane), 128 rows of w_up for ReLU / GELU layers, 128 rows of w_down for the down projection; so all
// weight rows of a wavefront's fragments lie in one scale block and the scale of a k block is one scalar (two for a
// SwiGLU up projection).
//   * four wavefronts of 64 x 64 outputs, v_mfma_f32_16x16x32_bf16, weights as the "A" operand;
//   * K slabs of 64: token rows go from global memory straight into LDS (global_load ... lds) as 128-byte rows with
//     xor-swizzled 16-byte chunks; weight bytes are fetched into registers two slabs ahead, widened to bf16 once per
//     workgroup (cvt_pk_f32_fp8 + byte permute, exact) and written to LDS in the same layout, so the fragment reads and
//     MFMAs are those of a bf16 tile;
//   * a second accumulator set takes the 128-deep partial sums (its first MFMA of a k block starts from zero); after
//     every second slab acc = fma(scale, partial, acc) in fp32;
//   * two 32 KiB LDS stages per workgroup, two workgroups per compute unit.
#include <type_traits>

#include "ffn_common.hpp"

namespace moe355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

constexpr int PBM = 128;          // token rows per row block
constexpr int PBN = 128;          // weight rows per tile
constexpr int PN0 = 64;           // intermediate columns per up-projection task (64 gate + 64 up rows)
constexpr int PN1 = 128;          // output columns per down-projection task
constexpr int PBK = 64;           // k per slab
constexpr int PROW = 128;         // bytes per LDS row (64 bf16)
constexpr int PSTAGE = (PBM + PBN) * PROW;
constexpr int PLDS = 2 * PSTAGE;
constexpr int PLDS_M8 = PLDS + 2 * PBM * 4;       // e4m3 x e4m3 loop: behind the two stages, the token rows' scales of either slab
constexpr int PTHREADS = 256;
constexpr int PTM = 4, PTN = 4;   // 16 x 16 fragments per wavefront: tokens, weight rows
constexpr int PRA = PBM * 8 / PTHREADS;        // 16-byte token loads per thread per slab
constexpr int PRB = PBN * 4 / PTHREADS;        // 16-byte weight loads (16 e4m3 values) per thread per slab

struct TileTask {
    const uint16_t* a_base;     // x or h
    const int32_t* gather;      // token_indices + row0, or null
    int64_t a_row0;
    const uint8_t* w[2];        // up projection: {w_gate, w_up} of the expert; down projection: {w_down, w_down}
    const float* s[2];          // their scale rows: &scale[expert][c0 / 128][0]
    const uint16_t* bias[2];
    uint16_t* c_base;           // h or y at the first row of the block
    int K, N, rows, c0, phase;
    int act;                    // up projection without SwiGLU: the activation of the epilogue (else MOE_ACT_NONE)
    bool paired;                // up projection with SwiGLU: 64 gate + 64 up rows; otherwise 128 rows of one matrix
    bool publish;               // rows are read by other workgroups of the same launch
    // e4m3 x e4m3 plan: the token operand as e4m3 codes (rows as a_base's: gathered or a_row0 + r) and its scales
    const uint8_t* aq;          // [*, K]
    const float* sa;            // [*, K / 128]
};

// 16 e4m3 bytes -> 2 x 8 bf16.  Every e4m3 value is a bf16 value, so the upper half of its fp32 form is exact.
__device__ __forceinline__ void widen16(const u32x4& q, u32x4& lo, u32x4& hi) {
    const uint32_t w[4] = {q[0], q[1], q[2], q[3]};
    uint32_t o[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
        o[2 * i] = __builtin_amdgcn_perm(__float_as_uint(a[1]), __float_as_uint(a[0]), 0x07060302u);
        o[2 * i + 1] = __builtin_amdgcn_perm(__float_as_uint(b[1]), __float_as_uint(b[0]), 0x07060302u);
    }
    lo = u32x4{o[0], o[1], o[2], o[3]};
    hi = u32x4{o[4], o[5], o[6], o[7]};
}

// PARTIAL: the row block holds fewer than 128 rows; fragments that lie entirely in the padding are skipped.
template <bool PARTIAL>
__device__ __forceinline__ void tile_mainloop(const TileTask& p, unsigned char* smem, f32x4 (&acc)[PTM][PTN]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // token rows: 8 threads per row, LDS slot (row, c) holds global chunk c ^ ((row >> 1) & 7)
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ ((prow >> 1) & 7);
    const uint16_t* a_src[PRA];
#pragma unroll
    for (int i = 0; i < PRA; ++i) {
        int r = prow + i * 32;
        if (r >= p.rows) r = 0;                                   // padding rows re-read row 0; never stored
        const int64_t src_row = p.gather ? (int64_t)p.gather[r] : p.a_row0 + r;
        a_src[i] = p.a_base + src_row * p.K + chunk * 8;
    }
    // weight rows: 4 threads per row, 16 e4m3 bytes each = two bf16 chunks of the LDS row.  Which lanes take which rows
    // decides the bank conflicts of the 16-byte LDS writes: the LDS serves such a write eight consecutive lanes at a time,
    // 128 bytes a cycle, so the eight must differ in their 16-byte position modulo 128 bytes -- the row does not matter,
    // rows are 128 bytes apart.  Four lanes of a row write chunks {0, 2, 4, 6} ^ swizzle (then {1, 3, 5, 7} ^ swizzle);
    // the other four lanes of the pass must therefore sit in a row whose swizzle differs in its lowest bit: rows r and
    // r + 2.  (With lanes 4..7 in row r + 1, which has the swizzle of row r, every such write took twice its cycles:
    // a conflict in every fourth LDS cycle of the kernel, measured with two-lane and whole-wavefront probes under
    // SQ_LDS_BANK_CONFLICT.)
    const int t = tid >> 2;
    const int brow = (t & ~3) | ((t & 1) << 1) | ((t >> 1) & 1), bc = tid & 3;
    const uint8_t* b_src[PRB];
    int b_dst[PRB][2];
#pragma unroll
    for (int i = 0; i < PRB; ++i) {
        const int j = brow + i * 64;                              // row of the weight tile
        const uint8_t* base = p.w[0];
        int col;
        if (p.paired) {       // wavefront column w owns tile rows [64 w, 64 w + 64): 32 gate rows, then 32 up rows
            const int w = j >> 6, jj = j & 63;
            col = p.c0 + w * 32 + (jj & 31);
            base = (jj >> 5) ? p.w[1] : p.w[0];
        } else {
            col = p.c0 + j;
        }
        b_src[i] = base + (int64_t)col * p.K + bc * 16;
        const int sw = (j >> 1) & 7;
        b_dst[i][0] = PBM * PROW + j * PROW + (((2 * bc) ^ sw) << 4);
        b_dst[i][1] = PBM * PROW + j * PROW + (((2 * bc + 1) ^ sw) << 4);
    }

    const int wrow = __builtin_amdgcn_readfirstlane(prow & ~7);
    auto issue_a = [&](int kt) {
        unsigned char* sa = smem + (kt & 1) * PSTAGE;
#pragma unroll
        for (int i = 0; i < PRA; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(a_src[i] + kt * PBK),
                                             (lds_void*)(sa + (wrow + i * 32) * PROW), 16, 0, 0);
    };
    // The weight bytes travel through registers for more than a slab.  Their loads are written in assembly so that the
    // wait for them can say "all but the PRA token-row loads issued since" -- the compiler, which sees direct-to-LDS
    // loads and register loads in one counter, would wait for everything.
    u32x4 breg[PRB];
    auto fetch_b = [&](int kt) {
#pragma unroll
        for (int i = 0; i < PRB; ++i)
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(breg[i]) : "v"(b_src[i] + kt * PBK) : "memory");
    };
    auto store_b = [&](int kt) {
        unsigned char* st = smem + (kt & 1) * PSTAGE;
        static_assert(PRB == 2, "the wait below names both registers");
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(breg[0]), "+v"(breg[1]) : "n"(PRA) : "memory");
#pragma unroll
        for (int i = 0; i < PRB; ++i) {
            u32x4 lo, hi;
            widen16(breg[i], lo, hi);
            *reinterpret_cast<u32x4*>(st + b_dst[i][0]) = lo;
            *reinterpret_cast<u32x4*>(st + b_dst[i][1]) = hi;
        }
    };

    const int frow = lane & 15, fk = lane >> 4;
    const int sw = (frow >> 1) & 7;
    const int ta = PARTIAL ? min(PTM, max(0, (p.rows - wm * 16 * PTM + 15) >> 4)) : PTM;
    const int a_off = (wm * 16 * PTM + frow) * PROW;
    const int b_off = PBM * PROW + (wn * 16 * PTN + frow) * PROW;

    f32x4 part[PTM][PTN];
#pragma unroll
    for (int i = 0; i < PTM; ++i)
#pragma unroll
        for (int j = 0; j < PTN; ++j) {
            acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            part[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        }

    // The scales are read-only for the whole launch: scalar loads through the constant address space, issued a k block
    // ahead of their use.
    typedef const __attribute__((address_space(4))) float cfloat;
    cfloat* sc0 = (cfloat*)(uintptr_t)p.s[0];
    cfloat* sc1 = (cfloat*)(uintptr_t)p.s[1];

    // one k half (32) of a slab: fragments from LDS, PTM x PTN MFMAs into the partial sums.  (Holding both halves'
    // fragments at once does not fit beside the two accumulator sets in the 256 registers of a wavefront.)
    auto half_slab = [&](const unsigned char* st, int s, bool from_zero) {
        const int c = ((s * 4 + fk) ^ sw) << 4;
        bf16x8 af[PTM], bf[PTN];
#pragma unroll
        for (int j = 0; j < PTN; ++j) bf[j] = *reinterpret_cast<const bf16x8*>(st + b_off + j * 16 * PROW + c);
#pragma unroll
        for (int i = 0; i < PTM; ++i)
            if (!PARTIAL || i < ta) af[i] = *reinterpret_cast<const bf16x8*>(st + a_off + i * 16 * PROW + c);
#pragma unroll
        for (int i = 0; i < PTM; ++i) {
            if (PARTIAL && i >= ta) continue;
#pragma unroll
            for (int j = 0; j < PTN; ++j)
                part[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[j], af[i],
                                                                     from_zero ? f32x4{0.f, 0.f, 0.f, 0.f} : part[i][j], 0, 0, 0);
        }
    };
    // The workgroup barrier without the fences of __syncthreads(): a workgroup-scope release would make the compiler
    // wait for every outstanding vector memory operation, the weight bytes in flight for a later slab included.  The
    // waits that matter are spelled out in front of it.
    auto barrier = [&]() {
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // Slab kt sits in stage kt & 1 and the other stage is free (every wavefront is past the barrier that ended slab
    // kt - 1).  The token rows of slab kt + 1 are requested first; with the MFMAs of the first k half the weight bytes
    // of slab kt + 1 (fetched during slab kt - 1) are widened and written beside them, and the bytes of slab kt + 2 take
    // their place in the registers.
    // parity_c: kt & 1; next_c / next2_c: slabs kt + 1 and kt + 2 exist -- constants, so that the steady-state slab is one
    // basic block (the last k block is peeled off).
    auto slab = [&](int kt, auto parity_c, auto next_c, auto next2_c) {
        constexpr int PAR = decltype(parity_c)::value;
        constexpr bool NEXT = decltype(next_c)::value, NEXT2 = decltype(next2_c)::value;
        const unsigned char* st = smem + PAR * PSTAGE;
        if (NEXT) issue_a(kt + 1);
        __builtin_amdgcn_sched_barrier(0);
        half_slab(st, 0, PAR == 0);            // a k block starts at an even slab: its first MFMAs start from zero
        if (NEXT) store_b(kt + 1);
        if (NEXT2) fetch_b(kt + 2);
        __builtin_amdgcn_sched_barrier(0);
        half_slab(st, 1, false);
    };
    auto end_slab = [&](auto next2_c) {
        // token rows of slab kt + 1 landed (loads return in issue order; only the weight bytes of slab kt + 2, requested
        // behind them, may still be in flight), this wavefront's LDS writes and reads done
        if (decltype(next2_c)::value) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(PRB) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        barrier();
    };
    auto fold = [&](float s0, float s1) {
#pragma unroll
        for (int i = 0; i < PTM; ++i)
#pragma unroll
            for (int j = 0; j < PTN; ++j) {
                const float sc = j < PTN / 2 ? s0 : s1;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = __builtin_fmaf(sc, part[i][j][r], acc[i][j][r]);
            }
    };
    typedef std::integral_constant<int, 0> Even;
    typedef std::integral_constant<int, 1> Odd;

    __syncthreads();                        // the previous task may still be reading the stages
    fetch_b(0);
    issue_a(0);
    store_b(0);
    fetch_b(1);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(PRB) : "memory");
    barrier();
    const int KB = p.K >> 7;
    int kb = 0;
    for (; kb < KB - 1; ++kb) {
        const float s0 = sc0[kb], s1 = sc1[kb];
        slab(2 * kb, Even{}, std::true_type{}, std::true_type{});
        end_slab(std::true_type{});
        slab(2 * kb + 1, Odd{}, std::true_type{}, std::true_type{});
        fold(s0, s1);
        end_slab(std::true_type{});
    }
    const float s0 = sc0[kb], s1 = sc1[kb];
    slab(2 * kb, Even{}, std::true_type{}, std::false_type{});
    end_slab(std::false_type{});
    slab(2 * kb + 1, Odd{}, std::false_type{}, std::false_type{});
    fold(s0, s1);
    end_slab(std::false_type{});
}

// ---- the same tile with both operands e4m3: v_mfma_f32_16x16x128_f8f6f4 ----
//
// One matrix instruction takes a whole 128-wide k block (32 bytes of each operand per lane), twice the rate of the 16-bit
// instructions, and nothing is widened: token rows arrive as e4m3 codes with one fp32 scale per (row, k block)
// (quant_rows128 passes in front of the two projections), weights are fed as stored.  A slab is one k block: 128 bytes
// per row, both operands global -> LDS directly, the 16-bit tiles' row layout (128-byte rows, 16-byte chunks xor-swizzled
// by (row >> 1) & 7); a lane's fragment is chunks fk and 4 + fk of its row -- the two chunks the 16-bit tiles read, a
// pattern without LDS bank conflicts; with chunks 2 fk and 2 fk + 1 every second cycle of the reads was one (which k a
// lane's bytes stand for inside the instruction does not matter as long as both operands agree: the block's dot product
// is a sum over all of them).
// Every MFMA starts from zero; its 16 x 16 partial sums are scaled by (weight block scale) x (token row scale) and added
// in fp32: y[t, n] = sum over k blocks of s_w[n / 128][kb] * s_a[t][kb] * (dot product of the block's codes).
typedef int i32x8 __attribute__((ext_vector_type(8)));

template <bool PARTIAL>
__device__ __forceinline__ void tile_mainloop_mfma8(const TileTask& p, unsigned char* smem, f32x4 (&acc)[PTM][PTN]) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int KB = p.K >> 7;

    // both operands: 8 threads per 128-byte row, four passes of 32 rows; LDS slot (row, c) holds chunk c ^ ((row >> 1) & 7)
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ ((prow >> 1) & 7);
    const uint8_t* a_src[4];
    const uint8_t* b_src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int r = prow + i * 32;
        if (r >= p.rows) r = 0;                                   // padding rows re-read row 0; never stored
        const int64_t src_row = p.gather ? (int64_t)p.gather[r] : p.a_row0 + r;
        a_src[i] = p.aq + src_row * p.K + chunk * 16;
        const int j = prow + i * 32;                              // row of the weight tile
        const uint8_t* base = p.w[0];
        int col;
        if (p.paired) {       // wavefront column w owns tile rows [64 w, 64 w + 64): 32 gate rows, then 32 up rows
            const int w = j >> 6, jj = j & 63;
            col = p.c0 + w * 32 + (jj & 31);
            base = (jj >> 5) ? p.w[1] : p.w[0];
        } else {
            col = p.c0 + j;
        }
        b_src[i] = base + (int64_t)col * p.K + chunk * 16;
    }
    const int wrow = __builtin_amdgcn_readfirstlane(prow & ~7);
    // The scales of the slab's token rows travel like the slab, global -> LDS, one float per row (wavefronts 0 and 1: a row
    // per lane).  As register loads they sat between the slab's requests in the memory counter, and the wait the compiler
    // puts in front of their use waited for the next slab's requests as well: no request was in flight during a slab's
    // MFMAs (MFMA pipes busy 24 % of the time).
    float* const ssc = reinterpret_cast<float*>(smem + 2 * PSTAGE);        // [stage][PBM]
    const float* sc_src = nullptr;
    if (wave < 2) {
        int r = tid;
        if (r >= p.rows) r = 0;
        const int64_t src_row = p.gather ? (int64_t)p.gather[r] : p.a_row0 + r;
        sc_src = p.sa + src_row * KB;
    }
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto issue = [&](int kb) {
        unsigned char* sa = smem + (kb & 1) * PSTAGE;
        unsigned char* sb = sa + PBM * PROW;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(a_src[i] + kb * 128), (lds_void*)(sa + (wrow + i * 32) * PROW), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_global_load_lds((gbl_void*)(b_src[i] + kb * 128), (lds_void*)(sb + (wrow + i * 32) * PROW), 16, 0, 0);
        if (wave_u < 2)
            __builtin_amdgcn_global_load_lds((gbl_void*)(sc_src + kb), (lds_void*)(ssc + (kb & 1) * PBM + wave_u * 64), 4, 0, 0);
    };

    const int frow = lane & 15, fk = lane >> 4;
    const int sw = (frow >> 1) & 7;
    const int ta = PARTIAL ? min(PTM, max(0, (p.rows - wm * 16 * PTM + 15) >> 4)) : PTM;
    const int a_off = (wm * 16 * PTM + frow) * PROW;
    const int b_off = PBM * PROW + (wn * 16 * PTN + frow) * PROW;
    const int c0 = (fk ^ sw) << 4, c1 = ((4 + fk) ^ sw) << 4;

    const int sc_off = wm * 16 * PTM + frow;          // this lane's token rows (one per 16 x 16 fragment) in a stage's scales
    typedef const __attribute__((address_space(4))) float cfloat;
    cfloat* sc0 = (cfloat*)(uintptr_t)p.s[0];
    cfloat* sc1 = (cfloat*)(uintptr_t)p.s[1];

#pragma unroll
    for (int i = 0; i < PTM; ++i)
#pragma unroll
        for (int j = 0; j < PTN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto frag = [&](const unsigned char* base) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(base + c0), hi = *reinterpret_cast<const u32x4*>(base + c1);
        return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    };

    __syncthreads();                        // the previous task may still be reading the stages
    issue(0);
    for (int kb = 0; kb < KB; ++kb) {
        // slab kb has landed (it was requested a whole slab ago, and nothing younger is outstanding that we could let
        // fly: wait for all), and every wavefront is done reading the other stage
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (kb + 1 < KB) issue(kb + 1);
        float sac[PTM];
#pragma unroll
        for (int i = 0; i < PTM; ++i) sac[i] = ssc[(kb & 1) * PBM + sc_off + i * 16];
        const float s0 = sc0[kb], s1 = sc1[kb];
        const unsigned char* st = smem + (kb & 1) * PSTAGE;
        i32x8 bf[PTN];
#pragma unroll
        for (int j = 0; j < PTN; ++j) bf[j] = frag(st + b_off + j * 16 * PROW);
#pragma unroll
        for (int i = 0; i < PTM; ++i) {
            if (PARTIAL && i >= ta) continue;
            const i32x8 af = frag(st + a_off + i * 16 * PROW);
            const float m0 = s0 * sac[i], m1 = s1 * sac[i];
#pragma unroll
            for (int j = 0; j < PTN; ++j) {
                const f32x4 part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], af, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                const float m = j < PTN / 2 ? m0 : m1;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = __builtin_fmaf(m, part[r], acc[i][j][r]);
            }
        }
    }
}

// acc[i][j][r]: token row = 64 wm + 16 i + (lane & 15); weight row inside fragment j = 4 (lane >> 4) + r.
__device__ __forceinline__ void tile_epilogue(const TileTask& p, f32x4 (&acc)[PTM][PTN]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 15, fk = lane >> 4;
#pragma unroll
    for (int i = 0; i < PTM; ++i) {
        const int m = wm * 16 * PTM + i * 16 + frow;
        if (m >= p.rows) continue;
        uint16_t* crow = p.c_base + (int64_t)m * p.N;
        if (p.paired) {
#pragma unroll
            for (int j = 0; j < PTN / 2; ++j) {
                const int col = p.c0 + wn * 32 + j * 16 + 4 * fk;
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float g = acc[i][j][r], u = acc[i][j + PTN / 2][r];
                    if (p.bias[0]) g = g + bf16_bits_to_f32(p.bias[0][col + r]);
                    if (p.bias[1]) u = u + bf16_bits_to_f32(p.bias[1][col + r]);
                    o[r] = silu(g) * u;
                }
                const uint32_t lo = pack2_bf16(o[0], o[1]), hi = pack2_bf16(o[2], o[3]);
                if (p.publish) publish8(crow + col, lo, hi);
                else *reinterpret_cast<uint2*>(crow + col) = uint2{lo, hi};
            }
        } else {
#pragma unroll
            for (int j = 0; j < PTN; ++j) {
                const int col = p.c0 + wn * 64 + j * 16 + 4 * fk;
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    o[r] = acc[i][j][r];
                    if (p.bias[0]) o[r] = o[r] + bf16_bits_to_f32(p.bias[0][col + r]);
                    o[r] = act_apply(o[r], p.act);
                }
                const uint32_t lo = pack2_bf16(o[0], o[1]), hi = pack2_bf16(o[2], o[3]);
                if (p.publish) publish8(crow + col, lo, hi);
                else *reinterpret_cast<uint2*>(crow + col) = uint2{lo, hi};
            }
        }
    }
}

__device__ __forceinline__ void fp8_gemm_tile(const TileTask& p, unsigned char* smem) {
    f32x4 acc[PTM][PTN];
    if (p.rows < PBM) tile_mainloop<true>(p, smem, acc);
    else tile_mainloop<false>(p, smem, acc);
    tile_epilogue(p, acc);
}
__device__ __forceinline__ void fp8_gemm_tile_mfma8(const TileTask& p, unsigned char* smem) {
    f32x4 acc[PTM][PTN];
    if (p.rows < PBM) tile_mainloop_mfma8<true>(p, smem, acc);
    else tile_mainloop_mfma8<false>(p, smem, acc);
    tile_epilogue(p, acc);
}

__device__ __forceinline__ TileTask resolve_tile(const FfnArgs& a, const Task& t, bool publish) {
    TileTask p;
    p.publish = publish;
    const int64_t HI = (int64_t)a.H * a.I;
    const int kbH = a.H >> 7, kbI = a.I >> 7;
    p.phase = t.phase;
    p.rows = t.rows;
    p.act = MOE_ACT_NONE;
    p.aq = t.phase == 0 ? a.xq : a.hq;
    p.sa = t.phase == 0 ? a.sx : a.sh;
    p.paired = t.phase == 0 && a.act == MOE_ACT_SWIGLU;
    if (t.phase == 0) {
        p.c0 = t.ntile * (p.paired ? PN0 : PN1);
        p.K = a.H;
        p.N = a.I;
        const int64_t srow = ((int64_t)t.expert * kbI + (p.c0 >> 7)) * kbH;
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
        p.c0 = t.ntile * PN1;
        p.K = a.I;
        p.N = a.H;
        p.w[0] = p.w[1] = (const uint8_t*)a.w_down + t.expert * HI;
        const int64_t srow = ((int64_t)t.expert * kbH + (p.c0 >> 7)) * kbI;
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

__global__ __launch_bounds__(PTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void ffn_tiled_fp8_tile_kernel(FfnArgs a, int phase) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_list[1 + PBM];
    if (phase == 0) zero_unrouted_rows(a, 2);
    Task t;
    if (!tiled_task(a, phase, blockIdx.x, t)) return;
    const TileTask p = resolve_tile(a, t, phase == 1 && a.arrive);
    fp8_gemm_tile(p, smem);
    if (phase == 1 && a.arrive) combine_arrivals<bf16_s>(combine_args(a), t.row0, t.rows, t.ntile, p.c0, PN1, s_list);
}

__global__ __launch_bounds__(PTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void ffn_persistent_fp8_tile_kernel(FfnArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_task, s_ok;
    __shared__ int s_cmb[kCombineLds];
    __shared__ int s_list[1 + PBM];
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
        const TileTask p = resolve_tile(a, t, t.phase == 0 || publish_y(a));
        const long long started = trace_clock(a.task_trace);
        if (ok) fp8_gemm_tile(p, smem);
        else poison_tile(p.c_base, p.rows, p.N, p.c0, PN1, 2);
        if (a.task_trace) trace_task(a.task_trace, a.task_trace_cap, t.phase, t.expert, t.mtile, t.ntile, t.rows, started);
        if (t.phase == 0) signal_phase0_done(a.done0, t.mtile);
        else after_down_tile<bf16_s>(a, t.row0, t.rows, t.mtile, t.ntile, p.c0, PN1, s_list);
    }
    if (a.combined) combine_while_idle_narrow<bf16_s>(sweep_args(a), &s_task, s_cmb);
    queue_clock_stamp(a.wg_clock, 1);
}

// The e4m3 x e4m3 plan: one launch per projection (the intermediate rows are quantised by a pass of their own between
// the two, so the projections cannot share a queue).
__global__ __launch_bounds__(PTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void ffn_tiled_fp8_mfma_kernel(FfnArgs a, int phase) {
    extern __shared__ __align__(16) unsigned char smem[];
    Task t;
    if (!tiled_task(a, phase, blockIdx.x, t)) return;
    const TileTask p = resolve_tile(a, t, false);
    fp8_gemm_tile_mfma8(p, smem);
}

template <class K>
hipError_t allow_lds(K kernel) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, PLDS);
}

}  // namespace

int fp8_tile_block_m() { return PBM; }
int fp8_tile_block_n0(int swiglu) { return swiglu ? PN0 : PN1; }
int fp8_tile_block_n1() { return PN1; }

int ffn_persistent_occupancy_fp8_tile() {
    int n = 0;
    if (allow_lds(&ffn_persistent_fp8_tile_kernel) != hipSuccess) return 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(&ffn_persistent_fp8_tile_kernel),
                                                     PTHREADS, PLDS) != hipSuccess || n < 1)
        n = 1;
    return n;
}

hipError_t launch_ffn_fp8_tile(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, int blocks, hipStream_t st) {
    if (blocks > 0) {
        hipError_t e = allow_lds(&ffn_persistent_fp8_tile_kernel);
        if (e != hipSuccess) return e;
        ffn_persistent_fp8_tile_kernel<<<blocks, PTHREADS, PLDS, st>>>(a);
    } else {
        hipError_t e = allow_lds(&ffn_tiled_fp8_tile_kernel);
        if (e != hipSuccess) return e;
        ffn_tiled_fp8_tile_kernel<<<tiled_grid(max_mtiles, nnt0, a.groups), PTHREADS, PLDS, st>>>(a, 0);
        ffn_tiled_fp8_tile_kernel<<<tiled_grid(max_mtiles, nnt1, a.groups), PTHREADS, PLDS, st>>>(a, 1);
    }
    return hipGetLastError();
}

// x -> e4m3 rows, up projection, h -> e4m3 rows (the kept ones), down projection.
hipError_t launch_ffn_fp8_mfma(const FfnArgs& a, int S, int64_t A, int max_mtiles, int nnt0, int nnt1, hipStream_t st) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&ffn_tiled_fp8_mfma_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, PLDS_M8);
    if (e != hipSuccess) return e;
    e = launch_quant_rows128(a.x, a.xq, a.sx, S, a.H, nullptr, st);
    if (e != hipSuccess) return e;
    ffn_tiled_fp8_mfma_kernel<<<tiled_grid(max_mtiles, nnt0, a.groups), PTHREADS, PLDS_M8, st>>>(a, 0);
    e = launch_quant_rows128(a.h, a.hq, a.sh, A, a.I, &a.q->kept_rows, st);
    if (e != hipSuccess) return e;
    ffn_tiled_fp8_mfma_kernel<<<tiled_grid(max_mtiles, nnt1, a.groups), PTHREADS, PLDS_M8, st>>>(a, 1);
    return hipGetLastError();
}

}  // namespace moe355
