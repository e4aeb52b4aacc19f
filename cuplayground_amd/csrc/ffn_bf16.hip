// Expert FFN on bf16 MFMA: the tile GEMM "processor" of the reference, rebuilt for gfx950.
//
// Contract kept from the reference (mma.cuh:46-179, processor/tiling.cuh:273-323): C = act(A.B^T + bias)
// with A (M,K) and B (N,K) row-major, fp32 accumulation, one cast to the storage type on store, epilogue
// order add-then-activate (processor/tiling.cuh:29-38).  Everything else is designed for CDNA4:
//   * v_mfma_f32_16x16x32_bf16; the weight tile is the MFMA "A" operand and the token tile the "B" operand,
//     so each lane ends up with 4 consecutive output columns of one token row (SwiGLU pairs stay in-lane);
//   * K slabs of 64 bf16 go from global memory straight into LDS (buffer_load ... lds, no VGPR staging)
//     as 128-byte rows whose 16-byte chunks are xor-swizzled with (row >> 1) & 7: the LDS has 64 banks, a
//     ds_read_b128 is served 16 lanes at a time, and with this swizzle 16 consecutive rows of one logical
//     chunk fall into 16 distinct bank groups;
//   * two LDS stages; MFMA operand fragments are double buffered in registers;
//   * dispatch is fused into the A-tile load: phase 0 gathers token rows through token_indices[];
//   * SwiGLU pairs gate and up columns inside one wavefront (first half of its tile rows from w_gate, second
//     half from w_up), so silu(g)*u happens in registers.
// Two plans.  "Large": 256-row blocks, 256 x 256 tiles for both projections, four wavefronts of 128 x 128 with the
// slab loop ordered by hand (gemm_tile_ring) and an epilogue staged through LDS; chosen when experts see many rows
// and every tile of the layer meets that loop's conditions (large_tile_ok).  "Small": 128 x 128 tiles, four
// wavefronts of 64 x 64, compiler-scheduled loop (mainloop_generic), general epilogue; takes everything else.
#include <type_traits>

#include "ffn_common.hpp"
#include "act_deriv.hpp"

namespace moe355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

constexpr int kBK = 64;               // bf16 elements of K per slab = one 128-byte LDS row
constexpr int kRowBytes = kBK * 2;

// F16: operands and results are IEEE binary16 (torch_dtype 3) instead of bfloat16; same tile, same loops, the other
// MFMA instruction and the other conversions.
template <int BM_, int BN_, int WM_, int WN_, int NS_, bool F16_ = false>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, NS = NS_;
    static constexpr bool F16 = F16_;
    static constexpr int THREADS = WM * WN * kWave;
    static constexpr int TM = BM / WM / 16;       // 16x16 MFMA tiles per wavefront along tokens
    static constexpr int TN = BN / WN / 16;       // ... along weight rows
    static constexpr int ROWS_PER_PASS = THREADS / 8;
    static constexpr int RA = BM / ROWS_PER_PASS; // 16-byte loads per thread per slab, token tile
    static constexpr int RB = BN / ROWS_PER_PASS; // ... weight tile
    static constexpr int STAGE_BYTES = (BM + BN) * kRowBytes;
    // four wavefronts of 128 x 128 outputs: this tile runs the hand-ordered slab loop (gemm_tile_ring)
    static constexpr bool RING = BM == 256 && BN == 256 && WM == 2 && WN == 2;
    // four wavefronts of 128 x 64 outputs, side by side (128 x 256) or two by two (256 x 128): the same loop with
    // half the weight fragments per wavefront
    static constexpr bool HALF = TM == 8 && TN == 4 && WM * WN == 4;
    static constexpr bool HAND = RING || HALF;
    static constexpr int WB = BN / WN;            // weight rows per wavefront
    // behind the stages: where the four wavefronts of a hand-ordered tile turn 16 rows of results at a time into
    // row-major order (row pitch: the wavefront's columns in bytes + 16)
    static constexpr int STAGING_BYTES = HAND ? 4 * 16 * (TN * 32 + 16) : 0;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + STAGING_BYTES;
    static_assert(TM >= 2 && TM % 2 == 0 && TN >= 2 && TN % 2 == 0, "a wavefront's tile is split in token halves; SwiGLU pairs weight-row halves");
    static_assert(RA >= 1 && RB >= 1, "tile too small for the workgroup");
    static_assert(NS == 2, "two LDS stages");
};

// What one task needs, resolved to pointers.
struct TaskPtrs {
    const uint16_t* a_base;      // phase 0: x; phase 1: h
    const int32_t* gather;       // phase 0: token_indices + row0; phase 1: null
    int64_t a_row0;              // phase 1: first row of h
    int a_ld;                    // K
    const uint16_t* b0;          // weight matrix of this expert (w_up or w_down)
    const uint16_t* b1;          // SwiGLU: w_gate of this expert, else null
    int b_ld;                    // elements between weight rows (K unless the operand is a window of a wider matrix)
    const uint16_t* bias0;
    const uint16_t* bias1;
    uint16_t* c_base;            // h or y, first row of the block
    int N;                       // output columns (I for phase 0, H for phase 1)
    int K;
    int rows;
    int n0;                      // first output column of this tile
    int act;                     // epilogue
    bool swiglu;
    bool publish;                // the rows will be read by other workgroups of the same launch
    uint32_t a_extent, b_extent; // bytes of the token operand (from a_base) and of one weight matrix (from b0 / b1)
    // A task that is one of `kparts` partial sums of its tile over the contraction dimension (null part: a whole tile):
    float* part;                 // the tile's partial-sum buffers, kparts x (block rows x block columns) fp32
    int32_t* part_cnt;           // parts of the tile stored so far
    int kparts, kpart;
    bool poison;                 // such a task whose rows never became ready: its part is NaN
    // The data gradient of the down projection with the activation's derivative in its epilogue (grouped kernel only;
    // deriv 0: an ordinary task): the tile's sums are dh, and what is stored is dh * act'(u) (and, for SwiGLU, the gate's
    // share beside it) from the saved projections u (and g), which have the output's shape.
    int deriv;                   // 0, or 1 + the layer's hidden_act
    const uint16_t* aux0;        // u rows, first row of the block
    const uint16_t* aux1;        // g rows (SwiGLU), else null
    uint16_t* c1_base;           // dg rows (SwiGLU), else null
};

// silu for a bf16 result: hardware exp2 and reciprocal (about 1 ulp each in fp32, far below the bf16 rounding of
// the product that follows) instead of the library expf and an IEEE division.
__device__ __forceinline__ float silu_fast(float g) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
}

// GELU (exact-erf form) for a bf16 result without the library erff, which costs some 40 instructions and two
// divergent branches per element: u * Phi(u) with erfc(x) = t (a1 + t (a2 + t (a3 + t (a4 + t a5)))) exp(-x^2),
// t = 1 / (1 + p x), x = |u| / sqrt 2 (Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7 on erfc).  The error of the
// result stays below 5e-7 in absolute terms and below one bf16 unit in the last place for |u| < 6.
__device__ __forceinline__ float gelu_fast(float u) {
    const float x = fabsf(u) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, x, 1.0f));
    float q = fmaf(1.061405429f, t, -1.453152027f);
    q = fmaf(q, t, 1.421413741f);
    q = fmaf(q, t, -0.284496736f);
    q = fmaf(q, t, 0.254829592f);
    const float half_erfc = 0.5f * q * t * __builtin_amdgcn_exp2f(x * x * -1.4426950408889634f);
    return u * (u >= 0.0f ? 1.0f - half_erfc : half_erfc);
}

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// Two fp32 values rounded to the tile's 16-bit storage type (nearest even), and one stored value widened.
template <class T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    if constexpr (T::F16) {
        typedef float f32x2_t __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
        const f32x2_t v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
    } else {
        return pack2_bf16(lo, hi);
    }
}
template <class T>
__device__ __forceinline__ float widen1(uint16_t v) {
    if constexpr (T::F16) return (float)__builtin_bit_cast(_Float16, v);
    else return bf16_bits_to_f32(v);
}

// 8 bytes of output; rows that another workgroup of the same launch will read are published (ffn_common.hpp).
__device__ __forceinline__ void store8(uint16_t* p, uint32_t lo, uint32_t hi, bool publish) {
    if (publish) {
        publish8(p, lo, hi);
    } else {
        u32x2 o = {lo, hi};
        *reinterpret_cast<u32x2*>(p) = o;
    }
}

// PARTIAL: the row block holds fewer than BM rows; 16-row MFMA sub-tiles that lie entirely in the padding are
// skipped (their LDS reads too).  A separate instantiation keeps the full-tile loop free of branches.
//
// Loop structure.  A 64-wide slab is consumed in four units (k half s, token half h) of HM x TN MFMAs; the
// fragments of the next unit are read from LDS under the MFMAs of the current one.  The one barrier per slab sits
// before the last unit: by then every wavefront has read all of the slab's fragments, so the barrier both frees
// this stage for the loads of slab kt+2 (issued right behind it) and publishes slab kt+1, whose first fragments
// are read under the last unit's MFMAs.  The first and the last two slabs are peeled off so that the steady-state
// loop is one basic block, which is what lets the scheduling hints hold.
template <class T, bool PARTIAL>
__device__ __forceinline__ void mainloop_generic(const TaskPtrs& p, unsigned char* smem, f32x4 (&acc)[T::TM][T::TN]) {
    constexpr int BM = T::BM, BN = T::BN, TM = T::TM, TN = T::TN, HM = TM / 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / T::WN, wn = wave % T::WN;
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ ((prow >> 1) & 7);   // LDS slot (row, c) holds global chunk c ^ ((row >> 1) & 7)

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
        b_src[i] = base + (int64_t)col * p.b_ld + chunk * 8;
    }

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

    // One global_load_lds_dwordx4 per 8 rows and wavefront writes 1 KiB of consecutive LDS: lane l lands in
    // row (l >> 3), chunk slot (l & 7); the swizzle is applied on the global side (see `chunk`).
    const int wrow = __builtin_amdgcn_readfirstlane(prow & ~7);
    const int KT = p.K / kBK;
    auto issue = [&](int kt) {
        unsigned char* sa = smem + (kt & 1) * T::STAGE_BYTES;
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
    __syncthreads();                        // the previous task may still be reading the stages
    issue(0);
    if (KT > 1) issue(1);

    const int frow = lane & 15, fk = lane >> 4;
    const int sw = (frow >> 1) & 7;
    // 16-row sub-tiles of this wavefront that contain at least one real row (wavefront-uniform)
    const int ta = PARTIAL ? min(TM, max(0, (p.rows - wm * 16 * TM + 15) >> 4)) : TM;
    const int a_base = (wm * 16 * TM + frow) * kRowBytes;
    const int b_base = BM * kRowBytes + (wn * 16 * TN + frow) * kRowBytes;

    bf16x8 af[2][HM], bfr[2][TN];
    auto read_a = [&](const unsigned char* st, int s, int h, int buf) {
        const int c = ((s * 4 + fk) ^ sw) << 4;
#pragma unroll
        for (int i = 0; i < HM; ++i)
            if (!PARTIAL || h * HM + i < ta)
                af[buf][i] = *reinterpret_cast<const bf16x8*>(st + a_base + (h * HM + i) * 16 * kRowBytes + c);
    };
    auto read_b = [&](const unsigned char* st, int s, int buf) {
        const int c = ((s * 4 + fk) ^ sw) << 4;
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[buf][j] = *reinterpret_cast<const bf16x8*>(st + b_base + j * 16 * kRowBytes + c);
    };
    auto mfmas = [&](int h, int abuf, int bbuf) {
#pragma unroll
        for (int i = 0; i < HM; ++i) {
            if (PARTIAL && h * HM + i >= ta) continue;
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[h * HM + i][j] =
                    T::F16 ? __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, bfr[bbuf][j]),
                                                                      __builtin_bit_cast(f16x8, af[abuf][i]), acc[h * HM + i][j], 0, 0, 0)
                           : __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[bbuf][j], af[abuf][i], acc[h * HM + i][j], 0, 0, 0);
        }
    };
    // instruction order inside a unit: behind every second MFMA one LDS read and (last unit) one global load
    auto hints = [&](auto nds_c, auto nvm_c) {
        constexpr int nds = decltype(nds_c)::value, nvm = decltype(nvm_c)::value;
        if (PARTIAL) return;
        constexpr int npair = nds > nvm ? nds : nvm;
        constexpr int NM = HM * TN;
#pragma unroll
        for (int n = 0; n < npair; ++n) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            if (n < nds) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (n < nvm) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        if (NM > 2 * npair) __builtin_amdgcn_sched_group_barrier(0x008, NM - 2 * npair, 0);
    };
    constexpr int NLOADS = T::RA + T::RB;
    typedef std::integral_constant<int, 0> Zero;

    // slab 0 has landed when at most the loads of slab 1 are outstanding (loads return in issue order)
    if (KT > 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLOADS) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read_a(smem, 0, 0, 0);
    read_b(smem, 0, 0);
    auto slab = [&](auto more_c, auto pre2_c, int kt) {
        constexpr bool MORE = decltype(more_c)::value, PRE2 = decltype(pre2_c)::value;
        const unsigned char* st = smem + (kt & 1) * T::STAGE_BYTES;
        const unsigned char* sn = smem + ((kt + 1) & 1) * T::STAGE_BYTES;
        read_a(st, 0, 1, 1);
        mfmas(0, 0, 0);
        hints(std::integral_constant<int, HM>{}, Zero{});
        read_a(st, 1, 0, 0);
        read_b(st, 1, 1);
        mfmas(1, 1, 0);
        hints(std::integral_constant<int, HM + TN>{}, Zero{});
        read_a(st, 1, 1, 1);
        mfmas(0, 0, 1);
        hints(std::integral_constant<int, HM>{}, Zero{});
        // every fragment of slab kt is in registers; this wavefront's share of slab kt+1 has landed
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        if (MORE) {
            read_a(sn, 0, 0, 0);
            read_b(sn, 0, 0);
        }
        if (PRE2) issue(kt + 2);
        mfmas(1, 1, 1);
        hints(std::integral_constant<int, MORE ? HM + TN : 0>{}, std::integral_constant<int, PRE2 ? NLOADS : 0>{});
    };
    int kt = 0;
    for (; kt < KT - 2; ++kt) slab(std::true_type{}, std::true_type{}, kt);
    if (KT > 1) {
        slab(std::true_type{}, std::false_type{}, kt);
        ++kt;
    }
    slab(std::false_type{}, std::false_type{}, kt);
}

// acc[i][j][r]: token row = wm*16*TM + i*16 + (lane & 15); weight row inside the 16-wide MFMA tile = 4*(lane >> 4) + r.
// MODE: 0 none / ReLU, 2 GELU (erf form), 3 SwiGLU.  The choice is made once per tile so that the unrolled store loop
// does not branch around the (large) GELU code for every element.
template <class T, int MODE>
__device__ __forceinline__ void epilogue_impl(const TaskPtrs& p, f32x4 (&acc)[T::TM][T::TN]) {
    constexpr int TM = T::TM, TN = T::TN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / T::WN, wn = wave % T::WN;
    const int frow = lane & 15, fk = lane >> 4;
    // MODE 0: u below the floor becomes the floor.  Written as a compare and select, not as fmaxf: a max returns its
    // other operand for a NaN, and a NaN must stay a NaN (the reference's __hfma_relu propagates it too, processor/tiling.cuh:45,54)
    const float relu_floor = p.act == MOE_ACT_RELU ? 0.0f : -INFINITY;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = wm * 16 * TM + i * 16 + frow;
        if (m >= p.rows) continue;
        uint16_t* crow = p.c_base + (int64_t)m * p.N;
        if constexpr (MODE == 3) {
#pragma unroll
            for (int j = 0; j < TN / 2; ++j) {
                const int col = p.n0 + wn * 8 * TN + j * 16 + 4 * fk;
                if (col >= p.N) continue;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float g = acc[i][j][r], u = acc[i][j + TN / 2][r];
                    if (p.bias1) g = g + widen1<T>(p.bias1[col + r]);
                    if (p.bias0) u = u + widen1<T>(p.bias0[col + r]);
                    v[r] = silu_fast(g) * u;
                }
                store8(crow + col, pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]), p.publish);
            }
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = p.n0 + wn * 16 * TN + j * 16 + 4 * fk;
                if (col >= p.N) continue;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float u = acc[i][j][r];
                    if (p.bias0) u = u + widen1<T>(p.bias0[col + r]);
                    v[r] = MODE == 2 ? gelu_fast(u) : (u < relu_floor ? relu_floor : u);
                }
                store8(crow + col, pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]), p.publish);
            }
        }
    }
}

template <class T>
__device__ __forceinline__ void epilogue(const TaskPtrs& p, f32x4 (&acc)[T::TM][T::TN]) {
    if (p.swiglu) epilogue_impl<T, 3>(p, acc);
    else if (p.act == MOE_ACT_GELU) epilogue_impl<T, 2>(p, acc);
    else epilogue_impl<T, 0>(p, acc);
}

// The epilogue of a tile that is not ragged in N (rows may be), staged through LDS.
//
// In the accumulator layout the 16 lanes that are neighbours in the wavefront hold 16 different rows, so a store
// straight from the registers writes 64 separate 8-byte pieces per instruction.  Each wavefront therefore writes its
// bf16 results, 16 rows at a time, into its own piece of LDS behind the slab stages and reads them back row-major:
// 16 bytes per lane, a whole row of the wavefront's columns per 16 (8 for SwiGLU) neighbouring lanes, four (eight)
// rows per store instruction.  No barrier is involved (same wavefront, LDS operations complete in order), and the
// slab stages stay free: the loads of the workgroup's next task may already be landing in them.  The row pitch is
// padded by 16 bytes, which puts the 8-byte writes of 32 neighbouring lanes on distinct banks.  The bias values of
// this lane's columns are loaded once (or are -0.0f, the neutral element of the addition), so the element loop has
// no branch.
// A store of more than 8 bytes reads its data registers over the cycles behind its issue, and an instruction that
// writes one of them must keep two wait states' distance.  The compiler sees to that for the stores it emits, not for one
// inside an asm statement -- it may well put the next value into the same registers right behind it -- so the statement
// brings the wait states along.
#define MOE_STORE16_AGENT "global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1"
__device__ __forceinline__ void store16(uint16_t* p, u32x4 v, bool publish) {
    if (publish) asm volatile(MOE_STORE16_AGENT ::"v"(p), "v"(v) : "memory");   // agent scope, as publish8
    else *reinterpret_cast<u32x4*>(p) = v;
}

struct NoHook {
    __device__ __forceinline__ void operator()(int) const {}
};
// The epilogue of a tile that was computed as KP partial sums (partial_tile_arrive): `base` is this lane's place in the
// partial-sum buffers of the tile (two parts: in the other part's buffer; four parts: in the buffer of part 0).
struct WholeTile {
    static constexpr int KP = 1;
};
template <int KP_>
struct SummedTile {
    static constexpr int KP = KP_;
    const float* base;
};

// `between(i)` runs in front of row group i (i = 0..7): the queue kernel issues the next task's first loads there, a
// few at a time, so that they leave the compute unit under the epilogue's arithmetic instead of in front of it.
// DERIV: what leaves the staging area is not stored as it is (dh, rounded to 16 bits as a stored data gradient would be)
// but multiplied by the activation's derivative at the saved projections (TaskPtrs::deriv): a row segment's 8 values
// meet the 8 values of u (and g) of the same rows and columns, loaded at the top of the row group.
template <class T, int MODE, class Hook, class Parts = WholeTile, bool DERIV = false>
__device__ __forceinline__ void epilogue_full_n_impl(const TaskPtrs& p, unsigned char* smem, f32x4 (&acc)[8][T::TN], const Hook& between,
                                                     const Parts& parts = Parts()) {
    static_assert(Parts::KP == 1 || MODE == 0, "partial sums: the down projection only");
    static_assert(!DERIV || (MODE == 0 && Parts::KP == 1), "the derivative follows a plain product");

    static_assert(T::HAND, "four wavefronts of 128 x 128 or 128 x 64");
    constexpr int NJ = MODE == 3 ? T::TN / 2 : T::TN;   // groups of 16 output columns per wavefront
    constexpr int ROW_BYTES = NJ * 32, PITCH = ROW_BYTES + 16;
    constexpr int LANES_PER_ROW = ROW_BYTES / 16, ROWS_PER_PASS = 64 / LANES_PER_ROW;
    static_assert(4 * 16 * PITCH <= T::STAGING_BYTES, "the staging pieces of the four wavefronts fit behind the slab stages");
    // Everything below is derived from a thread id the compiler cannot see through: otherwise it computes these
    // addresses before the slab loop, finds no register to keep them in, and reloads them from scratch memory
    // between the stores (each reload then waits for the store before it).
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / T::WN, wn = wave % T::WN;
    const int frow = lane & 15, fk = lane >> 4;
    const int col0 = p.n0 + wn * 16 * NJ;        // first output column of this wavefront
    float b0[NJ][4], b1[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) b0[j][r] = b1[j][r] = -0.0f;
    if (p.bias0) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) b0[j][r] = widen1<T>(p.bias0[col0 + 16 * j + 4 * fk + r]);
    }
    if (MODE == 3 && p.bias1) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) b1[j][r] = widen1<T>(p.bias1[col0 + 16 * j + 4 * fk + r]);
    }
    // MODE 0: u below the floor becomes the floor.  Written as a compare and select, not as fmaxf: a max returns its
    // other operand for a NaN, and a NaN must stay a NaN (the reference's __hfma_relu propagates it too, processor/tiling.cuh:45,54)
    const float relu_floor = p.act == MOE_ACT_RELU ? 0.0f : -INFINITY;
    unsigned char* stage = smem + T::NS * T::STAGE_BYTES + wave * (16 * PITCH);
    unsigned char* wr = stage + frow * PITCH + fk * 8;
    const int rd_row = lane / LANES_PER_ROW, rd_chunk = lane % LANES_PER_ROW;
    const unsigned char* rd = stage + rd_row * PITCH + rd_chunk * 16;
    const int rows_left = p.rows - wm * 128 - rd_row;                 // this lane stores row r0 + rd_row when r0 < rows_left
    const uint32_t lane_off = (uint32_t)(rd_row * p.N + col0 + rd_chunk * 8);   // elements from the uniform row pointer
    const bool publish = p.publish;
    constexpr int NQ = 16 / ROWS_PER_PASS;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        between(i);
        // (DERIV) the saved projections of this row group's rows: requested here, used behind the staging round trip
        u32x4 uu[DERIV ? NQ : 1], gg[DERIV ? NQ : 1];
        if constexpr (DERIV) {
            const int64_t group = (int64_t)(wm * 128 + i * 16) * p.N;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                uu[q] = gg[q] = u32x4{0u, 0u, 0u, 0u};
                if (i * 16 + q * ROWS_PER_PASS < rows_left) {
                    const int64_t at = group + (int64_t)(q * ROWS_PER_PASS) * p.N + lane_off;
                    uu[q] = *reinterpret_cast<const u32x4*>(p.aux0 + at);
                    if (p.deriv == 1 + MOE_ACT_SWIGLU) gg[q] = *reinterpret_cast<const u32x4*>(p.aux1 + at);
                }
            }
        }
        // Partial sums: the row group's sums of the other parts come back from memory (written through by their tasks,
        // read past this XCD's L2) and are added here -- two parts: own registers + the other part, which is the same
        // in either order; four parts: all four as stored, in the order of the parts, whichever of them runs this.
        f32x4 whole[Parts::KP == 1 ? 1 : NJ];
        if constexpr (Parts::KP == 2) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(whole[j]) : "v"(parts.base + (i * NJ + j) * 256) : "memory");
#pragma unroll
            for (int j = 0; j < NJ; ++j) asm volatile("s_waitcnt vmcnt(0)" : "+v"(whole[j])::"memory");
#pragma unroll
            for (int j = 0; j < NJ; ++j) whole[j] = acc[i][j] + whole[j];
        } else if constexpr (Parts::KP == 4) {
            constexpr size_t kPartFloats = (size_t)T::BM * T::BN;
#pragma unroll
            for (int j0 = 0; j0 < NJ; j0 += 4) {
                f32x4 v[4][4];
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[k][j]) : "v"(parts.base + k * kPartFloats + (i * NJ + j0 + j) * 256) : "memory");
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int j = 0; j < 4; ++j) asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[k][j])::"memory");
#pragma unroll
                for (int j = 0; j < 4; ++j) whole[j0 + j] = ((v[0][j] + v[1][j]) + v[2][j]) + v[3][j];
            }
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if constexpr (MODE == 3) {
                    const float g = acc[i][j][r] + b1[j][r], u = acc[i][j + NJ][r] + b0[j][r];
                    v[r] = silu_fast(g) * u;
                } else {
                    float sum;
                    if constexpr (Parts::KP == 1) sum = acc[i][j][r]; else sum = whole[j][r];
                    const float u = sum + b0[j][r];
                    v[r] = MODE == 2 ? gelu_fast(u) : (u < relu_floor ? relu_floor : u);
                }
            }
            u32x2 o = {pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3])};
            *reinterpret_cast<u32x2*>(wr + j * 32) = o;
        }
        u32x4 v[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) v[q] = *reinterpret_cast<const u32x4*>(rd + q * ROWS_PER_PASS * PITCH);
        uint16_t* rows0 = p.c_base + (int64_t)(wm * 128 + i * 16) * p.N;   // uniform
        if constexpr (DERIV) {
            const int64_t group = (int64_t)(wm * 128 + i * 16) * p.N;
            const bool gated = p.deriv == 1 + MOE_ACT_SWIGLU;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                if (i * 16 + q * ROWS_PER_PASS >= rows_left) continue;
                const int64_t at = group + (int64_t)(q * ROWS_PER_PASS) * p.N + lane_off;
                u32x4 o0, o1 = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float d0 = widen1<T>((uint16_t)(v[q][w] & 0xFFFFu)), d1 = widen1<T>((uint16_t)(v[q][w] >> 16));
                    const float u0 = widen1<T>((uint16_t)(uu[q][w] & 0xFFFFu)), u1 = widen1<T>((uint16_t)(uu[q][w] >> 16));
                    float a0, a1, b0v = 0.0f, b1v = 0.0f;
                    if (gated) {
                        const float g0 = widen1<T>((uint16_t)(gg[q][w] & 0xFFFFu)), g1 = widen1<T>((uint16_t)(gg[q][w] >> 16));
                        dswiglu16(d0, u0, g0, a0, b0v);
                        dswiglu16(d1, u1, g1, a1, b1v);
                    } else if (p.deriv == 1 + MOE_ACT_GELU) {
                        a0 = dgelu16(d0, u0);
                        a1 = dgelu16(d1, u1);
                    } else {
                        a0 = drelu16(d0, u0);
                        a1 = drelu16(d1, u1);
                    }
                    o0[w] = pack2<T>(a0, a1);
                    o1[w] = pack2<T>(b0v, b1v);
                }
                store16(p.c_base + at, o0, false);
                if (gated) store16(p.c1_base + at, o1, false);
            }
            continue;
        }
        if (publish) {
#pragma unroll
            for (int q = 0; q < NQ; ++q)
                if (i * 16 + q * ROWS_PER_PASS < rows_left)
                    store16(rows0 + (int64_t)(q * ROWS_PER_PASS) * p.N + lane_off, v[q], true);
        } else {
#pragma unroll
            for (int q = 0; q < NQ; ++q)
                if (i * 16 + q * ROWS_PER_PASS < rows_left)
                    store16(rows0 + (int64_t)(q * ROWS_PER_PASS) * p.N + lane_off, v[q], false);
        }
    }
}

template <class T, class Hook = NoHook>
__device__ __forceinline__ void epilogue_full_n(const TaskPtrs& p, unsigned char* smem, f32x4 (&acc)[8][T::TN], const Hook& between = Hook()) {
    if (p.swiglu) epilogue_full_n_impl<T, 3>(p, smem, acc, between);
    else if (p.act == MOE_ACT_GELU) epilogue_full_n_impl<T, 2>(p, smem, acc, between);
    else epilogue_full_n_impl<T, 0>(p, smem, acc, between);
}

// The slab loop of a full 256 x 256 tile on four wavefronts of 128 x 128, with the instruction order fixed by hand.
//
// Why not the compiler's order: with one wavefront per SIMD nothing else hides a stall, and the global->LDS loads of
// a slab (64 KB per compute unit) need more than one slab of flight time to stream in at the rate the L2 delivers.
// So (a) both k halves of a slab's fragments are double buffered in registers, which frees the slab's LDS stage at
// mid-slab, (b) the loads of slab kt+2 are issued into that stage right away, two per MFMA row, and stay in flight
// across the barriers (bare s_barrier: a __syncthreads() would wait for them), (c) MFMAs, LDS reads and their
// s_waitcnt are inline asm in the order written by gen_slab_schedule.py (ffn_bf16_slab_steady.inc); the compiler places
// nothing between them but the scalar address updates of the loads.  The accumulators are tied asm operands in
// AGPRs, so they stay put for the whole loop.  Loads use buffer addressing: a 32-bit byte offset per row, computed
// once per task, plus a scalar k offset -- no vector ALU instruction is left in the loop.
// Takes partial row blocks too (the whole tile is computed, rows past the end are not stored).
// Needs: K a multiple of 128, a tile that is not ragged in N, operand extents below 4 GiB.
// What the loads of one task of the hand-ordered tile need; computed once per task (ring_prepare).
struct RingLoads {
    unsigned voff_a[8], voff_b[8];   // byte offsets of this thread's eight token rows / weight rows (row + 16-byte chunk)
    const void* base_a;              // wavefront-uniform operand bases
    const void* base_b0;
    const void* base_b1;
    uint32_t a_extent, b_extent;
    int KT;                          // slabs of 64: even, >= 2
    int wrow;                        // first of the eight consecutive stage rows this wavefront's loads fill per pass
};

// The part of a task's load state that needs no memory access: weight-row offsets, bases, extents.
template <class T>
__device__ __forceinline__ RingLoads ring_prepare_weights(const TaskPtrs& p) {
    static_assert(T::HAND && T::ROWS_PER_PASS == 32, "four wavefronts of 128 x 128 or 128 x 64");
    // a thread id the compiler cannot see through: what is derived from it is computed here, not once at the top of
    // the kernel and then kept (and spilled) across the slab loop
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ ((prow >> 1) & 7);
    RingLoads L;
#pragma unroll
    for (int n = 0; n < 8; ++n) L.voff_a[n] = L.voff_b[n] = p.a_extent;
#pragma unroll
    for (int n = 0; n < T::RB; ++n) {
        // SwiGLU: a wavefront's weight rows are the gate rows of its output columns followed by their up rows
        const int j = prow + n * T::ROWS_PER_PASS;
        const int col = p.swiglu ? p.n0 + (j / T::WB) * (T::WB / 2) + (j % (T::WB / 2)) : p.n0 + j;
        L.voff_b[n] = (unsigned)(((int64_t)col * p.b_ld + chunk * 8) * 2);
    }
    auto uniform = [](const void* q) {          // the bases are the same in every lane; say so, or each load loops over lanes
        const uint64_t v = (uint64_t)q;
        // readfirstlane returns int: go through uint32_t, or a low half with bit 31 set sign-extends over the high half
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        return (const void*)(((uint64_t)hi << 32) | (uint64_t)lo);
    };
    L.base_a = uniform(p.a_base);
    L.base_b0 = uniform(p.b0);
    L.base_b1 = uniform(p.swiglu ? p.b1 : p.b0);
    L.a_extent = p.a_extent;
    L.b_extent = p.b_extent;
    L.KT = p.K / kBK;
    L.wrow = __builtin_amdgcn_readfirstlane(prow & ~7);
    return L;
}

// The token-row offsets: phase 0 gathers the row numbers through token_indices[] (eight loads per thread).
template <class T>
__device__ __forceinline__ void ring_prepare_tokens(const TaskPtrs& p, RingLoads& L) {
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int prow = tid >> 3;
    const int chunk = (tid & 7) ^ ((prow >> 1) & 7);
#pragma unroll
    for (int n = 0; n < T::RA; ++n) {
        // Padding rows are never stored.  Their loads are aimed behind the end of the buffer, which the hardware
        // answers with zeros without touching memory: MFMAs on zeros draw less of the power budget than MFMAs on a
        // copy of real rows.
        const int r0 = prow + n * T::ROWS_PER_PASS, r = max(min(r0, p.rows - 1), 0);
        const int64_t src_row = p.gather ? (int64_t)p.gather[r] : p.a_row0 + r;
        L.voff_a[n] = r0 < p.rows ? (unsigned)((src_row * p.a_ld + chunk * 8) * 2) : p.a_extent;
    }
}

template <class T>
__device__ __forceinline__ RingLoads ring_prepare(const TaskPtrs& p) {
    RingLoads L = ring_prepare_weights<T>(p);
    ring_prepare_tokens<T>(p, L);
    return L;
}

// Load n of slab `slab` of a task: n < RA token rows, else weight rows; the weight rows of pass m come from w_gate when
// they lie in the first half of a wavefront's weight rows.  Raw buffers (stride 0) that end where the operand ends.  Slabs past the end of K go through descriptors of
// zero length, which the hardware answers with zeros without touching memory (the stages they land in are never read).
template <class T>
__device__ __forceinline__ void ring_load_one(const RingLoads& L, unsigned char* smem, int slab, int n) {
    const int wrow = L.wrow;
    unsigned char* base = smem + (slab & 1) * T::STAGE_BYTES;
    const int soff = slab * kRowBytes;
    const bool live = slab < L.KT;
    if (n < T::RA) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(L.base_a), 0, live ? (int)L.a_extent : 0, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(base + (wrow + n * T::ROWS_PER_PASS) * kRowBytes), 16,
                                                 L.voff_a[n], soff, 0, 0);
    } else {
        const int m = n - T::RA;
        const bool up_rows = (m * T::ROWS_PER_PASS) % T::WB >= T::WB / 2;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(up_rows ? L.base_b0 : L.base_b1), 0,
                                                                             live ? (int)L.b_extent : 0, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(base + T::BM * kRowBytes + (wrow + m * T::ROWS_PER_PASS) * kRowBytes),
                                                 16, L.voff_b[m], soff, 0, 0);
    }
}

// The loads of a task's first two slabs: the weight rows of slab 0 and of slab 1, then the token rows of slab 0 and of
// slab 1 -- weights first because their addresses need no gathered row numbers, so the queue kernel can send them
// off while those are still on their way.  Slab 0 is complete when at most the last RA of them are outstanding.
// Nobody may still be reading the stages (the caller sees to that).
template <class T>
__device__ __forceinline__ void ring_first_weight_loads(const RingLoads& L, unsigned char* smem) {
#pragma unroll
    for (int n = T::RA; n < T::RA + T::RB; ++n) ring_load_one<T>(L, smem, 0, n);
#pragma unroll
    for (int n = T::RA; n < T::RA + T::RB; ++n) ring_load_one<T>(L, smem, 1, n);
}
template <class T>
__device__ __forceinline__ void ring_first_token_load(const RingLoads& L, unsigned char* smem, int q) {   // q = 0..2 RA - 1
    if (q < 2 * T::RA) ring_load_one<T>(L, smem, q / T::RA, q % T::RA);
}
template <class T>
__device__ __forceinline__ void ring_first_loads(const RingLoads& L, unsigned char* smem) {
    ring_first_weight_loads<T>(L, smem);
#pragma unroll
    for (int q = 0; q < 16; ++q) ring_first_token_load<T>(L, smem, q);
}

// The slab loop of a full 256 x 256 tile on four wavefronts of 128 x 128, with the instruction order fixed by hand.
//
// Why not the compiler's order: with one wavefront per SIMD nothing else hides a stall, and the global->LDS loads of
// a slab (64 KB per compute unit) need more than one slab of flight time to stream in at the rate the L2 delivers.
// So (a) both k halves of a slab's fragments are double buffered in registers, which frees the slab's LDS stage at
// mid-slab, (b) the loads of slab kt+2 are issued into that stage right away, two per MFMA row, and stay in flight
// across the barriers (bare s_barrier: a __syncthreads() would wait for them), (c) MFMAs, LDS reads and their
// s_waitcnt are inline asm in the order written by gen_slab_schedule.py (ffn_bf16_slab_steady.inc); the compiler places
// nothing between them but the scalar address updates of the loads.  The accumulators are tied asm operands in
// AGPRs, so they stay put for the whole loop.  Loads use buffer addressing: a 32-bit byte offset per row, computed
// once per task, plus a scalar k offset -- no vector ALU instruction is left in the loop.
// Takes partial row blocks too (the whole tile is computed, rows past the end are not stored).
// Needs: K a multiple of 128, a tile that is not ragged in N, operand extents below 4 GiB.
// On entry the loads of slabs 0 and 1 (ring_first_loads, in that order) are the 32 youngest vector loads of this
// wavefront (stores issued behind them only make the first wait more conservative).  Returns false for a wavefront whose 128 rows are all
// padding: it has taken part in the loads and barriers only and holds no results.
template <class T>
__device__ __forceinline__ bool ring_slabs(int rows, const RingLoads& L, unsigned char* smem, f32x4 (&acc)[8][T::TN]) {
    constexpr int BM = T::BM, STAGE = T::STAGE_BYTES, TN = T::TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / T::WN, wn = wave % T::WN;
    // The scalar members are the same in every lane; say so here, behind whatever control flow handed L over, or the
    // compiler builds every buffer descriptor in a loop over the lanes.
    RingLoads U = L;
    {
        auto uni = [](unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); };
        auto unip = [&](const void* q) {
            const uint64_t v = (uint64_t)q;
            return (const void*)(((uint64_t)uni((unsigned)(v >> 32)) << 32) | (uint64_t)uni((unsigned)v));
        };
        U.base_a = unip(L.base_a); U.base_b0 = unip(L.base_b0); U.base_b1 = unip(L.base_b1);
        U.a_extent = uni(L.a_extent); U.b_extent = uni(L.b_extent);
        U.KT = (int)uni((unsigned)L.KT); U.wrow = (int)uni((unsigned)L.wrow);
    }
    const int KT = U.KT;
    auto load_one = [&](int slab, int n) { ring_load_one<T>(U, smem, slab, n); };

#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    const int frow = lane & 15, fk = lane >> 4;
    const int sw = (frow >> 1) & 7;
    // LDS addresses of this lane's fragment rows: [stage][k half]
    // (the asm reads take raw LDS byte addresses: start from where the dynamic array really begins -- a kernel with
    // static __shared__ variables places it behind them)
    const unsigned lds0 = (unsigned)(__UINTPTR_TYPE__)(lds_void*)smem;
    const unsigned a_row = lds0 + (unsigned)((wm * 128 + frow) * kRowBytes), b_row = lds0 + (unsigned)(BM * kRowBytes + (wn * T::WB + frow) * kRowBytes);
    const unsigned c0 = (unsigned)((fk ^ sw) << 4), c1 = (unsigned)(((4 + fk) ^ sw) << 4);
    const unsigned la0[2] = {a_row + c0, a_row + c1}, lb0[2] = {b_row + c0, b_row + c1};
    const unsigned la1[2] = {la0[0] + STAGE, la0[1] + STAGE}, lb1[2] = {lb0[0] + STAGE, lb0[1] + STAGE};
    bf16x8 af[2][8], bfr[2][TN];
    int kt = 0;

#define MF(i, j, s)                                                                                                      \
    do {                                                                                                                 \
        if constexpr (T::F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(bfr[s][j]), "v"(af[s][i])); \
        else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(bfr[s][j]), "v"(af[s][i]));                  \
    } while (0)
#define RA(stg, half, idx) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[half][idx]) : "v"((stg) ? la1[half] : la0[half]), "n"((idx) * 16 * kRowBytes))
#define RB(stg, half, j) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(bfr[half][j]) : "v"((stg) ? lb1[half] : lb0[half]), "n"((j) * 16 * kRowBytes))
#define WL(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n))
#define BAR1 do { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); __builtin_amdgcn_s_barrier(); } while (0)
#define BAR2(n) do { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory"); __builtin_amdgcn_s_barrier(); } while (0)
#define GL(n) load_one(kt + 2, n)
#define TAIL asm volatile("s_nop 15\n\ts_nop 3" ::: "memory")
    // Padding rows.  The MFMA pipes run against the board's power limit, so an MFMA on padding rows costs everybody
    // clock.  A wavefront whose 128 rows are all padding (a row block of at most 128 rows: the upper two wavefronts)
    // therefore takes part in the loads and the barriers only: the same slab body with the MFMAs, the fragment reads
    // and their waits left out.  The tile takes as long as before; the layer gains 1 % (Mixtral shape) to 4 % (many
    // small experts) from the clock.  (Skipping the empty 16-row groups of partly filled wavefronts as well, with a
    // scalar branch around their MFMAs, cost more in the full tiles than it returned.)
    if (__builtin_amdgcn_readfirstlane(wm) * 128 >= rows) {
#pragma push_macro("MF")
#pragma push_macro("RA")
#pragma push_macro("RB")
#pragma push_macro("WL")
#undef MF
#undef RA
#undef RB
#undef WL
#define MF(i, j, s) ((void)0)
#define RA(stg, half, idx) ((void)0)
#define RB(stg, half, j) ((void)0)
#define WL(n) ((void)0)
        if constexpr (T::RA == 8) BAR2(8); else BAR2(4);
        for (; kt < KT; kt += 2) {
            {
                constexpr unsigned st = 0, sn = 1;
                (void)st; (void)sn;
                if constexpr (TN == 8) {
#include "ffn_bf16_slab_steady.inc"
                } else {
#include "ffn_bf16_slab_half.inc"
                }
            }
            ++kt;
            {
                constexpr unsigned st = 1, sn = 0;
                (void)st; (void)sn;
                if constexpr (TN == 8) {
#include "ffn_bf16_slab_steady.inc"
                } else {
#include "ffn_bf16_slab_half.inc"
                }
            }
            --kt;
        }
#pragma pop_macro("WL")
#pragma pop_macro("RB")
#pragma pop_macro("RA")
#pragma pop_macro("MF")
        return false;                           // nothing to store either
    }
    // slab 0 has landed (loads return in issue order; see ring_first_loads)
    if constexpr (T::RA == 8) BAR2(8); else BAR2(4);
    {   // same order as the reads behind BAR2 of a steady-state slab
        constexpr unsigned sn = 0;
        RA(sn, 0, 0);
        RB(sn, 0, 0); RB(sn, 0, 1); RB(sn, 0, 2); RB(sn, 0, 3);
        if constexpr (TN == 8) { RB(sn, 0, 4); RB(sn, 0, 5); RB(sn, 0, 6); RB(sn, 0, 7); }
        RA(sn, 0, 1); RA(sn, 0, 2); RA(sn, 0, 3); RA(sn, 0, 4); RA(sn, 0, 5); RA(sn, 0, 6); RA(sn, 0, 7);
    }
    // Every slab runs the same body, the last two included: their loads (of slabs KT and KT+1) fetch nothing and
    // land in stages nobody reads any more.  Separate tail bodies would be shorter, but between them the compiler is
    // free to spill or copy an accumulator right behind the asm MFMA that writes it, and it does not know that the
    // value is still in flight.
    for (; kt < KT; kt += 2) {
        {
            constexpr unsigned st = 0, sn = 1;
                if constexpr (TN == 8) {
#include "ffn_bf16_slab_steady.inc"
                } else {
#include "ffn_bf16_slab_half.inc"
                }
        }
        ++kt;
        {
            constexpr unsigned st = 1, sn = 0;
                if constexpr (TN == 8) {
#include "ffn_bf16_slab_steady.inc"
                } else {
#include "ffn_bf16_slab_half.inc"
                }
        }
        --kt;
    }
    // (the TAIL of the last slab also covers the first read of an accumulator behind the loop)
    // The last slab body has read fragments of a slab past the end.  Nobody uses them, so for the compiler their
    // registers are free from here on -- but the reads are still in flight.  Wait for them, and keep the registers
    // occupied until behind that wait.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" ::"v"(af[h][i]));
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" ::"v"(bfr[h][j]));
    }
#undef MF
#undef RA
#undef RB
#undef WL
#undef BAR1
#undef BAR2
#undef GL
#undef TAIL
    return true;
}

// A tile computed as kparts partial sums over the contraction dimension, one task each (the down-projection tiles at the
// end of the task queue: the tasks every workgroup ends its launch with, made short).  Every part stores its fp32
// accumulators (written through: the parts run on any compute unit of the chip), then adds one to the tile's counter;
// the part that finds all the others there runs the epilogue, which adds the parts up in an order that does not depend
// on which part that is (epilogue_full_n_impl), so the result depends on kparts only, never on the schedule.  Returns
// true in that workgroup; every wavefront of the workgroup calls it, `active` false for one whose rows are all padding (it
// keeps the barriers company).
// The buffer has the accumulator layout: [part][wavefront][register group i * TN + j][lane], 16 bytes each; tile_lane is
// this lane's place in part 0.
template <class T>
__device__ __forceinline__ bool partial_tile_arrive(const TaskPtrs& p, unsigned char* smem, f32x4 (&acc)[8][T::TN], bool active,
                                                    float* tile_lane) {
    constexpr int TN = T::TN;
    constexpr size_t kPartFloats = (size_t)T::BM * T::BN;
    static_assert((size_t)T::THREADS / 64 * 8 * TN * 64 * 4 == kPartFloats, "the accumulators of the workgroup are the tile");
    if (active) {
        float* mine = tile_lane + (size_t)p.kpart * kPartFloats;
        const float fill = __int_as_float(0x7FC00000);
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                // (a part whose rows never became ready stores NaN: that is what the tile then holds)
                const f32x4 v = p.poison ? f32x4{fill, fill, fill, fill} : acc[i][j];
                asm volatile(MOE_STORE16_AGENT ::"v"(mine + (i * TN + j) * 256), "v"(v) : "memory");
            }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wavefront's part has reached memory
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    int* s_before = reinterpret_cast<int*>(smem + T::NS * T::STAGE_BYTES);    // the staging area is idle until the epilogue
    __syncthreads();
    if (threadIdx.x == 0) *s_before = __hip_atomic_fetch_add(p.part_cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int before = __builtin_amdgcn_readfirstlane(*s_before);
    __syncthreads();                                      // the word may be overwritten from here on
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    return before == p.kparts - 1;
}

// A task that is a part of a tile, behind its slab loop.
template <class T>
__device__ __forceinline__ void partial_tile_finish(const TaskPtrs& p, unsigned char* smem, f32x4 (&acc)[8][T::TN], bool active) {
    constexpr size_t kPartFloats = (size_t)T::BM * T::BN;
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = tid >> 6;
    float* tile_lane = p.part + ((size_t)wave * 8 * T::TN * 64 + lane) * 4;
    if (!partial_tile_arrive<T>(p, smem, acc, active, tile_lane) || !active) return;
    if (p.kparts == 2) {
        const SummedTile<2> parts{tile_lane + (size_t)(1 - p.kpart) * kPartFloats};
        epilogue_full_n_impl<T, 0>(p, smem, acc, NoHook(), parts);
    } else {
        const SummedTile<4> parts{tile_lane};
        epilogue_full_n_impl<T, 0>(p, smem, acc, NoHook(), parts);
    }
}

// One task from start to end: the form the two-launch and the plain-GEMM kernels use.
template <class T>
__device__ __forceinline__ void gemm_tile_ring(const TaskPtrs& p, unsigned char* smem) {
    const RingLoads L = ring_prepare<T>(p);
    __syncthreads();                            // the previous task may still be reading the stages
    ring_first_loads<T>(L, smem);
    f32x4 acc[8][T::TN];
    if (ring_slabs<T>(p.rows, L, smem, acc)) epilogue_full_n<T>(p, smem, acc);
}
// The same with the activation's derivative behind the product (TaskPtrs::deriv; the grouped kernel of the backward pass).
template <class T>
__device__ __forceinline__ void gemm_tile_ring_deriv(const TaskPtrs& p, unsigned char* smem) {
    const RingLoads L = ring_prepare<T>(p);
    __syncthreads();
    ring_first_loads<T>(L, smem);
    f32x4 acc[8][T::TN];
    if (ring_slabs<T>(p.rows, L, smem, acc)) epilogue_full_n_impl<T, 0, NoHook, WholeTile, true>(p, smem, acc, NoHook());
}
// The same for a task that is a part of a tile (TaskPtrs::part).  A copy of its own, slab loop included: with both ends
// behind one loop the compiler reads all accumulators in front of the branch between them and spills what does not fit,
// which costs the whole tiles -- nearly all of them -- 4 to 13 % of their time.
template <class T>
__device__ __forceinline__ void gemm_tile_ring_part(const TaskPtrs& p, unsigned char* smem) {
    const RingLoads L = ring_prepare<T>(p);
    __syncthreads();
    ring_first_loads<T>(L, smem);
    f32x4 acc[8][T::TN];
    const bool active = ring_slabs<T>(p.rows, L, smem, acc);
    partial_tile_finish<T>(p, smem, acc, active);
}

template <class T, bool PARTIAL>
__device__ __forceinline__ void gemm_tile_generic(const TaskPtrs& p, unsigned char* smem) {
    f32x4 acc[T::TM][T::TN];
    mainloop_generic<T, PARTIAL>(p, smem, acc);
    epilogue<T>(p, acc);
}

// The 256 x 256 tile only exists with the hand-ordered slab loop; the host selects it when every task of the launch
// meets that loop's conditions (large_tile_ok) and falls back to the 128 x 128 tile otherwise.
template <class T>
__device__ __forceinline__ void gemm_tile(const TaskPtrs& p, unsigned char* smem) {
    if constexpr (T::HAND) {
        gemm_tile_ring<T>(p, smem);
    } else {
        if (p.rows >= T::BM) gemm_tile_generic<T, false>(p, smem);
        else gemm_tile_generic<T, true>(p, smem);
    }
}

template <class T>
__device__ __forceinline__ TaskPtrs resolve(const FfnArgs& a, const Task& t, bool publish) {
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
        p.b_ld = a.H;
        p.n0 = t.ntile * (sw ? T::BN / 2 : T::BN);
        p.act = a.act;
        p.swiglu = sw;
        p.publish = publish;
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
        p.b_ld = a.I;
        p.n0 = t.ntile * T::BN;
        p.act = MOE_ACT_NONE;
        p.swiglu = false;
        p.publish = publish;
    }
    p.rows = t.rows;
    p.a_extent = t.phase == 0 ? a.x_bytes : a.h_bytes;
    p.b_extent = a.w_bytes;
    p.part = nullptr;
    p.part_cnt = nullptr;
    p.kparts = 1;
    p.kpart = 0;
    p.poison = false;
    p.deriv = 0;
    p.aux0 = nullptr;
    p.aux1 = nullptr;
    p.c1_base = nullptr;
    if (t.phase == 1 && t.kparts > 1) {       // one of kparts partial sums: this part's share of the intermediate dimension
        const int Kp = a.I / t.kparts, k0 = t.kpart * Kp;
        p.K = Kp;
        p.a_base += k0;
        p.b0 += k0;
        p.a_extent -= (uint32_t)k0 * 2;       // the descriptors start where the operands now start
        p.b_extent -= (uint32_t)k0 * 2;
        const int tile = (t.mtile - a.q->split_mt0) * a.nnt1 + t.ntile;
        p.part = a.split_part + (size_t)tile * t.kparts * ((size_t)T::BM * T::BN);
        p.part_cnt = a.split_cnt + tile;
        p.kparts = t.kparts;
        p.kpart = t.kpart;
        p.poison = t.poison;
    }
    return p;
}

// A plan pairs the tile of the up(/gate) projection with the tile of the down projection; both use the
// same row-block height and the same workgroup size.
//
// TS (optional): the tile that takes the row blocks of at most TS::BM rows -- the ragged last block of an expert --
// in place of T0 / T1.  It covers the same columns per task, so the task tables do not change; it only does not
// spend a full tile's MFMAs on rows that are mostly padding.
template <class T0_, class T1_, class TS_ = void>
struct Plan {
    using T0 = T0_;
    using T1 = T1_;
    using TS = TS_;
    static constexpr bool MIXED = !std::is_void<TS_>::value;
    static_assert(T0::BM == T1::BM && T0::THREADS == T1::THREADS, "phases share row blocks and workgroup size");
    static constexpr int THREADS = T0::THREADS;
    static constexpr int LDS_BYTES = T0::LDS_BYTES > T1::LDS_BYTES ? T0::LDS_BYTES : T1::LDS_BYTES;
};
using Tile256 = Tile<256, 256, 2, 2, 2>;
using Tile128x256 = Tile<128, 256, 1, 4, 2>;     // hand-ordered, four wavefronts of 128 x 64 side by side
using Tile256H = Tile<256, 256, 2, 2, 2, true>;  // fp16
using Tile128x256H = Tile<128, 256, 1, 4, 2, true>;
using LargePlan = Plan<Tile256, Tile256>;
using MixedPlan = Plan<Tile256, Tile256, Tile128x256>;
using MediumPlan = Plan<Tile128x256, Tile128x256>;
using SmallPlan = Plan<Tile<128, 128, 2, 2, 2>, Tile<128, 128, 2, 2, 2>>;
using LargePlanH = Plan<Tile256H, Tile256H>;
using MixedPlanH = Plan<Tile256H, Tile256H, Tile128x256H>;
using MediumPlanH = Plan<Tile128x256H, Tile128x256H>;
using SmallPlanH = Plan<Tile<128, 128, 2, 2, 2, true>, Tile<128, 128, 2, 2, 2, true>>;

// One task of a plan: the plan's tile, or its small-row-block tile when the block has few enough rows.
// SPLIT: the task may be a part of a tile (kernels of their own: the code for it costs the others 1-2 % in short tasks).
template <class P, bool SPLIT = false>
__device__ __forceinline__ void plan_tile(const FfnArgs& a, const Task& t, bool publish, unsigned char* smem) {
    static_assert(std::is_same<typename P::T0, typename P::T1>::value, "one tile for both projections: one inlined copy");
    const TaskPtrs p = resolve<typename P::T0>(a, t, publish);
    if constexpr (P::MIXED) {
        static_assert(P::TS::BN == P::T0::BN && P::TS::LDS_BYTES <= P::LDS_BYTES, "same columns per task");
        if (t.rows <= P::TS::BM) {
            if constexpr (SPLIT && P::TS::HAND) {
                if (p.part) {
                    gemm_tile_ring_part<typename P::TS>(p, smem);
                    return;
                }
            }
            gemm_tile<typename P::TS>(p, smem);
            return;
        }
    }
    if constexpr (SPLIT && P::T0::HAND) {
        if (p.part) {
            gemm_tile_ring_part<typename P::T0>(p, smem);
            return;
        }
    }
    gemm_tile<typename P::T0>(p, smem);
}

// One launch per phase; workgroup b runs task b of that phase.
template <class P, bool SPLIT = false>
__global__ __launch_bounds__(P::THREADS) void ffn_tiled_kernel(FfnArgs a, int phase) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_list[1 + P::T0::BM];
    using ET = typename std::conditional<P::T0::F16, f16_s, bf16_s>::type;
    if (phase == 0) zero_unrouted_rows(a, 2);
    Task t;
    if (!tiled_task(a, phase, blockIdx.x, t)) return;
    plan_tile<P, SPLIT>(a, t, phase == 1 && a.arrive, smem);   // rows another workgroup may combine go out write-through
    if (phase == 1 && a.arrive) combine_arrivals<ET>(combine_args(a), t.row0, t.rows, t.ntile, t.ntile * P::T1::BN, P::T1::BN, s_list);
}

// The kernel's argument block, read again from the kernel-argument segment through a pointer the compiler cannot see
// through: values loaded from it live only as long as they are used, instead of occupying forty scalar registers
// across the slab loop (which then spill into vector registers and bring vector instructions into the loop).
__device__ __forceinline__ const FfnArgs& kernel_args_again() {
    typedef const __attribute__((address_space(4))) FfnArgs* args_ptr;
    args_ptr q = (args_ptr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(q));
    return *(const FfnArgs*)q;
}

// Persistent workgroups popping (expert, tile) tasks from the queue of their XCD (protocol: ffn_common.hpp).
template <class P, bool SPLIT = false>
__global__ __launch_bounds__(P::THREADS) void ffn_persistent_kernel(FfnArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_task, s_ok;
    __shared__ int s_list[1 + P::T0::BM];
    static_assert(1 + P::T0::BM >= kCombineLds, "s_list doubles as the scratch of the combine tasks");
    using ET = typename std::conditional<P::T0::F16, f16_s, bf16_s>::type;
    queue_kernel_entry();
    queue_clock_stamp(kernel_args_again().wg_clock, 0);
    zero_unrouted_rows(kernel_args_again(), 2);
    const int ids = a.q->ids_queue;
    const int nseg = a.q->nseg;
    const int nnt0 = a.seg_phase0[0].nnt;
    QueueCursor cur = queue_cursor(a.groups);
    Task t;
    while (next_task(a, cur, &s_task, ids, nseg, nnt0, t)) {   // uniform exit: every wavefront leaves together
        if (t.phase == 1 && !wait_phase0_done(a.done0, t.mtile, nnt0, a.spin_limit, a.q, a.host_stall, &s_ok)) {
            // the rows never became ready: NaN instead of a result, and a tile of no rows (it loads, computes and
            // stores nothing of its own), so that the loop keeps its one shape; a part of a tile keeps its shape too (the
            // parts must agree on it) and hands on NaN in place of its sums
            if (t.kparts > 1) {
                t.poison = true;
            } else {
                poison_tile((uint16_t*)a.y + (int64_t)t.row0 * a.H, t.rows, a.H, t.ntile * P::T1::BN, P::T1::BN, 2);
                t.rows = 0;
            }
        }
        const long long started = trace_clock(kernel_args_again().task_trace);
        plan_tile<P, SPLIT>(a, t, t.phase == 0 || publish_y(a), smem);
        if (kernel_args_again().task_trace)
            trace_task(kernel_args_again().task_trace, kernel_args_again().task_trace_cap, t.phase | (t.kparts > 1 ? (t.kpart << 2) | (t.kparts << 4) : 0), t.expert, t.mtile, t.ntile, t.rows, started);
        if (t.phase == 0) signal_phase0_done(a.done0, t.mtile);
        else                 // the row count from the table: a tile whose wait expired runs with none, and still arrives
            after_down_tile<ET>(kernel_args_again(), t.row0, a.mtiles[t.mtile].rows, t.mtile, t.ntile, t.ntile * P::T1::BN, P::T1::BN, s_list);
    }
    if (kernel_args_again().combined) combine_while_idle<ET>(sweep_args(kernel_args_again()), &s_task, s_list);
    queue_clock_stamp(kernel_args_again().wg_clock, 1);
}

// The same queue for the 256 x 256 tile, with the start of the next task moved under the end of the current one
// (opt-in: option queue_early = 1).
//
// Between two tiles a workgroup pops (an atomic round trip and two barriers), decodes, computes its row offsets (eight
// gathered token indices per thread), issues the first 32 loads and waits for slab 0.  Here the next id is reserved
// with an asynchronous pop when the current tile's slab loop begins (its latency disappears under the loop), and right
// behind the loop -- the LDS stages are free, the accumulators still hold the tile -- the next task is decoded, its
// dependency polled once, the weight rows of its first two slabs are requested, and the token rows follow two at a
// time between the row groups of the current tile's epilogue.  A next task that cannot start (dependency not yet
// met, queue exhausted, a hole) is handled after the epilogue the plain way; a workgroup never blocks while it holds
// unstored results, so the queue's progress argument is unchanged.  Near the end of its queue a workgroup stops
// reserving: a task reserved behind a long tile would start late while other workgroups idle.
// Measured with timestamps inside the kernel (Mixtral shape, per tile): the wait for slab 0 (about 4 us) is gone, but
// pop result + barrier 0.8, decode 1.2, offsets 1.2 and issuing the loads 1.4 us now sit in front of the epilogue, so
// the time between two slab loops stays at 12-13 us and the launch takes the same number of cycles (MFMA pipes busy
// 74 % either way); short tiles lose 2-3 %.  Results are bit-identical to the plain loop.
constexpr int kReserveMargin = 64;   // ids left in the current queue below which tasks are popped late again

template <class P>
__global__ __launch_bounds__(P::THREADS) void ffn_persistent_ring_kernel(FfnArgs) {
    using T = typename P::T0;
    static_assert(std::is_same<typename P::T0, typename P::T1>::value && T::RING, "the hand-ordered tile for both projections");
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int s_task, s_ok, s_next[2];
    __shared__ int s_list[1 + T::BM];
    using ET = typename std::conditional<T::F16, f16_s, bf16_s>::type;
    queue_kernel_entry();
    queue_clock_stamp(kernel_args_again().wg_clock, 0);
    zero_unrouted_rows(kernel_args_again(), 2);
    int ids, nseg, nnt0, groups;
    {
        const FfnArgs& a = kernel_args_again();
        ids = a.q->ids_queue;
        nseg = a.q->nseg;
        nnt0 = a.seg_phase0[0].nnt;
        groups = a.groups;
    }
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    QueueCursor cur = queue_cursor(groups);
    // The current task as plain scalars (a struct carried around the loop ends up in scratch memory).
    int ph = 0, ex = 0, mt = 0, nt = 0, row0 = 0, rows = 0;
    auto as_task = [&]() {
        Task q;
        q.phase = ph; q.expert = ex; q.mtile = mt; q.ntile = nt; q.row0 = row0; q.rows = rows; q.nnt0 = nnt0; q.valid = true;
        q.kparts = 1; q.kpart = 0; q.poison = false;     // (the host never asks for this loop and partial sums together)
        return q;
    };
    RingLoads L;
    // a task started the plain way: wait for its rows if need be, offsets, first loads
    auto start_cold = [&]() {
        const FfnArgs& a = kernel_args_again();
        if (ph == 1 && !wait_phase0_done(a.done0, mt, nnt0, a.spin_limit, a.q, a.host_stall, &s_ok)) {
            poison_tile((uint16_t*)a.y + (int64_t)row0 * a.H, rows, a.H, nt * T::BN, T::BN, 2);
            rows = 0;
        }
        L = ring_prepare<T>(resolve<T>(a, as_task(), ph == 0));
        __syncthreads();                        // the previous task may still be reading the stages
        ring_first_loads<T>(L, smem);
    };
    auto pop_blocking = [&]() {
        Task q;
        const bool ok = next_task(kernel_args_again(), cur, &s_task, ids, nseg, nnt0, q);
        if (ok) { ph = q.phase; ex = q.expert; mt = q.mtile; nt = q.ntile; row0 = q.row0; rows = q.rows; }
        return ok;
    };
    bool have = pop_blocking();
    if (have) start_cold();
    while (have) {                              // uniform: every wavefront takes the same turns
        const bool reserve = cur.last_id + kReserveMargin < ids;
        int rid = 0;
        if (reserve && wave == 0) rid = pop_async(&kernel_args_again().q->heads[cur.group]);
        const long long traced_from = trace_clock(kernel_args_again().task_trace);   // the first loads left earlier, under the previous tile's end
        f32x4 acc[8][8];
        const bool active = ring_slabs<T>(rows, L, smem, acc);

        const FfnArgs& a = kernel_args_again();
        int nid = ids, n_valid = 0, n_ph = 0, n_ex = 0, n_mt = 0, n_nt = 0, n_row0 = 0, n_rows = 0, started = 0;
        if (reserve) {
            if (wave == 0) s_next[0] = pop_async_result(rid);
            __syncthreads();                    // also: every wavefront is done with the stages
            nid = __builtin_amdgcn_readfirstlane(s_next[0]);
            if (nid < ids) {
                const Task q = decode_task(a.seg_queue, nseg, a.mtiles, nid, cur.group, groups, nnt0, a.row_chunk);
                n_valid = q.valid; n_ph = q.phase; n_ex = q.expert; n_mt = q.mtile; n_nt = q.ntile; n_row0 = q.row0; n_rows = q.rows;
                if (n_valid) {
                    int ready = 1;
                    if (n_ph == 1) {            // one look at the dependency; the answer must be the workgroup's, not a wavefront's
                        if (wave == 0)
                            s_next[1] = __hip_atomic_load(a.done0 + n_mt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= nnt0;
                        __syncthreads();
                        ready = __builtin_amdgcn_readfirstlane(s_next[1]);
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                    }
                    if (ready) {                // the loop is done with the old offsets
                        const TaskPtrs pq = resolve<T>(a, q, n_ph == 0);
                        L = ring_prepare_weights<T>(pq);
                        ring_first_weight_loads<T>(L, smem);
                        ring_prepare_tokens<T>(pq, L);
                        started = 1;
                    }
                }
            }
        }
        // the token rows of the next task's first slabs leave two at a time under the epilogue's arithmetic
        auto token_loads = [&](int i) {
            if (started) {
                ring_first_token_load<T>(L, smem, 2 * i);
                ring_first_token_load<T>(L, smem, 2 * i + 1);
            }
        };
        if (active) {
            epilogue_full_n<T>(resolve<T>(a, as_task(), ph == 0 || publish_y(a)), smem, acc, token_loads);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) token_loads(i);
        }
        if (a.task_trace) trace_task(a.task_trace, a.task_trace_cap, ph, ex, mt, nt, rows, traced_from);
        if (ph == 0) signal_phase0_done(a.done0, mt);
        else after_down_tile<ET>(a, row0, a.mtiles[mt].rows, mt, nt, nt * T::BN, T::BN, s_list);
        if (reserve && nid < ids && n_valid) {   // the reserved task is the next one
            ph = n_ph; ex = n_ex; mt = n_mt; nt = n_nt; row0 = n_row0; rows = n_rows;
            cur.last_id = nid;
            if (!started) start_cold();          // its rows were not ready: wait now that nothing unstored is held
            continue;
        }
        if (reserve && nid >= ids) {             // the reserved pop found this queue empty: move on as next_task does
            if (++cur.exhausted >= groups) break;
            cur.group = cur.group + 1 == groups ? 0 : cur.group + 1;
        }
        have = pop_blocking();
        if (have) start_cold();
    }
    if (kernel_args_again().combined) combine_while_idle<ET>(sweep_args(kernel_args_again()), &s_task, s_list);
    queue_clock_stamp(kernel_args_again().wg_clock, 1);
}

// The bare reference contract on dense operands: rows [b*BM, ...) of A, one "expert".
template <class T>
__global__ __launch_bounds__(T::THREADS) void gemm_dense_kernel(const uint16_t* A, const uint16_t* B,
                                                                const uint16_t* bias, uint16_t* C, int M, int N, int K,
                                                                int act) {
    extern __shared__ __align__(16) unsigned char smem[];
    TaskPtrs p;
    const int row0 = blockIdx.x * T::BM;      // row tiles fastest: neighbouring workgroups share the weight tile
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
    p.b_ld = K;
    p.rows = min(T::BM, M - row0);
    p.n0 = blockIdx.y * T::BN;
    p.act = act;
    p.swiglu = false;
    p.publish = false;
    p.a_extent = (uint32_t)((int64_t)M * K * 2);
    p.b_extent = (uint32_t)((int64_t)N * K * 2);
    p.part = nullptr; p.part_cnt = nullptr; p.kparts = 1; p.kpart = 0; p.poison = false;
    p.deriv = 0; p.aux0 = nullptr; p.aux1 = nullptr; p.c1_base = nullptr;
    gemm_tile<T>(p, smem);
}

// Grouped GEMM on packed expert-major rows, outside the layer: out[r,:] = act(a[r,:] . w[e(r)]^T + bias[e(r)]) for
// the rows of every row block of the table -- the reference's tile GEMM (mma.cuh:46-179) once per expert, with the
// expert taken from the row block.  With the weight handed over in its K-major view this is the data gradient of a
// projection (dX = dY . W).  One workgroup per tile, in the order of the layer's task queue: expert by expert, column
// tile by column tile, an expert's row blocks fastest -- neighbouring workgroups share a weight tile and an expert's
// few row blocks stay in the caches while its column tiles pass by (column tiles of all experts' row blocks at once:
// 1.69 ms on the Mixtral-shaped data gradient of the down projection against 1.55 this way).  grid = row blocks upper bound x column tiles;
// mtiles[i].pad is the index of the first row block of that block's expert.
template <class T>
__global__ __launch_bounds__(T::THREADS) void grouped_gemm_kernel(const uint16_t* a_rows, const uint16_t* w,
                                                                  const uint16_t* bias, uint16_t* out,
                                                                  const MTile* mtiles, const int32_t* num_mtiles,
                                                                  const int32_t* count, int N, int K, int act,
                                                                  uint32_t a_bytes) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int ncol = (N + T::BN - 1) / T::BN;
    const int id = blockIdx.x;
    if (id >= *num_mtiles * ncol) return;
    // id / ncol is a row block of the expert this id belongs to: ids [ncol * first, ncol * (first + blocks)) are its own
    const MTile probe = mtiles[id / ncol];
    const int first = probe.pad, blocks = (max(count[probe.expert], 0) + T::BM - 1) / T::BM;
    const int local = id - ncol * first, ctile = local / blocks;
    const MTile m = mtiles[first + (local - ctile * blocks)];
    TaskPtrs p;
    p.a_base = a_rows;
    p.gather = nullptr;
    p.a_row0 = m.row0;
    p.a_ld = K;
    p.b0 = w + (int64_t)m.expert * N * K;
    p.b1 = nullptr;
    p.b_ld = K;
    p.bias0 = bias ? bias + (int64_t)m.expert * N : nullptr;
    p.bias1 = nullptr;
    p.c_base = out + (int64_t)m.row0 * N;
    p.N = N;
    p.K = K;
    p.rows = m.rows;
    p.n0 = ctile * T::BN;
    p.act = act;
    p.swiglu = false;
    p.publish = false;
    p.a_extent = a_bytes;
    p.b_extent = (uint32_t)((int64_t)N * K * 2);
    p.part = nullptr; p.part_cnt = nullptr; p.kparts = 1; p.kpart = 0; p.poison = false;
    p.deriv = 0; p.aux0 = nullptr; p.aux1 = nullptr; p.c1_base = nullptr;
    gemm_tile<T>(p, smem);
}

// The grouped product with the activation's derivative in its epilogue (gemm_tile_ring_deriv): the data gradient of the
// down projection that hands on dU (and dG) instead of dH.  Same grid, same order of the tiles as grouped_gemm_kernel.
template <class T>
__global__ __launch_bounds__(T::THREADS) void grouped_gemm_deriv_kernel(const uint16_t* a_rows, const uint16_t* w,
                                                                        const uint16_t* u_rows, const uint16_t* g_rows,
                                                                        uint16_t* du_rows, uint16_t* dg_rows,
                                                                        const MTile* mtiles, const int32_t* num_mtiles,
                                                                        const int32_t* count, int N, int K, int hidden_act,
                                                                        uint32_t a_bytes) {
    static_assert(T::HAND, "the derivative lives in the epilogue of the hand-ordered tiles");
    extern __shared__ __align__(16) unsigned char smem[];
    const int ncol = (N + T::BN - 1) / T::BN;
    const int id = blockIdx.x;
    if (id >= *num_mtiles * ncol) return;
    const MTile probe = mtiles[id / ncol];
    const int first = probe.pad, blocks = (max(count[probe.expert], 0) + T::BM - 1) / T::BM;
    const int local = id - ncol * first, ctile = local / blocks;
    const MTile m = mtiles[first + (local - ctile * blocks)];
    TaskPtrs p;
    p.a_base = a_rows;
    p.gather = nullptr;
    p.a_row0 = m.row0;
    p.a_ld = K;
    p.b0 = w + (int64_t)m.expert * N * K;
    p.b1 = nullptr;
    p.b_ld = K;
    p.bias0 = nullptr;
    p.bias1 = nullptr;
    p.c_base = du_rows + (int64_t)m.row0 * N;
    p.N = N;
    p.K = K;
    p.rows = m.rows;
    p.n0 = ctile * T::BN;
    p.act = MOE_ACT_NONE;
    p.swiglu = false;
    p.publish = false;
    p.a_extent = a_bytes;
    p.b_extent = (uint32_t)((int64_t)N * K * 2);
    p.part = nullptr; p.part_cnt = nullptr; p.kparts = 1; p.kpart = 0; p.poison = false;
    p.deriv = 1 + hidden_act;
    p.aux0 = u_rows + (int64_t)m.row0 * N;
    p.aux1 = g_rows ? g_rows + (int64_t)m.row0 * N : nullptr;
    p.c1_base = dg_rows ? dg_rows + (int64_t)m.row0 * N : nullptr;
    gemm_tile_ring_deriv<T>(p, smem);
}


// Weight gradient of one projection: dw[e] [N, K] = dy_e^T . a_e, the sum running over the rows of expert e.  Both
// operands arrive transposed and padded: dyT [N, ld] and aT [K, ld] hold expert e's rows in columns
// [poff[e], poff[e+1]) (zeros behind the last real row; every window is a multiple of 128 wide), so each expert is one
// (M,K) x (N,K)^T tile GEMM over its window.  grid = (row tiles of N, column tiles of K, experts).
template <class T>
__global__ __launch_bounds__(T::THREADS) void wgrad_kernel(const uint16_t* dyT, const uint16_t* aT, uint16_t* dw,
                                                           const int32_t* poff, int N, int K, int ld, uint32_t dy_bytes,
                                                           uint32_t a_bytes) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int e = blockIdx.z;
    const int row0 = blockIdx.x * T::BM, n0 = blockIdx.y * T::BN;
    const int p0 = poff[e], window = poff[e + 1] - p0;
    uint16_t* c = dw + (int64_t)e * N * K + (int64_t)row0 * K;
    const int rows = min(T::BM, N - row0);
    if (window == 0) {   // an expert that received no rows: its gradient is zero
        for (int i = threadIdx.x; i < rows * T::BN; i += T::THREADS) {
            const int r = i / T::BN, col = n0 + i % T::BN;
            if (col < K) c[(int64_t)r * K + col] = 0;
        }
        return;
    }
    TaskPtrs p;
    p.a_base = dyT + p0;
    p.gather = nullptr;
    p.a_row0 = row0;
    p.a_ld = ld;
    p.b0 = aT + p0;
    p.b1 = nullptr;
    p.b_ld = ld;
    p.bias0 = nullptr;
    p.bias1 = nullptr;
    p.c_base = c;
    p.N = K;
    p.K = window;
    p.rows = rows;
    p.n0 = n0;
    p.act = MOE_ACT_NONE;
    p.swiglu = false;
    p.publish = false;
    p.a_extent = dy_bytes - (uint32_t)p0 * 2;
    p.b_extent = a_bytes - (uint32_t)p0 * 2;
    p.part = nullptr; p.part_cnt = nullptr; p.kparts = 1; p.kpart = 0; p.poison = false;
    p.deriv = 0; p.aux0 = nullptr; p.aux1 = nullptr; p.c1_base = nullptr;
    gemm_tile<T>(p, smem);
}

template <class K>
hipError_t allow_lds(K kernel, int bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               bytes);
}

template <class P>
hipError_t launch_tiled(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, hipStream_t st) {
    hipError_t e = allow_lds(&ffn_tiled_kernel<P>, P::LDS_BYTES);
    if (e != hipSuccess) return e;
    ffn_tiled_kernel<P><<<tiled_grid(max_mtiles, nnt0, a.groups), P::THREADS, P::LDS_BYTES, st>>>(a, 0);
    if constexpr (P::T0::HAND) {
        if (a.split_cnt) {      // row blocks whose tiles run as partial sums count once per part
            e = allow_lds(&ffn_tiled_kernel<P, true>, P::LDS_BYTES);
            if (e != hipSuccess) return e;
            ffn_tiled_kernel<P, true><<<tiled_grid(max_mtiles + a.split_extra_blocks, nnt1, a.groups), P::THREADS, P::LDS_BYTES, st>>>(a, 1);
            return hipGetLastError();
        }
    }
    ffn_tiled_kernel<P><<<tiled_grid(max_mtiles, nnt1, a.groups), P::THREADS, P::LDS_BYTES, st>>>(a, 1);
    return hipGetLastError();
}

template <class P>
hipError_t launch_persistent(const FfnArgs& a, int blocks, bool early, hipStream_t st) {
    if constexpr (P::T0::RING && !P::MIXED) {
        // option queue_early: the queue loop that starts the next task under the end of the current one (measured: no
        // faster on the Mixtral shape, 2-3 % slower on short tiles; kept for machines where the balance differs)
        if (early) {
            hipError_t e = allow_lds(&ffn_persistent_ring_kernel<P>, P::LDS_BYTES);
            if (e != hipSuccess) return e;
            ffn_persistent_ring_kernel<P><<<blocks, P::THREADS, P::LDS_BYTES, st>>>(a);
            return hipGetLastError();
        }
    }
    if constexpr (P::T0::HAND) {
        if (a.split_cnt) {
            hipError_t e = allow_lds(&ffn_persistent_kernel<P, true>, P::LDS_BYTES);
            if (e != hipSuccess) return e;
            ffn_persistent_kernel<P, true><<<blocks, P::THREADS, P::LDS_BYTES, st>>>(a);
            return hipGetLastError();
        }
    }
    hipError_t e = allow_lds(&ffn_persistent_kernel<P>, P::LDS_BYTES);
    if (e != hipSuccess) return e;
    ffn_persistent_kernel<P><<<blocks, P::THREADS, P::LDS_BYTES, st>>>(a);
    return hipGetLastError();
}

template <class P>
int occupancy() {
    int n = 0;
    if (allow_lds(&ffn_persistent_kernel<P>, P::LDS_BYTES) != hipSuccess) return 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(&ffn_persistent_kernel<P>),
                                                     P::THREADS, P::LDS_BYTES) != hipSuccess || n < 1)
        n = 1;
    return n;
}

}  // namespace

// Row-block height chosen for a layer: 256 when the average expert sees at least 256 rows and the up
// projection still gives every compute unit a task at that size.
//
// The 256-row tile runs the hand-ordered slab loop only, which needs: K a multiple of 128 in both projections, no
// ragged column tile (the SwiGLU tile covers 128 intermediate columns, the others 256), and operands below 4 GiB
// (32-bit buffer offsets; `pairs` bounds the token count).
static bool large_tile_ok(int64_t pairs, int H, int I, bool swiglu) {
    const int64_t lim = (int64_t)1 << 32;
    return H % 256 == 0 && I % (swiglu ? 128 : 256) == 0 && pairs * H * 2 < lim && pairs * I * 2 < lim &&
           (int64_t)H * I * 2 < lim;
}

// Tile of a layer: 0 = 128 x 128, 1 = 256 x 256, 2 = 128 x 256, 3 = 256 x 256 with the 128 x 256 tile for the row
// blocks of at most 128 rows.  1 where its conditions hold and the layer has enough rows, else 0; 2 and 3 are tuning
// knobs (option tile16).
//
// Measured (FFN stage, one box, alternating runs): the 128 x 256 tile reaches 93 % of the 256 x 256 tile's rate on a
// plain 4096 x 8192 x 4096 GEMM, but as the tile of a whole layer it loses everywhere (Mixtral shape 5.48 against
// 4.26 ms, 16 experts of 512 rows 0.209 against 0.187 ms, 64 small experts 0.72 against 0.59 ms): twice the tasks,
// each with the same 12 us between two slab loops.  As the tile of short last blocks only it is no better either
// (Mixtral shape 4.38 against 4.26 ms, 16 experts 0.198 against 0.190 ms, 64 small experts 0.590 against 0.592 ms):
// such a task runs through K faster than the full blocks that share its weight tile, drops out of their lockstep
// and fetches its weights past the L2 on its own, with half the time per slab to hide that latency in (with a
// routing that leaves no partial blocks both kernels take the same time).
int bf16_tile(int64_t pairs, int experts, int H, int I, int swiglu, int opt_block_rows, int opt_tile) {
    if (!large_tile_ok(pairs, H, I, swiglu != 0)) return 0;
    const int up_columns = swiglu ? 2 * I : I;
    if (opt_block_rows == 128 || opt_block_rows == 256) return opt_block_rows == 256 ? 1 : 0;   // option block_rows ...
    if (opt_tile >= 0 && opt_tile <= 3) return opt_tile;                                        // ... or tile16
    const int64_t per_expert = pairs / (experts > 0 ? experts : 1);
    if (per_expert < 256) return 0;
    const int64_t tasks = (pairs / 256) * ((up_columns + Tile256::BN - 1) / Tile256::BN);
    return tasks >= 256 ? 1 : 0;
}
int bf16_block_m(int tile) { return tile == 1 || tile == 3 ? 256 : 128; }
int bf16_block_n0(int tile) { return tile == 0 ? SmallPlan::T0::BN : 256; }
int bf16_block_n1(int tile) { return tile == 0 ? SmallPlan::T1::BN : 256; }

template <template <class> class F, class... Args>
static auto for_plan(int tile, bool f16, Args&&... args) {
    if (f16) {
        if (tile == 1) return F<LargePlanH>::run(args...);
        if (tile == 3) return F<MixedPlanH>::run(args...);
        if (tile == 2) return F<MediumPlanH>::run(args...);
        return F<SmallPlanH>::run(args...);
    }
    if (tile == 1) return F<LargePlan>::run(args...);
    if (tile == 3) return F<MixedPlan>::run(args...);
    if (tile == 2) return F<MediumPlan>::run(args...);
    return F<SmallPlan>::run(args...);
}
template <class P> struct RunTiled {
    static hipError_t run(const FfnArgs& a, int max_mtiles, int nnt0, int nnt1, hipStream_t st) { return launch_tiled<P>(a, max_mtiles, nnt0, nnt1, st); }
};
template <class P> struct RunPersistent {
    static hipError_t run(const FfnArgs& a, int blocks, bool early, hipStream_t st) { return launch_persistent<P>(a, blocks, early, st); }
};
template <class P> struct RunOccupancy {
    static int run() { return occupancy<P>(); }
};

hipError_t launch_ffn_tiled_bf16(const FfnArgs& a, int tile, int max_mtiles, int nnt0, int nnt1, hipStream_t st,
                                 bool f16) {
    return for_plan<RunTiled>(tile, f16, a, max_mtiles, nnt0, nnt1, st);
}

hipError_t launch_ffn_persistent_bf16(const FfnArgs& a, int tile, int blocks, bool early, hipStream_t st, bool f16) {
    return for_plan<RunPersistent>(tile, f16, a, blocks, early, st);
}

int ffn_persistent_occupancy_bf16(int tile) { return for_plan<RunOccupancy>(tile, false); }

template <class T>
static hipError_t launch_dense(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                               int act, hipStream_t st) {
    hipError_t e = allow_lds(&gemm_dense_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)((M + T::BM - 1) / T::BM), (unsigned)((N + T::BN - 1) / T::BN));
    gemm_dense_kernel<T><<<grid, T::THREADS, T::LDS_BYTES, st>>>((const uint16_t*)A, (const uint16_t*)B,
                                                                 (const uint16_t*)bias, (uint16_t*)C, (int)M, (int)N,
                                                                 (int)K, act);
    return hipGetLastError();
}

hipError_t launch_gemm_dense_bf16(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                  int64_t K, int act, int opt_tile, hipStream_t st, bool f16) {
    const int64_t lim = (int64_t)1 << 32;
    const bool large = M >= 1024 && N >= 1024 && N % 256 == 0 && K % 128 == 0 && M * K * 2 < lim && N * K * 2 < lim;
    {   // the tile asked for: 1 = 256 x 256, 2 = 128 x 256 (shapes they accept only), 0 = 128 x 128
        const int v = opt_tile;
        if (v == 0) return f16 ? launch_dense<SmallPlanH::T0>(A, B, bias, C, M, N, K, act, st) : launch_dense<SmallPlan::T0>(A, B, bias, C, M, N, K, act, st);
        if ((v == 1 || v == 2) && N % 256 == 0 && K % 128 == 0 && M * K * 2 < lim && N * K * 2 < lim) {
            if (v == 1) return f16 ? launch_dense<Tile256H>(A, B, bias, C, M, N, K, act, st) : launch_dense<Tile256>(A, B, bias, C, M, N, K, act, st);
            return f16 ? launch_dense<Tile128x256H>(A, B, bias, C, M, N, K, act, st) : launch_dense<Tile128x256>(A, B, bias, C, M, N, K, act, st);
        }
    }
    if (f16)
        return large ? launch_dense<LargePlanH::T0>(A, B, bias, C, M, N, K, act, st)
                     : launch_dense<SmallPlanH::T0>(A, B, bias, C, M, N, K, act, st);
    return large ? launch_dense<LargePlan::T0>(A, B, bias, C, M, N, K, act, st)
                 : launch_dense<SmallPlan::T0>(A, B, bias, C, M, N, K, act, st);
}

// ---- building blocks of the backward pass (callers: csrc/backward.hip) ----
bool grouped_gemm_takes_large_tile(int64_t A, int E, int N, int K) {
    const int64_t lim = (int64_t)1 << 32;
    return N % 256 == 0 && K % 128 == 0 && A * K * 2 < lim && (int64_t)N * K * 2 < lim && A / (E > 0 ? E : 1) >= 256;
}

template <class T>
static hipError_t launch_grouped(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                 const int32_t* num_mtiles, const int32_t* count, int max_mtiles, int64_t A, int N, int K,
                                 int act, hipStream_t st) {
    hipError_t e = allow_lds(&grouped_gemm_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    const int64_t blocks = (int64_t)max_mtiles * ((N + T::BN - 1) / T::BN);
    if (blocks > INT32_MAX) return hipErrorInvalidValue;
    grouped_gemm_kernel<T><<<(unsigned)blocks, T::THREADS, T::LDS_BYTES, st>>>((const uint16_t*)a_rows, (const uint16_t*)w,
                                                                               (const uint16_t*)bias, (uint16_t*)out, mtiles,
                                                                               num_mtiles, count, N, K, act,
                                                                               (uint32_t)(A * K * 2));
    return hipGetLastError();
}

hipError_t launch_grouped_gemm_16(const void* a_rows, const void* w, const void* bias, void* out, const MTile* mtiles,
                                  const int32_t* num_mtiles, const int32_t* count, int max_mtiles, int tile, int64_t A,
                                  int N, int K, int act, bool f16, hipStream_t st) {
    if (tile == 2)   // 128-row blocks on the hand-ordered 128 x 256 tile
        return f16 ? launch_grouped<Tile128x256H>(a_rows, w, bias, out, mtiles, num_mtiles, count, max_mtiles, A, N, K, act, st)
                   : launch_grouped<Tile128x256>(a_rows, w, bias, out, mtiles, num_mtiles, count, max_mtiles, A, N, K, act, st);
    if (tile == 1)
        return f16 ? launch_grouped<LargePlanH::T0>(a_rows, w, bias, out, mtiles, num_mtiles, count, max_mtiles, A, N, K, act, st)
                   : launch_grouped<LargePlan::T0>(a_rows, w, bias, out, mtiles, num_mtiles, count, max_mtiles, A, N, K, act, st);
    return f16 ? launch_grouped<SmallPlanH::T0>(a_rows, w, bias, out, mtiles, num_mtiles, count, max_mtiles, A, N, K, act, st)
               : launch_grouped<SmallPlan::T0>(a_rows, w, bias, out, mtiles, num_mtiles, count, max_mtiles, A, N, K, act, st);
}

template <class T>
static hipError_t launch_grouped_deriv(const void* a_rows, const void* w, const void* u, const void* g, void* du, void* dg,
                                       const MTile* mtiles, const int32_t* num_mtiles, const int32_t* count, int max_mtiles,
                                       int64_t A, int N, int K, int hidden_act, hipStream_t st) {
    hipError_t e = allow_lds(&grouped_gemm_deriv_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    const int64_t blocks = (int64_t)max_mtiles * ((N + T::BN - 1) / T::BN);
    if (blocks > INT32_MAX) return hipErrorInvalidValue;
    grouped_gemm_deriv_kernel<T><<<(unsigned)blocks, T::THREADS, T::LDS_BYTES, st>>>(
        (const uint16_t*)a_rows, (const uint16_t*)w, (const uint16_t*)u, (const uint16_t*)g, (uint16_t*)du, (uint16_t*)dg, mtiles,
        num_mtiles, count, N, K, hidden_act, (uint32_t)(A * K * 2));
    return hipGetLastError();
}

// tile: 1 (256 x 256) or 2 (128 x 256): the hand-ordered tiles only.
hipError_t launch_grouped_gemm_deriv_16(const void* a_rows, const void* w, const void* u, const void* g, void* du, void* dg,
                                        const MTile* mtiles, const int32_t* num_mtiles, const int32_t* count, int max_mtiles,
                                        int tile, int64_t A, int N, int K, int hidden_act, bool f16, hipStream_t st) {
    if (tile == 2)
        return f16 ? launch_grouped_deriv<Tile128x256H>(a_rows, w, u, g, du, dg, mtiles, num_mtiles, count, max_mtiles, A, N, K, hidden_act, st)
                   : launch_grouped_deriv<Tile128x256>(a_rows, w, u, g, du, dg, mtiles, num_mtiles, count, max_mtiles, A, N, K, hidden_act, st);
    if (tile == 1)
        return f16 ? launch_grouped_deriv<LargePlanH::T0>(a_rows, w, u, g, du, dg, mtiles, num_mtiles, count, max_mtiles, A, N, K, hidden_act, st)
                   : launch_grouped_deriv<LargePlan::T0>(a_rows, w, u, g, du, dg, mtiles, num_mtiles, count, max_mtiles, A, N, K, hidden_act, st);
    return hipErrorInvalidValue;
}

template <class T>
static hipError_t launch_wgrad(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K,
                               int64_t ld, hipStream_t st) {
    hipError_t e = allow_lds(&wgrad_kernel<T>, T::LDS_BYTES);
    if (e != hipSuccess) return e;
    const dim3 grid((unsigned)((N + T::BM - 1) / T::BM), (unsigned)((K + T::BN - 1) / T::BN), (unsigned)E);
    wgrad_kernel<T><<<grid, T::THREADS, T::LDS_BYTES, st>>>((const uint16_t*)dyT, (const uint16_t*)aT, (uint16_t*)dw, poff,
                                                            N, K, (int)ld, (uint32_t)((int64_t)N * ld * 2),
                                                            (uint32_t)((int64_t)K * ld * 2));
    return hipGetLastError();
}

hipError_t launch_wgrad_16(const void* dyT, const void* aT, void* dw, const int32_t* poff, int E, int N, int K,
                           int64_t ld, bool f16, hipStream_t st) {
    const int64_t lim = (int64_t)1 << 32;
    const bool large = N >= 1024 && K >= 1024 && K % 256 == 0 && N * ld * 2 < lim && K * ld * 2 < lim;
    if (large) return f16 ? launch_wgrad<LargePlanH::T0>(dyT, aT, dw, poff, E, N, K, ld, st)
                          : launch_wgrad<LargePlan::T0>(dyT, aT, dw, poff, E, N, K, ld, st);
    return f16 ? launch_wgrad<SmallPlanH::T0>(dyT, aT, dw, poff, E, N, K, ld, st)
               : launch_wgrad<SmallPlan::T0>(dyT, aT, dw, poff, E, N, K, ld, st);
}

}  // namespace moe355
