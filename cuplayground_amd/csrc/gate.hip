// Router stage: gate logits, top-k selection and gate weights.
//
// The reference has no router (its config macros E_TOP_K / NUM_EXPERTS are defined at
// CMakeLists.txt:207,213 and never read), so the semantics are this library's:
//   logits[t,e] = sum_k x[t,k] * gate_w[e,k] (+ gate_bias[e]) with gate_w [E,H] row-major, the (N,K)
//   operand convention of the reference GEMM (mma.cuh:417-419).
// The fp32 summation order is fixed so that the integer routing results are reproducible bit for bit:
// lane l of a wavefront owns partial sum l and takes, in ascending k, every k with (k/8) % 64 == l using
// one fmaf per element; the 64 partials are folded by an xor butterfly (32,16,8,4,2,1); the bias is added
// last.  Top-k is taken on the logits (softmax and sigmoid are monotone), ties to the lower expert index.
#include <type_traits>
#include <cstdlib>

#include "moe_internal.hpp"
#include "topk.hpp"

namespace moe355 {
namespace {

__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    const float4 a = reinterpret_cast<const float4*>(p)[0];
    const float4 b = reinterpret_cast<const float4*>(p)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
// two 16-bit values packed in a dword -> fp32 (exact)
__device__ __forceinline__ float lo16(uint32_t w, bf16_s) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi16(uint32_t w, bf16_s) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ __forceinline__ float lo16(uint32_t w, f16_s) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu)); }
__device__ __forceinline__ float hi16(uint32_t w, f16_s) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }

template <typename T16>
__device__ __forceinline__ void load8(const T16* p, float (&v)[8]) {
    const uint4 a = reinterpret_cast<const uint4*>(p)[0];
    v[0] = lo16(a.x, T16{}); v[1] = hi16(a.x, T16{});
    v[2] = lo16(a.y, T16{}); v[3] = hi16(a.y, T16{});
    v[4] = lo16(a.z, T16{}); v[5] = hi16(a.z, T16{});
    v[6] = lo16(a.w, T16{}); v[7] = hi16(a.w, T16{});
}

// Folds the 64 per-lane partial sums of 16 independent sums at once.  At xor distance 32, 16, 8, 4 a lane keeps one
// register of each pair and hands the other to its partner (halving the registers per step), then distances 2 and 1
// on the one register left.  Each sum adds lane l to lane l ^ d for d = 32, 16, 8, 4, 2, 1 in that order: the result
// has the bits of the plain butterfly.  Returns the sum of red[index] with index = fold16_index(lane), valid in the
// lanes with (lane & 3) == 0.
// The exchanges stay in the vector ALU: v_permlane32_swap / v_permlane16_swap trade the halves (the odd 16-lane rows)
// of a register pair, which is the keep-one-hand-over-the-other step in one instruction; distances 8 .. 1 are DPP
// moves (row rotate by 8; row shifts by 4 under bank masks; quad permutes).  Through the LDS crossbar (ds_bpermute)
// the seventeen exchanges of a fold cost about as much as a quarter of the multiply-adds they follow.
template <int CTRL, int BANKS = 0xF>
__device__ __forceinline__ float dpp_from(float old, float v) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(old), __float_as_uint(v), CTRL, 0xF, BANKS, false));
}
__device__ __forceinline__ float lane_xor8(float v) { return dpp_from<0x128>(0.0f, v); }                    // row_ror:8
__device__ __forceinline__ float lane_xor4(float v) { return dpp_from<0x114, 0xA>(dpp_from<0x104, 0x5>(0.0f, v), v); }   // row_shl:4 | row_shr:4
__device__ __forceinline__ float lane_xor2(float v) { return dpp_from<0x4E>(0.0f, v); }                     // quad_perm [2,3,0,1]
__device__ __forceinline__ float lane_xor1(float v) { return dpp_from<0xB1>(0.0f, v); }                     // quad_perm [1,0,3,2]

__device__ __forceinline__ float fold16(float (&red)[16], int lane) {
    typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 8; ++i) {      // distance 32: lanes 0..31 keep red[2i], lanes 32..63 keep red[2i+1]
        const u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(red[2 * i]), __float_as_uint(red[2 * i + 1]), false, false);
        red[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {      // distance 16: even 16-lane rows keep red[2i], odd rows red[2i+1]
        const u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(red[2 * i]), __float_as_uint(red[2 * i + 1]), false, false);
        red[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    {
        const bool hi = (lane & 8) != 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float keep = hi ? red[2 * i + 1] : red[2 * i];
            const float send = hi ? red[2 * i] : red[2 * i + 1];
            red[i] = keep + lane_xor8(send);
        }
    }
    {
        const bool hi = (lane & 4) != 0;
        const float keep = hi ? red[1] : red[0];
        const float send = hi ? red[0] : red[1];
        red[0] = keep + lane_xor4(send);
    }
    float sum = red[0];
    sum = sum + lane_xor2(sum);
    sum = sum + lane_xor1(sum);
    return sum;
}
__device__ __forceinline__ int fold16_index(int lane) {
    return ((lane >> 5) & 1) | (((lane >> 4) & 1) << 1) | (((lane >> 3) & 1) << 2) | (((lane >> 2) & 1) << 3);
}

// A wavefront keeps TPW token rows in registers (lane l owns the 8-element chunks l, l+64, ... of each row, as
// fp32) and walks over its share of the experts: one 16-byte load of the expert's row per chunk feeds 8*TPW
// fmafs; the 64 partial sums of 16 (token, expert) pairs are folded together (see the loop).  grid = (token groups of 4*TPW, expert chunks); NCH = chunks per lane = ceil(H / 512).
template <typename T, int NCH, int TPW>
__global__ __launch_bounds__(256) void gate_logits_kernel(const T* __restrict__ x, const T* __restrict__ gate_w,
                                                          const float* __restrict__ gate_bias,
                                                          float* __restrict__ logits, int S, int H, int E,
                                                          int experts_per_block) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t0 = (blockIdx.x * 4 + wave) * TPW;
    if (t0 >= S) return;
    const int nchunk = H >> 3;
    float xr[TPW][NCH][8];
#pragma unroll
    for (int q = 0; q < TPW; ++q) {
        const int t = min(t0 + q, S - 1);          // a ragged last group recomputes the last token; not stored
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int c = lane + j * kWave;
            if (c < nchunk) load8(x + (size_t)t * H + c * 8, xr[q][j]);
            else {
#pragma unroll
                for (int v = 0; v < 8; ++v) xr[q][j][v] = 0.0f;
            }
        }
    }
    const int e0 = blockIdx.y * experts_per_block;
    const int e1 = min(E, e0 + experts_per_block);
    // raw 16-byte chunks of the next expert's row are fetched while the current expert is being summed
    typedef unsigned int raw_t __attribute__((ext_vector_type(sizeof(T) == 4 ? 8 : 4)));
    raw_t wn[NCH];
    auto fetch = [&](int e) {
        const T* wr = gate_w + (size_t)e * H;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int c = lane + j * kWave;
            if (c < nchunk) wn[j] = *reinterpret_cast<const raw_t*>(wr + c * 8);
        }
    };
    fetch(e0);
    // Experts are taken EG at a time so that EG * TPW = 16 partial-sum registers are folded together: at xor
    // distance 32, 16, 8, 4 a lane keeps one register of each pair and hands the other to its partner, which
    // halves the registers per step instead of running six shuffles per sum.  Every sum still adds lane l to
    // lane l ^ d for d = 32, 16, 8, 4, 2, 1 in that order, so the result is bit-identical to the plain butterfly.
    constexpr int EG = 16 / TPW;
    for (int eb = e0; eb < e1; eb += EG) {
        float red[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) red[r] = 0.0f;
#pragma unroll
        for (int g = 0; g < EG; ++g) {
            const int e = eb + g;
            if (e >= e1) break;
            raw_t wc[NCH];
#pragma unroll
            for (int j = 0; j < NCH; ++j) wc[j] = wn[j];
            if (e + 1 < e1) fetch(e + 1);
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                const int c = lane + j * kWave;
                if (c < nchunk) {
                    float wv[8];
                    if constexpr (sizeof(T) == 4) {
#pragma unroll
                        for (int v = 0; v < 8; ++v) wv[v] = __uint_as_float(wc[j][v]);
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            wv[2 * v] = lo16(wc[j][v], T{});
                            wv[2 * v + 1] = hi16(wc[j][v], T{});
                        }
                    }
#pragma unroll
                    for (int q = 0; q < TPW; ++q)
#pragma unroll
                        for (int v = 0; v < 8; ++v)
                            red[g * TPW + q] = __builtin_fmaf(xr[q][j][v], wv[v], red[g * TPW + q]);
                }
            }
        }
        const float sum = fold16(red, lane);
        const int r = fold16_index(lane);
        const int e = eb + r / TPW, t = t0 + r % TPW;
        if ((lane & 3) == 0 && e < e1 && t < S) logits[(size_t)t * E + e] = gate_bias ? sum + gate_bias[e] : sum;
    }
}

template <typename T, int NCH, int TPW>
hipError_t launch_gate_variant(const void* x, const void* gate_w, const float* gate_bias, float* logits, int S, int H,
                               int E, hipStream_t st) {
    const int token_blocks = (S + 4 * TPW - 1) / (4 * TPW);
    // enough workgroups to occupy the chip even when S is small (decode shapes)
    int chunks = 1;
    while (token_blocks * chunks < 1024 && chunks < E) chunks *= 2;
    const int per = (E + chunks - 1) / chunks;
    chunks = (E + per - 1) / per;
    gate_logits_kernel<T, NCH, TPW><<<dim3(token_blocks, chunks), 256, 0, st>>>((const T*)x, (const T*)gate_w,
                                                                                gate_bias, logits, S, H, E, per);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_gate_typed(const void* x, const void* gate_w, const float* gate_bias, float* logits, int S, int H,
                             int E, hipStream_t st) {
    const bool many = (int64_t)S * E >= 4 * 4096;   // enough (token, expert) work to give each wavefront 4 tokens
    if (H <= 1024) return many ? launch_gate_variant<T, 2, 4>(x, gate_w, gate_bias, logits, S, H, E, st)
                               : launch_gate_variant<T, 2, 1>(x, gate_w, gate_bias, logits, S, H, E, st);
    if (H <= 2048) return many ? launch_gate_variant<T, 4, 4>(x, gate_w, gate_bias, logits, S, H, E, st)
                               : launch_gate_variant<T, 4, 1>(x, gate_w, gate_bias, logits, S, H, E, st);
    if (H <= 4096) return many ? launch_gate_variant<T, 8, 2>(x, gate_w, gate_bias, logits, S, H, E, st)
                               : launch_gate_variant<T, 8, 1>(x, gate_w, gate_bias, logits, S, H, E, st);
    if (H <= 8192) return launch_gate_variant<T, 16, 1>(x, gate_w, gate_bias, logits, S, H, E, st);
    if (H <= 16384) return launch_gate_variant<T, 32, 1>(x, gate_w, gate_bias, logits, S, H, E, st);
    return hipErrorInvalidValue;
}

// ---- second logits kernel: register tiles of (tokens x experts), K streamed ----
//
// The kernel above keeps whole token rows in registers and walks the experts one after the other, one 16-byte load
// in flight per chunk: with many experts or few tokens it waits on memory latency most of the time.  Here a wavefront
// owns TT tokens x TE experts (TT * TE running sums per lane), walks K in steps of one 8-element chunk per lane
// (chunk c = lane + 64 j, exactly the elements partial sum `lane` takes), and has the TT + TE loads of the next step
// in flight while it works on the current one.  Every sum sees the same fmaf sequence and the same fold as above, so
// the logits are bit-identical.  A workgroup is WT x WE wavefronts over (tokens, experts); neighbouring wavefronts
// read the same rows at the same time and share them in the compute unit's L1.
template <typename T>
struct RawChunk {
    typedef unsigned int type __attribute__((ext_vector_type(sizeof(T) == 4 ? 8 : 4)));
};

template <typename T>
__device__ __forceinline__ void widen8(const typename RawChunk<T>::type& r, float (&v)[8]) {
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __uint_as_float(r[i]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = lo16(r[i], T{});
            v[2 * i + 1] = hi16(r[i], T{});
        }
    }
}

// The token's top-k selection right behind its sums (FUSE): when the workgroup's WE x TE expert columns cover every
// expert, the logits of its WT x TT tokens meet in LDS and each wavefront selects for its share of the tokens with the
// very function the stand-alone top-k kernel runs -- one launch less, and the logits go to memory only when the caller
// asked for them (`logits` may then be null).
struct GateTopk {
    int32_t* idx;       // [S, k]
    float* w;           // [S, k]
    int k, gate_fn, norm;
};

template <typename T, int TT, int TE, int WT, int WE, bool FUSE>
__global__ __launch_bounds__(WT * WE * 64) void gate_tile_kernel(const T* __restrict__ x, const T* __restrict__ gate_w,
                                                                 const float* __restrict__ gate_bias,
                                                                 float* __restrict__ logits, int S, int H, int E,
                                                                 GateTopk tk) {
    static_assert((TT * TE) % 16 == 0 && 16 % TT == 0, "sums are folded sixteen at a time: TT tokens x 16/TT experts");
    typedef typename RawChunk<T>::type raw_t;
    constexpr int ECOLS = WE * TE;                        // expert columns of a workgroup
    __shared__ float s_log[FUSE ? WT * TT * ECOLS : 1];   // [token of the workgroup][expert]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t0 = (blockIdx.x * WT + wave / WE) * TT, e0 = (blockIdx.y * WE + wave % WE) * TE;
    const bool live = t0 < S && e0 < E;
    if (!FUSE && !live) return;
    if (live) {
        const int nchunk = H >> 3, nstep = (nchunk + kWave - 1) / kWave;
        const T* xrow[TT];
        const T* wrow[TE];
#pragma unroll
        for (int q = 0; q < TT; ++q) xrow[q] = x + (size_t)min(t0 + q, S - 1) * H + lane * 8;    // rows past the end are
#pragma unroll
        for (int g = 0; g < TE; ++g) wrow[g] = gate_w + (size_t)min(e0 + g, E - 1) * H + lane * 8;   // computed, not stored
        float acc[TT][TE];
#pragma unroll
        for (int q = 0; q < TT; ++q)
#pragma unroll
            for (int g = 0; g < TE; ++g) acc[q][g] = 0.0f;
        raw_t xn[TT], wn[TE];
        auto fetch = [&](int j) {
            if (lane + j * kWave < nchunk) {
#pragma unroll
                for (int q = 0; q < TT; ++q) xn[q] = *reinterpret_cast<const raw_t*>(xrow[q] + (size_t)j * (kWave * 8));
#pragma unroll
                for (int g = 0; g < TE; ++g) wn[g] = *reinterpret_cast<const raw_t*>(wrow[g] + (size_t)j * (kWave * 8));
            }
        };
        fetch(0);
        for (int j = 0; j < nstep; ++j) {
            raw_t xc[TT], wc[TE];
#pragma unroll
            for (int q = 0; q < TT; ++q) xc[q] = xn[q];
#pragma unroll
            for (int g = 0; g < TE; ++g) wc[g] = wn[g];
            if (j + 1 < nstep) fetch(j + 1);
            if (lane + j * kWave < nchunk) {      // partial sum `lane` takes chunk lane + 64 j only if the row has it
                float xv[TT][8];
#pragma unroll
                for (int q = 0; q < TT; ++q) widen8<T>(xc[q], xv[q]);
#pragma unroll
                for (int g = 0; g < TE; ++g) {
                    float wv[8];
                    widen8<T>(wc[g], wv);
#pragma unroll
                    for (int q = 0; q < TT; ++q)
#pragma unroll
                        for (int v = 0; v < 8; ++v) acc[q][g] = __builtin_fmaf(xv[q][v], wv[v], acc[q][g]);
                }
            }
        }
        constexpr int EG = 16 / TT;       // experts per fold
        const int r = fold16_index(lane);
#pragma unroll
        for (int gb = 0; gb < TE; gb += EG) {
            float red[16];
#pragma unroll
            for (int g = 0; g < EG; ++g)
#pragma unroll
                for (int q = 0; q < TT; ++q) red[g * TT + q] = acc[q][gb + g];
            const float sum = fold16(red, lane);
            const int e = e0 + gb + r / TT, t = t0 + r % TT;
            if ((lane & 3) == 0 && e < E && t < S) {
                const float val = gate_bias ? sum + gate_bias[e] : sum;
                if (!FUSE || logits) logits[(size_t)t * E + e] = val;
                if (FUSE) s_log[((wave / WE) * TT + r % TT) * ECOLS + e] = val;     // one expert tile per row: e < ECOLS
            }
        }
    }
    if constexpr (FUSE) {
        __syncthreads();
        for (int q = wave; q < WT * TT; q += WT * WE) {   // this wavefront's share of the workgroup's tokens
            const int t = blockIdx.x * (WT * TT) + q;
            if (t < S) topk_one_token<1>(s_log + q * ECOLS, t, E, tk.k, tk.gate_fn, tk.norm, tk.idx, tk.w, lane);
        }
    }
}

// Returns through *fused whether the launch also selected (tk non-null and every expert in one workgroup's columns).
template <typename T, int TT, int TE, int WT, int WE>
hipError_t launch_gate_tile(const void* x, const void* gate_w, const float* gate_bias, float* logits, bool keep_logits,
                            int S, int H, int E, const GateTopk* tk, bool* fused, hipStream_t st) {
    const dim3 grid((S + WT * TT - 1) / (WT * TT), (E + WE * TE - 1) / (WE * TE));
    if (tk && grid.y == 1) {
        gate_tile_kernel<T, TT, TE, WT, WE, true><<<grid, WT * WE * 64, 0, st>>>((const T*)x, (const T*)gate_w, gate_bias,
                                                                                keep_logits ? logits : nullptr, S, H, E, *tk);
        *fused = true;
    } else {
        gate_tile_kernel<T, TT, TE, WT, WE, false><<<grid, WT * WE * 64, 0, st>>>((const T*)x, (const T*)gate_w, gate_bias,
                                                                                 logits, S, H, E, GateTopk{});
    }
    return hipGetLastError();
}

// Tile choice: big tiles when there are enough (token, expert) pairs to fill the chip with them, small ones when
// the layer is decode-sized and only more wavefronts bring more loads in flight; a 4 x 1 wavefront arrangement when
// the experts fit one wavefront's tile.
template <typename T>
hipError_t launch_gate_tiled(const void* x, const void* gate_w, const float* gate_bias, float* logits, bool keep_logits,
                             int S, int H, int E, int opt_tile, const GateTopk* tk, bool* fused, hipStream_t st) {
    const int64_t pairs = (int64_t)S * E;
    int variant = pairs >= 32768 ? 0 : 1;
    if (opt_tile >= 0 && opt_tile <= 2) variant = opt_tile;
#define MOE355_GATE_TILE_ARGS x, gate_w, gate_bias, logits, keep_logits, S, H, E, tk, fused, st
    switch (variant) {
        case 0:
            return E <= 8 ? launch_gate_tile<T, 4, 8, 4, 1>(MOE355_GATE_TILE_ARGS) : launch_gate_tile<T, 4, 8, 2, 2>(MOE355_GATE_TILE_ARGS);
        case 1:
            return E <= 4 ? launch_gate_tile<T, 4, 4, 4, 1>(MOE355_GATE_TILE_ARGS) : launch_gate_tile<T, 4, 4, 2, 2>(MOE355_GATE_TILE_ARGS);
        default:
            return E <= 8 ? launch_gate_tile<T, 2, 8, 4, 1>(MOE355_GATE_TILE_ARGS) : launch_gate_tile<T, 2, 8, 2, 2>(MOE355_GATE_TILE_ARGS);
    }
#undef MOE355_GATE_TILE_ARGS
}

// ---- third logits kernel: the same sums on the matrix cores (16-bit layers, H a multiple of 512) ----
//
// v_mfma_f32_16x16x1_4b_f32 is four independent 16 x 16 outer products with k = 1: D_b[i][j] = C_b[i][j] + A_b[i] B_b[j],
// one multiply-add per element -- and the product of two bf16 (or fp16) values is exact in fp32, so each element sees
// exactly the fmaf the kernels above perform, at the full fp32 rate of the matrix pipe (twice the unpacked vector rate)
// with the widening running beside it on the vector ALU.  A pair of wavefronts owns 16 tokens x 16 experts.  Block b of
// accumulator g carries partial sum p = 4 g + b of every pair of the tile: lane 16 b + i loads the 16-byte chunk
// p + 64 j of token row i (and of expert row i) -- the chunk partial sum p takes in step j, i.e. elements
// 32 (16 j + g) + 8 b onwards -- and its 8 elements go through 8 MFMAs in ascending k.  The even g belong to one
// wavefront of the pair and the odd g to the other (8 accumulators = 128 registers each, so two wavefronts fit a
// SIMD and one's loads and widening hide behind the other's MFMAs).  The 32 partial sums a wavefront holds of a pair
// sit in one lane (accumulator g, register 4 b + r: token 4 (lane / 16) + r, expert lane % 16): p is folded with
// p + 32, 16 and 8 (g with g + 8, 4, 2) in the lane, with p + 4 (g with g + 1) across the two wavefronts through LDS,
// then with p + 2 and p + 1 (b) in the lane again -- the pairings of fold16, so the logits are bit-identical.
typedef float gate_f32x16 __attribute__((ext_vector_type(16)));

// PAIRS wavefront pairs per workgroup, 16 expert columns each.  FUSE: the workgroup's columns cover every expert
// (grid.y == 1) and the selection follows right behind the sums, as in gate_tile_kernel.
template <typename T, int PAIRS, bool FUSE>
__global__ __launch_bounds__(PAIRS * 128) __attribute__((amdgpu_waves_per_eu(2, 2))) void gate_mfma_kernel(const T* __restrict__ x, const T* __restrict__ gate_w,
                                                        const float* __restrict__ gate_bias, float* __restrict__ logits,
                                                        int S, int H, int E, GateTopk tk) {
    typedef typename RawChunk<T>::type raw_t;
    constexpr int ECOLS = PAIRS * 16;
    __shared__ float s_odd[PAIRS][16][64];      // [pair][4 b + r][lane]: the odd wavefront's sums over its g
    __shared__ float s_log[FUSE ? 16 * ECOLS : 1];   // [token of the tile][expert]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pair = wave >> 1, odd = wave & 1;
    const int b = lane >> 4, i = lane & 15;
    const int t0 = blockIdx.x * 16, e0 = (blockIdx.y * PAIRS + pair) * 16;
    const bool live = e0 < E;                   // an expert tile past the last one: nothing to do, but meet the barrier
    gate_f32x16 acc[8];
#pragma unroll
    for (int g = 0; g < 8; ++g)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[g][v] = 0.f;
    if (live) {
        // this wavefront's chunks: g = 2 gg + odd
        const T* xrow = x + (size_t)min(t0 + i, S - 1) * H + 8 * b + 32 * odd;
        const T* wrow = gate_w + (size_t)min(e0 + i, E - 1) * H + 8 * b + 32 * odd;
        raw_t xn[8], wn[8];
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            xn[g] = *reinterpret_cast<const raw_t*>(xrow + 64 * g);
            wn[g] = *reinterpret_cast<const raw_t*>(wrow + 64 * g);
        }
        // One step = 512 elements of every row.  The chunks of the next step are requested as soon as this step's have
        // been widened, each into the registers it will be used from, and the last step is a copy of the loop body
        // without requests: with a condition around the requests the chunks reach their registers through copies at the
        // end of the loop body, and the wait in front of those copies exposes the latency of the requests issued last
        // in every step (2.5 us of a step's 3.6 on a 64-expert layer).
        auto step = [&](const T* xnext, const T* wnext, auto more) {
#pragma unroll
            for (int g = 0; g < 8; g += 2) {    // two accumulators at a time: consecutive MFMAs are independent
                float xv[2][8], wv[2][8];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    widen8<T>(xn[g + h], xv[h]);
                    widen8<T>(wn[g + h], wv[h]);
                    if constexpr (decltype(more)::value) {
                        xn[g + h] = *reinterpret_cast<const raw_t*>(xnext + 64 * (g + h));
                        wn[g + h] = *reinterpret_cast<const raw_t*>(wnext + 64 * (g + h));
                    }
                }
#pragma unroll
                for (int v = 0; v < 8; ++v)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        acc[g + h] = __builtin_amdgcn_mfma_f32_16x16x1f32(xv[h][v], wv[h][v], acc[g + h], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);      // or the scheduler gathers every request of the step behind its last MFMA
            }
        };
        const int nstep = H / 512;
        for (int j = 1; j < nstep; ++j) step(xrow + 512 * j, wrow + 512 * j, std::true_type{});
        step(xrow, wrow, std::false_type{});
    }
    // acc[gg] holds g = 2 gg + odd: g + 8, g + 4, g + 2 are gg + 4, gg + 2, gg + 1
    float u[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const float s0 = acc[0][v] + acc[4][v], s1 = acc[1][v] + acc[5][v], s2 = acc[2][v] + acc[6][v],
                    s3 = acc[3][v] + acc[7][v];                                        // p with p + 32
        u[v] = (s0 + s2) + (s1 + s3);                                                  // ... p + 16, then p + 8
    }
    if (odd) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s_odd[pair][v][lane] = u[v];
    }
    __syncthreads();
    if (!FUSE && (odd || !live)) return;
    if (!odd && live) {
        const int e = e0 + i;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float q[4];
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) q[bb] = u[4 * bb + r] + s_odd[pair][4 * bb + r][lane];     // ... p + 4
            const float sum = (q[0] + q[2]) + (q[1] + q[3]);                                           // ... p + 2, p + 1
            const int t = t0 + 4 * b + r;
            if (t < S && e < E) {
                const float val = gate_bias ? sum + gate_bias[e] : sum;
                if (!FUSE || logits) logits[(size_t)t * E + e] = val;
                if (FUSE) s_log[(4 * b + r) * ECOLS + e] = val;                       // grid.y == 1: e < ECOLS
            }
        }
    }
    if constexpr (FUSE) {
        __syncthreads();
        for (int q = wave; q < 16; q += 2 * PAIRS) {      // this wavefront's share of the tile's tokens
            const int t = t0 + q;
            if (t < S) topk_one_token<1>(s_log + q * ECOLS, t, E, tk.k, tk.gate_fn, tk.norm, tk.idx, tk.w, lane);
        }
    }
}

// The matrix-core kernel takes 16-bit layers whose rows split into full steps of 512 elements, when the experts fill
// most of its 16 columns and there are enough 16 x 16 tiles for every SIMD of the chip to get several.  With at most 64
// experts one workgroup holds them all (two or four wavefront pairs) and selects as well (*fused).
template <typename T>
bool launch_gate_mfma(const void* x, const void* gate_w, const float* gate_bias, float* logits, bool keep_logits, int S,
                      int H, int E, int opt_mfma, const GateTopk* tk, bool wide_fusion, bool* fused, hipStream_t st,
                      hipError_t* err) {
    if (H % 512 != 0) return false;
    const int et = (E + 15) / 16;
    bool use = et * 16 * 3 <= E * 4 && (int64_t)((S + 15) / 16) * et >= 2048;
    if (opt_mfma != MOE_OPT_AUTO) use = opt_mfma != 0;
    if (!use) return false;
    const unsigned tiles = (unsigned)((S + 15) / 16);
    if (tk && et <= 2) {
        gate_mfma_kernel<T, 2, true><<<dim3(tiles, 1), 256, 0, st>>>((const T*)x, (const T*)gate_w, gate_bias,
                                                                    keep_logits ? logits : nullptr, S, H, E, *tk);
        *fused = true;
    } else if (tk && et <= 4 && wide_fusion) {   // on request only: the 512-thread form measured 17 us slower than two launches
        gate_mfma_kernel<T, 4, true><<<dim3(tiles, 1), 512, 0, st>>>((const T*)x, (const T*)gate_w, gate_bias,
                                                                    keep_logits ? logits : nullptr, S, H, E, *tk);
        *fused = true;
    } else {
        gate_mfma_kernel<T, 2, false><<<dim3(tiles, (et + 1) / 2), 256, 0, st>>>((const T*)x, (const T*)gate_w, gate_bias,
                                                                                logits, S, H, E, GateTopk{});
    }
    *err = hipGetLastError();
    return true;
}

// One wavefront per token.
template <int J>
__global__ __launch_bounds__(256) void topk_kernel(const float* __restrict__ logits, int S, int E, int k, int gate_fn,
                                                   int norm, int32_t* __restrict__ topk_idx,
                                                   float* __restrict__ topk_w) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + wave;
    if (t >= S) return;
    topk_one_token<J>(logits + (size_t)t * E, t, E, k, gate_fn, norm, topk_idx, topk_w, lane);
}

// Router statistics for a load-balancing loss.  Block b, wavefront w takes tokens (4b + w) + 4*gridDim.x*i; a lane
// keeps fp64 sums of the gate scores of its experts; wavefront sums meet in LDS in wavefront order and are written as
// per-block partials, so the result does not depend on scheduling.
__global__ __launch_bounds__(256) void router_stats_partial_kernel(const float* __restrict__ logits,
                                                                   const int32_t* __restrict__ topk_idx, int S, int E,
                                                                   int k, int gate_fn, double* __restrict__ part_prob,
                                                                   int32_t* __restrict__ part_cnt) {
    __shared__ double s_sum[4][kMaxExperts];
    __shared__ int s_cnt[kMaxExperts];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int J = kMaxExperts / kWave;
    for (int e = threadIdx.x; e < E; e += 256) s_cnt[e] = 0;
    __syncthreads();
    double acc[J];
#pragma unroll
    for (int j = 0; j < J; ++j) acc[j] = 0.0;
    for (int t = blockIdx.x * 4 + wave; t < S; t += 4 * gridDim.x) {
        float v[J];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int e = j * kWave + lane;
            v[j] = e < E ? logits[(size_t)t * E + e] : -INFINITY;
            mx = fmaxf(mx, v[j]);
        }
        if (gate_fn == MOE_GATE_SOFTMAX) {
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
            float part = 0.0f;
#pragma unroll
            for (int j = 0; j < J; ++j) {
                v[j] = j * kWave + lane < E ? expf(v[j] - mx) : 0.0f;
                part = part + v[j];
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) part = part + __shfl_xor(part, off, kWave);
#pragma unroll
            for (int j = 0; j < J; ++j) acc[j] += (double)(v[j] / part);
        } else {
#pragma unroll
            for (int j = 0; j < J; ++j)
                if (j * kWave + lane < E) acc[j] += (double)(1.0f / (1.0f + expf(-v[j])));
        }
        if (lane < k) {
            const int e = topk_idx[(size_t)t * k + lane];
            if ((unsigned)e < (unsigned)E) atomicAdd(&s_cnt[e], 1);   // ids outside [0, E) are counted nowhere
        }
    }
#pragma unroll
    for (int j = 0; j < J; ++j)
        if (j * kWave + lane < E) s_sum[wave][j * kWave + lane] = acc[j];
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) {
        part_prob[(size_t)blockIdx.x * E + e] = ((s_sum[0][e] + s_sum[1][e]) + s_sum[2][e]) + s_sum[3][e];
        part_cnt[(size_t)blockIdx.x * E + e] = s_cnt[e];
    }
}

__global__ __launch_bounds__(512) void router_stats_final_kernel(const double* __restrict__ part_prob,
                                                                 const int32_t* __restrict__ part_cnt, int blocks,
                                                                 int S, int E, int k, float* __restrict__ load,
                                                                 float* __restrict__ mean_prob,
                                                                 float* __restrict__ aux_loss) {
    __shared__ double s_prod[kMaxExperts];
    const int e = threadIdx.x;
    if (e < E) {
        double sum = 0.0;
        long long cnt = 0;
        for (int b = 0; b < blocks; ++b) {
            sum += part_prob[(size_t)b * E + e];
            cnt += part_cnt[(size_t)b * E + e];
        }
        const double mp = sum / (double)S, ld = (double)cnt / ((double)S * (double)k);
        if (mean_prob) mean_prob[e] = (float)mp;
        if (load) load[e] = (float)ld;
        s_prod[e] = mp * ld;
    }
    __syncthreads();
    if (threadIdx.x == 0 && aux_loss) {
        double a = 0.0;
        for (int i = 0; i < E; ++i) a += s_prod[i];
        *aux_loss = (float)((double)E * a);
    }
}

}  // namespace

hipError_t launch_router_stats(const float* logits, const int32_t* topk_idx, int S, int E, int k, int gate_fn,
                               double* part_prob, int32_t* part_cnt, float* load, float* mean_prob, float* aux_loss,
                               hipStream_t st) {
    const int blocks = min(kStatsBlocks, (S + 3) / 4);
    router_stats_partial_kernel<<<blocks, 256, 0, st>>>(logits, topk_idx, S, E, k, gate_fn, part_prob, part_cnt);
    router_stats_final_kernel<<<1, 512, 0, st>>>(part_prob, part_cnt, blocks, S, E, k, load, mean_prob, aux_loss);
    return hipGetLastError();
}

// Logits kernel by shape; *fused (when tk is given) says whether that launch has selected as well.
static hipError_t launch_gate_logits(const void* x, const void* gate_w, const float* gate_bias, float* logits, bool keep_logits,
                                     int S, int H, int E, int act_dtype, const moe_options& opt, const GateTopk* tk, bool* fused,
                                     hipStream_t st) {
    // Many experts on many tokens: the first kernel (token rows in registers, experts streamed) reads least per sum.
    // Everything else -- few experts, or decode-sized batches -- goes to the register-tiled kernel.
    if (act_dtype != MOE_DTYPE_F32) {
        hipError_t e = hipSuccess;
        const bool taken = act_dtype == MOE_DTYPE_FP16
            ? launch_gate_mfma<f16_s>(x, gate_w, gate_bias, logits, keep_logits, S, H, E, opt.gate_mfma, tk, opt.gate_fused_topk == 1, fused, st, &e)
            : launch_gate_mfma<bf16_s>(x, gate_w, gate_bias, logits, keep_logits, S, H, E, opt.gate_mfma, tk, opt.gate_fused_topk == 1, fused, st, &e);
        if (taken) return e;
    }
    bool rows_in_registers = E >= 32 && (int64_t)S * E >= ((int64_t)1 << 19);
    if (opt.gate_kernel != MOE_OPT_AUTO) rows_in_registers = opt.gate_kernel == 1;
    if (rows_in_registers) {
        if (act_dtype == MOE_DTYPE_F32) return launch_gate_typed<float>(x, gate_w, gate_bias, logits, S, H, E, st);
        if (act_dtype == MOE_DTYPE_FP16) return launch_gate_typed<f16_s>(x, gate_w, gate_bias, logits, S, H, E, st);
        return launch_gate_typed<bf16_s>(x, gate_w, gate_bias, logits, S, H, E, st);
    }
    if (act_dtype == MOE_DTYPE_F32) return launch_gate_tiled<float>(x, gate_w, gate_bias, logits, keep_logits, S, H, E, opt.gate_tile, tk, fused, st);
    if (act_dtype == MOE_DTYPE_FP16) return launch_gate_tiled<f16_s>(x, gate_w, gate_bias, logits, keep_logits, S, H, E, opt.gate_tile, tk, fused, st);
    return launch_gate_tiled<bf16_s>(x, gate_w, gate_bias, logits, keep_logits, S, H, E, opt.gate_tile, tk, fused, st);
}

static hipError_t launch_topk(const float* logits, int S, int E, int k, int gate_fn, int norm, int32_t* topk_idx,
                       float* topk_w, hipStream_t st) {
    const unsigned grid = (unsigned)((S + 3) / 4);
    if (E <= 64) topk_kernel<1><<<grid, 256, 0, st>>>(logits, S, E, k, gate_fn, norm, topk_idx, topk_w);
    else if (E <= 128) topk_kernel<2><<<grid, 256, 0, st>>>(logits, S, E, k, gate_fn, norm, topk_idx, topk_w);
    else if (E <= 256) topk_kernel<4><<<grid, 256, 0, st>>>(logits, S, E, k, gate_fn, norm, topk_idx, topk_w);
    else topk_kernel<kMaxExperts / kWave><<<grid, 256, 0, st>>>(logits, S, E, k, gate_fn, norm, topk_idx, topk_w);
    return hipGetLastError();
}

// The router: logits, selection, weights.  One launch where the logits kernel of the shape can hold every expert of a
// token in one workgroup (option gate_fused_topk, on unless 0), else the logits kernel followed by the top-k kernel.
// `logits` is always valid scratch [S, E]; with keep_logits false it is written only when the two-launch form needs it.
hipError_t launch_gate(const void* x, const void* gate_w, const float* gate_bias, float* logits, bool keep_logits, int S,
                       int H, int E, int k, int gate_fn, int norm, int32_t* topk_idx, float* topk_w, int act_dtype,
                       const moe_options& opt, hipStream_t st) {
    const GateTopk tk{topk_idx, topk_w, k, gate_fn, norm};
    bool fused = false;
    const hipError_t e = launch_gate_logits(x, gate_w, gate_bias, logits, keep_logits, S, H, E, act_dtype, opt,
                                            opt.gate_fused_topk == 0 ? nullptr : &tk, &fused, st);
    if (e != hipSuccess || fused) return e;
    return launch_topk(logits, S, E, k, gate_fn, norm, topk_idx, topk_w, st);
}

}  // namespace moe355
