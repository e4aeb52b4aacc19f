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
#include "moe_internal.hpp"

namespace moe355 {
namespace {

__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    const float4 a = reinterpret_cast<const float4*>(p)[0];
    const float4 b = reinterpret_cast<const float4*>(p)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const uint16_t* p, float (&v)[8]) {
    const uint4 a = reinterpret_cast<const uint4*>(p)[0];
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xFFFF0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xFFFF0000u);
    v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xFFFF0000u);
    v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xFFFF0000u);
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
                            wv[2 * v] = __uint_as_float(wc[j][v] << 16);
                            wv[2 * v + 1] = __uint_as_float(wc[j][v] & 0xFFFF0000u);
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
#pragma unroll
        for (int step = 0; step < 4; ++step) {
            const int off = 32 >> step, n = 16 >> step;
            const bool hi = (lane & off) != 0;
#pragma unroll
            for (int i = 0; i < n / 2; ++i) {
                const float keep = hi ? red[2 * i + 1] : red[2 * i];
                const float send = hi ? red[2 * i] : red[2 * i + 1];
                red[i] = keep + __shfl_xor(send, off, kWave);
            }
        }
        float sum = red[0];
        sum = sum + __shfl_xor(sum, 2, kWave);
        sum = sum + __shfl_xor(sum, 1, kWave);
        // the lane's register index: bit 0 came from lane bit 5, bit 1 from bit 4, bit 2 from bit 3, bit 3 from bit 2
        const int r = ((lane >> 5) & 1) | (((lane >> 4) & 1) << 1) | (((lane >> 3) & 1) << 2) | (((lane >> 2) & 1) << 3);
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

struct Cand {
    float v;
    int i;
};
__device__ __forceinline__ bool better(const Cand& a, const Cand& b) {
    return a.v > b.v || (a.v == b.v && a.i < b.i);
}

// One wavefront per token; lane l keeps logits of experts l, l+64, ... (at most 8) in registers.
// The selection is total: a NaN logit ranks as -inf (behind every number, ties to the lower index), so a token row
// that overflowed still gets k distinct, valid experts; its weights are computed from the logits as they are and
// come out NaN, which is what reaches the output of that token and of no other.
__global__ __launch_bounds__(256) void topk_kernel(const float* __restrict__ logits, int S, int E, int k, int gate_fn,
                                                   int norm, int32_t* __restrict__ topk_idx,
                                                   float* __restrict__ topk_w) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + wave;
    if (t >= S) return;
    constexpr int J = kMaxExperts / kWave;
    float v[J];
    unsigned avail = 0;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int e = j * kWave + lane;
        v[j] = 0.0f;
        if (e < E) {
            v[j] = logits[(size_t)t * E + e];
            avail |= 1u << j;
        }
    }
    const unsigned valid = avail;
    float my_l = 0.0f;
    int my_i = 0;
    float top_l = 0.0f;
    for (int r = 0; r < k; ++r) {
        Cand c{-INFINITY, 0x7FFFFFFF};
#pragma unroll
        for (int j = 0; j < J; ++j) {
            if ((avail >> j) & 1u) {
                Cand d{v[j] != v[j] ? -INFINITY : v[j], j * kWave + lane};
                if (better(d, c)) c = d;
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            Cand o{__shfl_xor(c.v, off, kWave), __shfl_xor(c.i, off, kWave)};
            if (better(o, c)) c = o;
        }
        if ((c.i & (kWave - 1)) == lane) avail &= ~(1u << (c.i >> 6));
        // the logit behind the winning key, as stored (a NaN ranks as -inf but stays a NaN in the weights)
        float mine = v[0];
#pragma unroll
        for (int j = 1; j < J; ++j) mine = (c.i >> 6) == j ? v[j] : mine;
        const float cv = __shfl(mine, c.i & (kWave - 1), kWave);
        if (lane == r) { my_l = cv; my_i = c.i; }
        if (r == 0) top_l = cv;
    }
    float p = 0.0f;
    if (gate_fn == MOE_GATE_SOFTMAX) {
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < J; ++j)
            if ((valid >> j) & 1u) part = part + expf(v[j] - top_l);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) part = part + __shfl_xor(part, off, kWave);
        if (lane < k) p = expf(my_l - top_l) / part;
    } else {
        if (lane < k) p = 1.0f / (1.0f + expf(-my_l));
    }
    if (norm) {
        float sum = p;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) sum = sum + __shfl_xor(sum, off, kWave);
        p = p / sum;
    }
    if (lane < k) {
        topk_idx[(size_t)t * k + lane] = my_i;
        topk_w[(size_t)t * k + lane] = p;
    }
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

hipError_t launch_gate_logits(const void* x, const void* gate_w, const float* gate_bias, float* logits, int S, int H,
                              int E, int act_dtype, hipStream_t st) {
    if (act_dtype == MOE_DTYPE_F32) return launch_gate_typed<float>(x, gate_w, gate_bias, logits, S, H, E, st);
    return launch_gate_typed<uint16_t>(x, gate_w, gate_bias, logits, S, H, E, st);
}

hipError_t launch_topk(const float* logits, int S, int E, int k, int gate_fn, int norm, int32_t* topk_idx,
                       float* topk_w, hipStream_t st) {
    topk_kernel<<<(S + 3) / 4, 256, 0, st>>>(logits, S, E, k, gate_fn, norm, topk_idx, topk_w);
    return hipGetLastError();
}

}  // namespace moe355
