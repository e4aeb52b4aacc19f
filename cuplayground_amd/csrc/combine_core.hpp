// The arithmetic of the combine, shared by the combine kernels (combine.hip) and by the FFN kernels that combine a
// token as soon as its last expert row is finished (ffn_common.hpp: combine_arrivals):
//   out[t, c..] = sum over ranks r (ascending) of topk_w[t,r] * y[pair_row[t,r], c..]
// accumulated in fp32 and rounded once; pairs with pair_row < 0 (dropped) contribute nothing.  One function for both
// callers, so that where a token is combined cannot change a bit of the result.
#pragma once

#include "moe_internal.hpp"

namespace moe355 {

__device__ __forceinline__ uint32_t cmb_pack2(float lo, float hi, bf16_s) {
    // round to nearest even, the rounding the oracle and torch use for bf16
    uint32_t a = __float_as_uint(lo), b = __float_as_uint(hi);
    a += 0x7FFFu + ((a >> 16) & 1u);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return (a >> 16) | (b & 0xFFFF0000u);
}
__device__ __forceinline__ uint32_t cmb_pack2(float lo, float hi, f16_s) {
    const uint32_t a = __builtin_bit_cast(uint16_t, (_Float16)lo), b = __builtin_bit_cast(uint16_t, (_Float16)hi);   // RNE
    return a | (b << 16);
}
__device__ __forceinline__ float cmb_lo(uint32_t w, bf16_s) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float cmb_hi(uint32_t w, bf16_s) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ __forceinline__ float cmb_lo(uint32_t w, f16_s) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu)); }
__device__ __forceinline__ float cmb_hi(uint32_t w, f16_s) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }

// 16-byte loads from global memory, four at a time.  FRESH: agent-scope loads, which are not answered from a cache
// that another XCD's stores do not reach -- for rows written earlier in the same launch by workgroups that may sit on
// another XCD.  The four loads of a group are in flight together and are waited for once.
template <bool FRESH>
__device__ __forceinline__ void cmb_load4(const void* const (&p)[4], const bool (&on)[4], uint4 (&v)[4]) {
    if constexpr (FRESH) {
        typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
        u32x4_t r0 = {0u, 0u, 0u, 0u}, r1 = r0, r2 = r0, r3 = r0;
        // each load is tied to the register it fills ("+v"), so that a lane that skips it keeps its zeros and the
        // compiler has no copy to make between the load and the wait
        if (on[0]) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "+v"(r0) : "v"(p[0]) : "memory");
        if (on[1]) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "+v"(r1) : "v"(p[1]) : "memory");
        if (on[2]) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "+v"(r2) : "v"(p[2]) : "memory");
        if (on[3]) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "+v"(r3) : "v"(p[3]) : "memory");
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3)::"memory");
        v[0] = uint4{r0[0], r0[1], r0[2], r0[3]};
        v[1] = uint4{r1[0], r1[1], r1[2], r1[3]};
        v[2] = uint4{r2[0], r2[1], r2[2], r2[3]};
        v[3] = uint4{r3[0], r3[1], r3[2], r3[3]};
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = on[j] ? *reinterpret_cast<const uint4*>(p[j]) : uint4{0u, 0u, 0u, 0u};
    }
}

// Eight consecutive columns [c, c + 8) of token t, 16-bit types.
template <typename T16, bool FRESH>
__device__ __forceinline__ void combine_token_16(const uint16_t* __restrict__ y, const int32_t* __restrict__ pair_row,
                                                 const float* __restrict__ topk_w, int t, int k, int H, int c,
                                                 uint16_t* __restrict__ out) {
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (int r0 = 0; r0 < k; r0 += 4) {
        const void* p[4];
        bool on[4];
        float w[4];
        uint4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = r0 + j < k ? pair_row[(size_t)t * k + r0 + j] : -1;
            on[j] = row >= 0;
            w[j] = on[j] ? topk_w[(size_t)t * k + r0 + j] : 0.0f;
            p[j] = y + (size_t)(on[j] ? row : 0) * H + c;
        }
        cmb_load4<FRESH>(p, on, v);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (!on[j]) continue;
            const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] = acc[2 * i] + w[j] * cmb_lo(u[i], T16{});
                acc[2 * i + 1] = acc[2 * i + 1] + w[j] * cmb_hi(u[i], T16{});
            }
        }
    }
    uint4 o;
    o.x = cmb_pack2(acc[0], acc[1], T16{});
    o.y = cmb_pack2(acc[2], acc[3], T16{});
    o.z = cmb_pack2(acc[4], acc[5], T16{});
    o.w = cmb_pack2(acc[6], acc[7], T16{});
    *reinterpret_cast<uint4*>(out + (size_t)t * H + c) = o;
}

// Four consecutive columns of token t, fp32.
template <bool FRESH>
__device__ __forceinline__ void combine_token_f32(const float* __restrict__ y, const int32_t* __restrict__ pair_row,
                                                  const float* __restrict__ topk_w, int t, int k, int H, int c,
                                                  float* __restrict__ out) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int r0 = 0; r0 < k; r0 += 4) {
        const void* p[4];
        bool on[4];
        float w[4];
        uint4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = r0 + j < k ? pair_row[(size_t)t * k + r0 + j] : -1;
            on[j] = row >= 0;
            w[j] = on[j] ? topk_w[(size_t)t * k + r0 + j] : 0.0f;
            p[j] = y + (size_t)(on[j] ? row : 0) * H + c;
        }
        cmb_load4<FRESH>(p, on, v);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (!on[j]) continue;
            acc[0] = acc[0] + w[j] * __uint_as_float(v[j].x);
            acc[1] = acc[1] + w[j] * __uint_as_float(v[j].y);
            acc[2] = acc[2] + w[j] * __uint_as_float(v[j].z);
            acc[3] = acc[3] + w[j] * __uint_as_float(v[j].w);
        }
    }
    uint4 o = {__float_as_uint(acc[0]), __float_as_uint(acc[1]), __float_as_uint(acc[2]), __float_as_uint(acc[3])};
    *reinterpret_cast<uint4*>(out + (size_t)t * H + c) = o;
}

// ---- U tokens at a time, for the combine that runs as tasks of the FFN queue kernels (ffn_common.hpp: combine_while_idle) ----
// A queue kernel keeps one to three workgroups per compute unit, so nothing but the code itself puts memory requests in
// flight: the rows of up to U tokens (R ranks each) are requested together and waited for once.  Per token the
// arithmetic is that of combine_token_16 / combine_token_f32 above, statement for statement -- acc = acc + w * y in
// ascending rank order, one rounding -- so where and how many at a time a token is combined cannot change a bit.
// All loads are agent-scope (the rows were written earlier in this launch, possibly on another XCD).
template <class ET> struct CmbElem;      // ET: bf16_s, f16_s or float
template <> struct CmbElem<bf16_s> { static constexpr int N = 8; };
template <> struct CmbElem<f16_s> { static constexpr int N = 8; };
template <> struct CmbElem<float> { static constexpr int N = 4; };

template <class ET>
__device__ __forceinline__ void cmb_accumulate(float (&acc)[CmbElem<ET>::N], float w, const uint32_t (&u)[4]) {
    if constexpr (CmbElem<ET>::N == 4) {
        acc[0] = acc[0] + w * __uint_as_float(u[0]);
        acc[1] = acc[1] + w * __uint_as_float(u[1]);
        acc[2] = acc[2] + w * __uint_as_float(u[2]);
        acc[3] = acc[3] + w * __uint_as_float(u[3]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = acc[2 * i] + w * cmb_lo(u[i], ET{});
            acc[2 * i + 1] = acc[2 * i + 1] + w * cmb_hi(u[i], ET{});
        }
    }
}

// tok[u] (u < n <= U): the tokens; c: this thread's first column (CmbElem<ET>::N consecutive columns, c < H).  The ranks
// are taken R at a time (U x R rows in flight).
template <class ET, int U, int R>
__device__ __forceinline__ void combine_tokens_fresh(const void* __restrict__ y, const int32_t* __restrict__ pair_row,
                                                     const float* __restrict__ topk_w, const int (&tok)[U], int n, int k,
                                                     int H, int c, void* __restrict__ out) {
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    constexpr int N = CmbElem<ET>::N;
    constexpr int EB = 16 / N;                 // bytes per element
    float acc[U][N];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < N; ++i) acc[u][i] = 0.0f;
    for (int r0 = 0; r0 < k; r0 += R) {
        bool on[U][R];
        float w[U][R];
        u32x4_t v[U][R];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < R; ++j) {
                const int row = (u < n && r0 + j < k) ? pair_row[(size_t)tok[u] * k + r0 + j] : -1;
                on[u][j] = row >= 0;
                w[u][j] = on[u][j] ? topk_w[(size_t)tok[u] * k + r0 + j] : 0.0f;
                const char* p = static_cast<const char*>(y) + ((size_t)(on[u][j] ? row : 0) * H + c) * EB;
                v[u][j] = u32x4_t{0u, 0u, 0u, 0u};
                // tied to the register it fills: a lane that skips the load keeps its zeros
                if (on[u][j]) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "+v"(v[u][j]) : "v"(p) : "memory");
            }
        // one wait for everything in flight; every destination register is named so that no use can move above it
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < R; ++j) asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[u][j])::"memory");
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < R; ++j) {
                if (!on[u][j]) continue;
                const uint32_t q[4] = {v[u][j][0], v[u][j][1], v[u][j][2], v[u][j][3]};
                cmb_accumulate<ET>(acc[u], w[u][j], q);
            }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (u >= n) continue;
        uint4 o;
        if constexpr (N == 4) {
            o = uint4{__float_as_uint(acc[u][0]), __float_as_uint(acc[u][1]), __float_as_uint(acc[u][2]), __float_as_uint(acc[u][3])};
        } else {
            o.x = cmb_pack2(acc[u][0], acc[u][1], ET{});
            o.y = cmb_pack2(acc[u][2], acc[u][3], ET{});
            o.z = cmb_pack2(acc[u][4], acc[u][5], ET{});
            o.w = cmb_pack2(acc[u][6], acc[u][7], ET{});
        }
        *reinterpret_cast<uint4*>(static_cast<char*>(out) + ((size_t)tok[u] * H + c) * EB) = o;
    }
}

}  // namespace moe355
