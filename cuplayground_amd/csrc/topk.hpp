// Top-k selection and gate weights of one token by one wavefront; shared by the stand-alone top-k kernel and by the
// single-workgroup router of decode-sized layers.
#pragma once

#include "moe_internal.hpp"

namespace moe355 {

struct Cand {
    float v;
    int i;
};
__device__ __forceinline__ bool better(const Cand& a, const Cand& b) {
    return a.v > b.v || (a.v == b.v && a.i < b.i);
}

// The best candidate of the 64 lanes, in every lane.  `better` is a total order, so the result does not depend on the
// order of the comparisons: lanes exchange through the cross-lane data paths of the ALU (within quads, then mirrored
// within 8 and 16 lanes), which cost a few cycles each where a shuffle through the LDS crossbar costs a round trip,
// and the four rows meet through scalar registers.
template <int CTRL>
__device__ __forceinline__ Cand dpp_cand(const Cand& c) {
    Cand o;
    o.v = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(c.v), CTRL, 0xF, 0xF, false));
    o.i = __builtin_amdgcn_update_dpp(0, c.i, CTRL, 0xF, 0xF, false);
    return o;
}
__device__ __forceinline__ Cand wave_best(Cand c) {
    Cand o = dpp_cand<0xB1>(c);            // quad_perm [1,0,3,2]: lane ^ 1
    if (better(o, c)) c = o;
    o = dpp_cand<0x4E>(c);                 // quad_perm [2,3,0,1]: lane ^ 2
    if (better(o, c)) c = o;
    o = dpp_cand<0x141>(c);                // row_half_mirror: i <-> 7 - i within 8 lanes
    if (better(o, c)) c = o;
    o = dpp_cand<0x140>(c);                // row_mirror: i <-> 15 - i within 16 lanes
    if (better(o, c)) c = o;
    Cand best{__int_as_float(__builtin_amdgcn_readlane(__float_as_int(c.v), 0)), __builtin_amdgcn_readlane(c.i, 0)};
#pragma unroll
    for (int row = 1; row < 4; ++row) {
        const Cand r{__int_as_float(__builtin_amdgcn_readlane(__float_as_int(c.v), 16 * row)),
                     __builtin_amdgcn_readlane(c.i, 16 * row)};
        if (better(r, best)) best = r;
    }
    return best;
}

// `row`: the E logits of token t (global memory, or LDS when the logits kernel selects right behind its sums).
// Lane l keeps the logits of experts l, l+64, ... (J of them; J * 64 >= E) in registers.  Called by all 64 lanes of a
// wavefront.  J is a template parameter so that layers with up to 64 experts do not walk eight slots per step.
// The selection is total: a NaN logit ranks as -inf (behind every number, ties to the lower index), so a token row
// that overflowed still gets k distinct, valid experts; its weights are computed from the logits as they are and
// come out NaN, which is what reaches the output of that token and of no other.
template <int J>
__device__ __forceinline__ void topk_one_token(const float* __restrict__ row, int t, int E, int k, int gate_fn,
                                               int norm, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
                                               int lane) {
    static_assert(J >= 1 && J <= kMaxExperts / kWave, "slots per lane");
    float v[J];
    unsigned avail = 0;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int e = j * kWave + lane;
        v[j] = 0.0f;
        if (e < E) {
            v[j] = row[e];
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
        c = wave_best(c);
        if ((c.i & (kWave - 1)) == lane) avail &= ~(1u << (c.i >> 6));
        // the logit behind the winning key, as stored (a NaN ranks as -inf but stays a NaN in the weights)
        float mine = v[0];
#pragma unroll
        for (int j = 1; j < J; ++j) mine = (c.i >> 6) == j ? v[j] : mine;
        // c comes out of wave_best through scalar registers: the winner's lane is uniform, so a lane read, not a shuffle
        const float cv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), c.i & (kWave - 1)));
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

}  // namespace moe355
