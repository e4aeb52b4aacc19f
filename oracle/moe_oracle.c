/*
 * CPU oracle for the fused MoE forward path.  TEST INFRASTRUCTURE ONLY -- see moe_oracle.h.
 *
 * Plain C11 + OpenMP, fp32 accumulation, built with -ffp-contract=off so that every fused multiply-add
 * in this file is one written as fmaf() on purpose.
 */
#include "moe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------------
 * Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11).  The reference
 * draws its synthetic operands from the same generator family through cuRAND (main.cu:22-31).
 * ---------------------------------------------------------------------------------------------- */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Element i of tensor `stream` under `seed` comes from Philox block i/4 with
 * counter = (block_lo, block_hi, stream_lo, stream_hi) and key = (seed_lo, seed_hi); words (0,1) and (2,3)
 * each feed one Box-Muller pair evaluated in double precision. */
void orc_fill_normal(float* dst, int64_t n, uint64_t seed, uint64_t stream, float mean, float stddev) {
    const int64_t blocks = (n + 3) / 4;
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    const double two_pi = 6.283185307179586476925286766559;
    const double inv32 = 1.0 / 4294967296.0;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < blocks; ++b) {
        uint32_t ctr[4] = {(uint32_t)b, (uint32_t)((uint64_t)b >> 32), (uint32_t)stream, (uint32_t)(stream >> 32)};
        uint32_t r[4];
        orc_philox4x32_10(ctr, key, r);
        double z[4];
        for (int h = 0; h < 2; ++h) {
            double u1 = ((double)r[2 * h] + 1.0) * inv32;
            double u2 = (double)r[2 * h + 1] * inv32;
            double rad = sqrt(-2.0 * log(u1));
            z[2 * h] = rad * cos(two_pi * u2);
            z[2 * h + 1] = rad * sin(two_pi * u2);
        }
        for (int j = 0; j < 4; ++j) {
            int64_t i = 4 * b + j;
            if (i < n) dst[i] = (float)((double)mean + (double)stddev * z[j]);
        }
    }
}

void orc_fill_uniform(float* dst, int64_t n, uint64_t seed, uint64_t stream) {
    const int64_t blocks = (n + 3) / 4;
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < blocks; ++b) {
        uint32_t ctr[4] = {(uint32_t)b, (uint32_t)((uint64_t)b >> 32), (uint32_t)stream, (uint32_t)(stream >> 32)};
        uint32_t r[4];
        orc_philox4x32_10(ctr, key, r);
        for (int j = 0; j < 4; ++j) {
            int64_t i = 4 * b + j;
            if (i < n) dst[i] = (float)((r[j] >> 8) * (1.0 / 16777216.0));
        }
    }
}

/* ------------------------------------------------------------------------------------------------
 * Storage formats.  bf16 is the reference's torch_dtype 2 (aristos_config.schema.json:54-58); e4m3 with
 * a 128x128-block fp32 scale is this build's extension (the reference rules fp8 out, combine.cuh:129-131).
 * ---------------------------------------------------------------------------------------------- */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t orc_f32_to_bf16(float v) {
    uint32_t u = f2u(v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7FFFu + ((u >> 16) & 1u);                                               /* round to nearest even */
    return (uint16_t)(u >> 16);
}
float orc_bf16_to_f32(uint16_t v) { return u2f((uint32_t)v << 16); }

/* OCP FP8 E4M3 ("e4m3fn"): 1-4-3, bias 7, no infinities, 0x7F/0xFF = NaN, largest finite 448.
 * Conversion rounds to nearest even and saturates to +-448. */
uint8_t orc_f32_to_e4m3(float v) {
    uint32_t u = f2u(v);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint8_t)(sign | 0x7Fu);
    float a = fabsf(v);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7Eu);
    if (a < 0.015625f) {                 /* below the smallest normal 2^-6: units of 2^-9 */
        int q = (int)rintf(a * 512.0f);  /* 0..8; 8 is the code of 2^-6 itself */
        return (uint8_t)(sign | (uint8_t)q);
    }
    int e;
    float m = frexpf(a, &e);             /* a = m * 2^e, m in [0.5,1) */
    int E = e - 1;                       /* a = (2m) * 2^E, 2m in [1,2) */
    int mant = (int)rintf((2.0f * m - 1.0f) * 8.0f);
    if (mant == 8) { mant = 0; E += 1; }
    int code = ((E + 7) << 3) | mant;
    if (code > 0x7E) code = 0x7E;
    return (uint8_t)(sign | (uint8_t)code);
}
float orc_e4m3_to_f32(uint8_t v) {
    int e = (v >> 3) & 0xF, m = v & 7;
    float a;
    if (e == 0xF && m == 7) return u2f(0x7FC00000u | ((uint32_t)(v & 0x80u) << 24));
    if (e == 0) a = ldexpf((float)m, -9);
    else a = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (v & 0x80u) ? -a : a;
}

/* IEEE binary16 (the reference's torch_dtype 3, aristos_config.schema.json:54-58): round to nearest even, overflow
 * to infinity, subnormals kept. */
uint16_t orc_f32_to_f16(float v) {
    const uint32_t u = f2u(v);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));   /* NaN, quieted */
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);          /* >= 65520 rounds to infinity (and inf itself) */
    if (a < 0x33000001u) return sign;                                  /* <= 2^-25 rounds to zero (ties to even) */
    int e = (int)(a >> 23) - 127;                                      /* unbiased exponent of the fp32 value */
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;                          /* 24-bit significand */
    int shift = e >= -14 ? 13 : 13 + (-14 - e);                        /* bits dropped; more for fp16 subnormals */
    uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1u;
    if (e >= -14) return (uint16_t)(sign + (uint16_t)(((uint32_t)(e + 15) << 10) + (q - 0x400u)));  /* carry may bump the exponent */
    return (uint16_t)(sign | (uint16_t)q);                              /* subnormal (q == 0x400 is the smallest normal) */
}
float orc_f16_to_f32(uint16_t v) {
    const uint32_t sign = ((uint32_t)v & 0x8000u) << 16;
    const int e = (v >> 10) & 0x1F;
    const uint32_t m = v & 0x3FFu;
    if (e == 0x1F) return u2f(sign | 0x7F800000u | (m << 13));
    if (e == 0) {
        const float a = ldexpf((float)m, -24);
        return (v & 0x8000u) ? -a : a;
    }
    return u2f(sign | ((uint32_t)(e + 112) << 23) | (m << 13));
}
void orc_round_f16(const float* src, uint16_t* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) dst[i] = orc_f32_to_f16(src[i]);
}
void orc_widen_f16(const uint16_t* src, float* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) dst[i] = orc_f16_to_f32(src[i]);
}

void orc_round_bf16(const float* src, uint16_t* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) dst[i] = orc_f32_to_bf16(src[i]);
}
void orc_widen_bf16(const uint16_t* src, float* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) dst[i] = orc_bf16_to_f32(src[i]);
}

/* One fp32 scale per 128x128 block of a row-major [N,K] matrix: scale = amax/448 (1 when the block is all
 * zero), q = e4m3(w / scale).  scales is [ceil(N/128), ceil(K/128)] row-major. */
void orc_quant_block128(const float* w, int64_t N, int64_t K, uint8_t* q, float* scales) {
    const int64_t nb = (N + 127) / 128, kb = (K + 127) / 128;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t bi = 0; bi < nb; ++bi) {
        for (int64_t bj = 0; bj < kb; ++bj) {
            const int64_t n1 = (bi * 128 + 128 < N) ? bi * 128 + 128 : N;
            const int64_t k1 = (bj * 128 + 128 < K) ? bj * 128 + 128 : K;
            float amax = 0.0f;
            for (int64_t n = bi * 128; n < n1; ++n)
                for (int64_t k = bj * 128; k < k1; ++k) {
                    float a = fabsf(w[n * K + k]);
                    if (a > amax) amax = a;
                }
            float s = amax > 0.0f ? amax / 448.0f : 1.0f;
            scales[bi * kb + bj] = s;
            for (int64_t n = bi * 128; n < n1; ++n)
                for (int64_t k = bj * 128; k < k1; ++k) q[n * K + k] = orc_f32_to_e4m3(w[n * K + k] / s);
        }
    }
}
void orc_dequant_block128(const uint8_t* q, const float* scales, int64_t N, int64_t K, float* w) {
    const int64_t kb = (K + 127) / 128;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) w[n * K + k] = orc_e4m3_to_f32(q[n * K + k]) * scales[(n / 128) * kb + k / 128];
}

/* Activation rows for the products of two e4m3 operands (build-defined, like the weight format above): one fp32 scale
 * per row and 128-wide block of columns, scale = amax/448 over that piece of the row (1 when it is all zero),
 * q = e4m3(x / scale).  x is [R,K] in fp32 (the widened bf16 activations), scales is [R, ceil(K/128)] row-major.
 * A NaN in a piece makes its amax comparison false everywhere, so the scale comes from the other elements and the NaN
 * becomes the e4m3 NaN code. */
void orc_quant_rows128(const float* x, int64_t R, int64_t K, uint8_t* q, float* scales) {
    const int64_t kb = (K + 127) / 128;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        for (int64_t bj = 0; bj < kb; ++bj) {
            const int64_t k1 = (bj * 128 + 128 < K) ? bj * 128 + 128 : K;
            float amax = 0.0f;
            for (int64_t k = bj * 128; k < k1; ++k) {
                float a = fabsf(x[r * K + k]);
                if (a > amax) amax = a;
            }
            float s = amax > 0.0f ? amax / 448.0f : 1.0f;
            scales[r * kb + bj] = s;
            for (int64_t k = bj * 128; k < k1; ++k) q[r * K + k] = orc_f32_to_e4m3(x[r * K + k] / s);
        }
    }
}
void orc_dequant_rows128(const uint8_t* q, const float* scales, int64_t R, int64_t K, float* x) {
    const int64_t kb = (K + 127) / 128;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r)
        for (int64_t k = 0; k < K; ++k) x[r * K + k] = orc_e4m3_to_f32(q[r * K + k]) * scales[r * kb + k / 128];
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------------
 * Capacity.  Build-defined (the reference defines CAP_FACTOR at CMakeLists.txt:204 and never reads it):
 * C = ceil(capacity_factor * S * k / E), evaluated in double precision.
 * ---------------------------------------------------------------------------------------------- */
int orc_capacity(double capacity_factor, int64_t S, int64_t k, int64_t E, int64_t* out) {
    if (E <= 0 || S < 0 || k <= 0 || !(capacity_factor > 0.0)) return 1;
    double c = ceil(capacity_factor * (double)(S * k) / (double)E);
    if (c < 1.0) c = 1.0;
    *out = (int64_t)c;
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Gate logits.  logits = X . Wg^T with Wg [E,H] row-major -- the (N,K) operand convention of the
 * reference GEMM (mma.cuh:417-419).  The reference has no gate; the summation order is build-defined so
 * that the integer routing results can be bit-exact on every machine:
 *   64 partial sums; partial p takes, in ascending k, every k with (k / 8) % 64 == p, each step being
 *   acc = fmaf(x[k], w[k], acc) in fp32; the partials are then folded pairwise, p with p+32, then +16,
 *   +8, +4, +2, +1; the bias (if any) is added last.
 * ---------------------------------------------------------------------------------------------- */
static inline float load_act(const void* p, int64_t i, int dtype) {
    if (dtype == ORC_F32 || dtype == ORC_TF32) return ((const float*)p)[i];
    return dtype == ORC_F16 ? orc_f16_to_f32(((const uint16_t*)p)[i]) : orc_bf16_to_f32(((const uint16_t*)p)[i]);
}
static inline void store_act(void* p, int64_t i, int dtype, float v) {
    if (dtype == ORC_F32 || dtype == ORC_TF32) ((float*)p)[i] = v;
    else if (dtype == ORC_F16) ((uint16_t*)p)[i] = orc_f32_to_f16(v);
    else ((uint16_t*)p)[i] = orc_f32_to_bf16(v);
}
static inline float round_act(float v, int dtype) {
    if (dtype == ORC_F32 || dtype == ORC_TF32) return v;
    return dtype == ORC_F16 ? orc_f16_to_f32(orc_f32_to_f16(v)) : orc_bf16_to_f32(orc_f32_to_bf16(v));
}
/* activations travel in the layer's storage type; the e4m3 layers keep bf16 activations; tf32 (the reference's
 * torch_dtype 1) is fp32 storage, computed here in full fp32 */
static inline int act_dtype_of(int dtype) {
    if (dtype == ORC_F32 || dtype == ORC_TF32) return ORC_F32;
    return dtype == ORC_F16 ? ORC_F16 : ORC_BF16;
}

static float gate_dot(const float* x, const float* w, int32_t H) {
    float acc[64];
    for (int p = 0; p < 64; ++p) acc[p] = 0.0f;
    for (int32_t k0 = 0; k0 < H; k0 += 8) {
        int p = (k0 / 8) % 64;
        int32_t k1 = k0 + 8 < H ? k0 + 8 : H;
        float a = acc[p];
        for (int32_t k = k0; k < k1; ++k) a = fmaf(x[k], w[k], a);
        acc[p] = a;
    }
    for (int off = 32; off >= 1; off >>= 1)
        for (int p = 0; p < off; ++p) acc[p] = acc[p] + acc[p + off];
    return acc[0];
}

void orc_gate_logits(const void* x, const void* gate_w, const float* gate_bias,
                     int32_t S, int32_t H, int32_t E, int32_t act_dtype, float* logits) {
    float* wf = (float*)malloc(sizeof(float) * (size_t)E * (size_t)H);
    for (int64_t i = 0; i < (int64_t)E * H; ++i) wf[i] = load_act(gate_w, i, act_dtype);
#pragma omp parallel
    {
        float* xf = (float*)malloc(sizeof(float) * (size_t)H);
#pragma omp for schedule(static)
        for (int32_t t = 0; t < S; ++t) {
            for (int32_t k = 0; k < H; ++k) xf[k] = load_act(x, (int64_t)t * H + k, act_dtype);
            for (int32_t e = 0; e < E; ++e) {
                float l = gate_dot(xf, wf + (int64_t)e * H, H);
                if (gate_bias) l = l + gate_bias[e];
                logits[(int64_t)t * E + e] = l;
            }
        }
        free(xf);
    }
    free(wf);
}

/* ------------------------------------------------------------------------------------------------
 * Top-k and gate weights.  Build-defined.  Selection is on the logits (softmax and sigmoid are monotone, so
 * the chosen set equals the one chosen on scores) by descending value, ties to the lower expert index.
 * Scores are fp32: softmax over all E experts, or elementwise sigmoid; with norm_topk the k selected
 * scores are divided by their sum (ascending rank).  The selection is total: a NaN logit ranks as -inf
 * (behind every number; among themselves and with real -inf, lower index first), so every token gets k
 * distinct valid experts; the scores are computed from the logits as stored, so such a token's weights
 * are NaN where the arithmetic says so.
 * ---------------------------------------------------------------------------------------------- */
static float topk_key(float v) { return v != v ? -INFINITY : v; }
void orc_topk(const float* logits, int32_t S, int32_t E, int32_t k, int32_t gate_fn, int32_t norm_topk,
              int32_t* topk_idx, float* topk_w) {
#pragma omp parallel
    {
        unsigned char* taken = (unsigned char*)malloc((size_t)E);
#pragma omp for schedule(static)
        for (int32_t t = 0; t < S; ++t) {
            const float* l = logits + (int64_t)t * E;
            memset(taken, 0, (size_t)E);
            for (int32_t r = 0; r < k; ++r) {
                int32_t best = -1;
                for (int32_t e = 0; e < E; ++e) {
                    if (taken[e]) continue;
                    if (best < 0 || topk_key(l[e]) > topk_key(l[best])) best = e;
                }
                taken[best] = 1;
                topk_idx[(int64_t)t * k + r] = best;
            }
            float sum = 0.0f;
            if (gate_fn == ORC_GATE_SOFTMAX) {
                float m = l[0];
                for (int32_t e = 1; e < E; ++e) if (l[e] > m) m = l[e];
                float denom = 0.0f;
                for (int32_t e = 0; e < E; ++e) denom = denom + expf(l[e] - m);
                for (int32_t r = 0; r < k; ++r) {
                    float p = expf(l[topk_idx[(int64_t)t * k + r]] - m) / denom;
                    topk_w[(int64_t)t * k + r] = p;
                    sum = sum + p;
                }
            } else {
                for (int32_t r = 0; r < k; ++r) {
                    float p = 1.0f / (1.0f + expf(-l[topk_idx[(int64_t)t * k + r]]));
                    topk_w[(int64_t)t * k + r] = p;
                    sum = sum + p;
                }
            }
            if (norm_topk)
                for (int32_t r = 0; r < k; ++r) topk_w[(int64_t)t * k + r] = topk_w[(int64_t)t * k + r] / sum;
        }
        free(taken);
    }
}

/* ------------------------------------------------------------------------------------------------
 * Router statistics for a load-balancing loss.  Build-defined: the reference parses is_training
 * (aristos_config.schema.json:20-23) and never reads it.  load[e] = assignments to expert e / (S*k) before
 * any drop; mean_prob[e] = mean over tokens of expert e's gate score (fp32 softmax over all E, or sigmoid),
 * summed in fp64 in ascending token order; aux_loss = E * sum_e load[e]*mean_prob[e].
 * ---------------------------------------------------------------------------------------------- */
void orc_router_stats(const float* logits, const int32_t* topk_idx, int32_t S, int32_t E, int32_t k, int32_t gate_fn,
                      float* load, float* mean_prob, float* aux_loss) {
    double* sum = (double*)calloc((size_t)E, sizeof(double));
    int64_t* cnt = (int64_t*)calloc((size_t)E, sizeof(int64_t));
    for (int32_t t = 0; t < S; ++t) {
        const float* l = logits + (int64_t)t * E;
        if (gate_fn == ORC_GATE_SOFTMAX) {
            float m = l[0];
            for (int32_t e = 1; e < E; ++e) if (l[e] > m) m = l[e];
            float denom = 0.0f;
            for (int32_t e = 0; e < E; ++e) denom = denom + expf(l[e] - m);
            for (int32_t e = 0; e < E; ++e) sum[e] += (double)(expf(l[e] - m) / denom);
        } else {
            for (int32_t e = 0; e < E; ++e) sum[e] += (double)(1.0f / (1.0f + expf(-l[e])));
        }
        for (int32_t r = 0; r < k; ++r) {
            const int32_t e = topk_idx[(int64_t)t * k + r];
            if (e >= 0 && e < E) cnt[e] += 1;   /* ids outside [0, E) are counted nowhere */
        }
    }
    double aux = 0.0;
    for (int32_t e = 0; e < E; ++e) {
        const double mp = sum[e] / (double)S, ld = (double)cnt[e] / ((double)S * (double)k);
        if (mean_prob) mean_prob[e] = (float)mp;
        if (load) load[e] = (float)ld;
        aux += mp * ld;
    }
    if (aux_loss) *aux_loss = (float)((double)E * aux);
    free(sum);
    free(cnt);
}

/* ------------------------------------------------------------------------------------------------
 * Slot assignment and capacity drop.  The reference only shows the consumer side: a tile of expert rows
 * carries tokenIndices[] and a valid-row count (combine.cuh:115,121-122,134,170).  Build-defined producer:
 * pairs are numbered p = t*k + r; slot[p] = number of earlier pairs routed to the same expert (a stable
 * counting sort by expert id); with drop != 0, pairs whose slot >= capacity are dropped (slot = -1).
 * expert_count is the kept count, expert_offset its exclusive scan, and kept pair p lives in packed row
 * expert_offset[e] + slot[p]; token_indices[row] = t.  A pair whose expert id lies outside [0, E) (only a
 * caller-supplied topk_idx can hold one) is dropped like a pair over capacity.
 * ---------------------------------------------------------------------------------------------- */
void orc_route(const int32_t* topk_idx, int32_t S, int32_t k, int32_t E, int32_t drop, int64_t capacity,
               int32_t* slot, int32_t* expert_count, int32_t* expert_offset, int32_t* token_indices,
               int32_t* pair_row) {
    const int64_t A = (int64_t)S * k;
    int32_t* seen = (int32_t*)calloc((size_t)E, sizeof(int32_t));
    for (int64_t p = 0; p < A; ++p) {
        int32_t e = topk_idx[p];
        if (e < 0 || e >= E) { slot[p] = -1; continue; }
        int32_t s = seen[e]++;
        slot[p] = (drop && s >= capacity) ? -1 : s;
    }
    int32_t run = 0;
    for (int32_t e = 0; e < E; ++e) {
        int32_t c = seen[e];
        if (drop && c > capacity) c = (int32_t)capacity;
        expert_count[e] = c;
        expert_offset[e] = run;
        run += c;
    }
    for (int64_t p = 0; p < A; ++p) {
        int32_t row = slot[p] < 0 ? -1 : expert_offset[topk_idx[p]] + slot[p];
        if (pair_row) pair_row[p] = row;
        if (token_indices && row >= 0) token_indices[row] = (int32_t)(p / k);
    }
    if (token_indices)
        for (int64_t r = run; r < A; ++r) token_indices[r] = -1;
    free(seen);
}

/* ------------------------------------------------------------------------------------------------
 * Dot products in fp32 with sixteen interleaved partial sums (so the compiler can vectorise without
 * being allowed to reassociate), folded in index order at the end.
 * ---------------------------------------------------------------------------------------------- */
static inline float fold16(const float* acc) {
    float s = 0.0f;
    for (int j = 0; j < 16; ++j) s = s + acc[j];
    return s;
}
static float dot_f32(const float* a, const float* b, int64_t K) {
    float acc[16] = {0};
    int64_t k = 0;
    for (; k + 16 <= K; k += 16)
        for (int j = 0; j < 16; ++j) acc[j] = acc[j] + a[k + j] * b[k + j];
    for (int j = 0; k < K; ++k, ++j) acc[j] = acc[j] + a[k] * b[k];
    return fold16(acc);
}
static float dot_bf16(const float* a, const uint16_t* b, int64_t K) {
    float acc[16] = {0};
    int64_t k = 0;
    for (; k + 16 <= K; k += 16)
        for (int j = 0; j < 16; ++j) acc[j] = acc[j] + a[k + j] * u2f((uint32_t)b[k + j] << 16);
    for (int j = 0; k < K; ++k, ++j) acc[j] = acc[j] + a[k] * u2f((uint32_t)b[k] << 16);
    return fold16(acc);
}
static float dot_f16(const float* a, const uint16_t* b, int64_t K) {
    float acc[16] = {0};
    int64_t k = 0;
    for (; k + 16 <= K; k += 16)
        for (int j = 0; j < 16; ++j) acc[j] = acc[j] + a[k + j] * orc_f16_to_f32(b[k + j]);
    for (int j = 0; k < K; ++k, ++j) acc[j] = acc[j] + a[k] * orc_f16_to_f32(b[k]);
    return fold16(acc);
}
static float e4m3_lut[256];
static int e4m3_lut_ready = 0;
static void e4m3_lut_init(void) {
    if (e4m3_lut_ready) return;
#pragma omp critical(orc_lut)
    {
        if (!e4m3_lut_ready) {
            for (int i = 0; i < 256; ++i) {
                float f = orc_e4m3_to_f32((uint8_t)i);
                e4m3_lut[i] = (f != f) ? 0.0f : f;
            }
            e4m3_lut_ready = 1;
        }
    }
}
/* y = sum over 128-wide k blocks of scale[kb] * (fp32 dot of that block) */
static float dot_fp8(const float* a, const uint8_t* q, const float* scale_row, int64_t K) {
    float y = 0.0f;
    for (int64_t k0 = 0, kb = 0; k0 < K; k0 += 128, ++kb) {
        int64_t k1 = k0 + 128 < K ? k0 + 128 : K;
        float acc[16] = {0};
        int64_t k = k0;
        for (; k + 16 <= k1; k += 16)
            for (int j = 0; j < 16; ++j) acc[j] = acc[j] + a[k + j] * e4m3_lut[q[k + j]];
        for (int j = 0; k < k1; ++k, ++j) acc[j] = acc[j] + a[k] * e4m3_lut[q[k]];
        y = y + scale_row[kb] * fold16(acc);
    }
    return y;
}
/* row n of a [N,K] weight matrix in storage dtype `dtype`, dotted with the fp32 vector a */
static inline float dot_w(const float* a, const void* W, const float* scales, int64_t n, int64_t K, int dtype) {
    if (dtype == ORC_F32 || dtype == ORC_TF32) return dot_f32(a, (const float*)W + n * K, K);
    if (dtype == ORC_BF16) return dot_bf16(a, (const uint16_t*)W + n * K, K);
    if (dtype == ORC_F16) return dot_f16(a, (const uint16_t*)W + n * K, K);
    const int64_t kb = (K + 127) / 128;
    return dot_fp8(a, (const uint8_t*)W + n * K, scales + (n / 128) * kb, K);
}

static inline float act_apply(float v, int act) {
    switch (act) {
        case ORC_ACT_RELU: return v < 0.0f ? 0.0f : v;   /* a NaN stays a NaN, as with the reference's __hfma_relu */
        case ORC_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
        default: return v;
    }
}
static inline float silu(float v) { return v / (1.0f + expf(-v)); }

/* ------------------------------------------------------------------------------------------------
 * The reference tile GEMM contract (mma.cuh:46-179): C = act(A . B^T + bias) with A (M,K), B (N,K) and
 * C (M,N) row-major, bias (1,N) broadcast over rows (mma.cuh:415-427), fp32 accumulation and one cast to
 * the storage type on store (mma.cuh:59,108-111,151); epilogue order is add, then activate
 * (processor/tiling.cuh:29-38).
 * ---------------------------------------------------------------------------------------------- */
void orc_gemm_bias_act(const void* A, const void* B, const void* bias, void* C,
                       int64_t M, int64_t N, int64_t K, int32_t dtype, int32_t act) {
#pragma omp parallel
    {
        float* a = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int64_t m = 0; m < M; ++m) {
            for (int64_t k = 0; k < K; ++k) a[k] = load_act(A, m * K + k, dtype);
            for (int64_t n = 0; n < N; ++n) {
                float v = dot_w(a, B, NULL, n, K, dtype);
                if (bias) v = v + load_act(bias, n, dtype);
                store_act(C, m * N + n, dtype, act_apply(v, act));
            }
        }
        free(a);
    }
}

/* ------------------------------------------------------------------------------------------------
 * Grouped products over packed expert-major rows (rows [offset[e], offset[e] + count[e]) belong to expert
 * e), the building blocks of a backward pass.  Build-defined: the reference parses a training flag
 * (aristos_config.schema.json:20-23) and holds no backward code.  Both keep the forward GEMM's contract:
 * fp32 accumulation, one rounding to the storage type on store.
 *   orc_expert_gemm:  out[r,:] = act(a[r,:K] . w[e]^T + bias[e]),   w [E,N,K], bias [E,N] or NULL
 *   orc_expert_wgrad: dw[e] [N,K] = sum over r of expert e, ascending, of dy[r,:N]^T a[r,:K]
 * Rows outside every expert's range are left untouched.
 * ---------------------------------------------------------------------------------------------- */
void orc_expert_gemm(const void* a_rows, const void* w, const void* bias, const int32_t* count, const int32_t* offset,
                     int32_t E, int64_t N, int64_t K, int32_t dtype, int32_t act, void* out_rows) {
    const size_t el = (dtype == ORC_F32 || dtype == ORC_TF32) ? 4 : 2;
    for (int32_t e = 0; e < E; ++e) {
        if (count[e] <= 0) continue;
        orc_gemm_bias_act((const char*)a_rows + (size_t)offset[e] * K * el, (const char*)w + (size_t)e * N * K * el,
                          bias ? (const char*)bias + (size_t)e * N * el : NULL,
                          (char*)out_rows + (size_t)offset[e] * N * el, count[e], N, K, dtype, act);
    }
}

void orc_expert_wgrad(const void* dy_rows, const void* a_rows, const int32_t* count, const int32_t* offset, int32_t E,
                      int64_t N, int64_t K, int32_t dtype, void* dw) {
    const int adt = act_dtype_of(dtype);
    for (int32_t e = 0; e < E; ++e) {
        const int64_t r0 = offset[e], r1 = r0 + (count[e] > 0 ? count[e] : 0);
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            for (int64_t k = 0; k < K; ++k) {
                float acc = 0.0f;
                for (int64_t r = r0; r < r1; ++r)
                    acc = fmaf(load_act(dy_rows, r * N + n, adt), load_act(a_rows, r * K + k, adt), acc);
                store_act(dw, ((int64_t)e * N + n) * K + k, adt, acc);
            }
        }
    }
}

/* The elementwise and reduction steps of a backward pass (build-defined, as the grouped products above).
 *   orc_act_backward:     du = dh * act'(u) (ReLU: 1 for u > 0; GELU: Phi(u) + u phi(u)), or for SwiGLU
 *                         (h = silu(g) u): du = dh silu(g), dg = dh u s (1 + g (1 - s)) with s = sigmoid(g);
 *                         fp32 arithmetic on the stored values, one rounding on store
 *   orc_bias_grad:        db[e,n] = sum over expert e's rows, ascending, of dy[r,n] in fp32, rounded once
 *   orc_combine_backward: dy[row(t,r),:] = w[t,r] * dout[t,:] (rounded once); dw[t,r] = <dout[t,:], y[row(t,r),:]> in
 *                         fp32, ascending column; dropped pairs get dw = 0 and no row */
void orc_act_backward(const void* dh, const void* u, const void* g, int64_t rows, int64_t I, int32_t dtype, int32_t act,
                      void* du, void* dg) {
    const int adt = act_dtype_of(dtype);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows * I; ++i) {
        const float d = load_act(dh, i, adt), uv = load_act(u, i, adt);
        if (act == ORC_ACT_SWIGLU) {
            const float gv = load_act(g, i, adt);
            const float sg = 1.0f / (1.0f + expf(-gv));
            store_act(du, i, adt, d * (gv * sg));
            store_act(dg, i, adt, d * uv * (sg * (1.0f + gv * (1.0f - sg))));
        } else if (act == ORC_ACT_GELU) {
            const float cdf = 0.5f * (1.0f + erff(uv * 0.70710678118654752440f));
            const float pdf = 0.39894228040143267794f * expf(-0.5f * uv * uv);
            store_act(du, i, adt, d * (cdf + uv * pdf));
        } else {
            store_act(du, i, adt, uv > 0.0f ? d : 0.0f);
        }
    }
}

void orc_bias_grad(const void* dy_rows, const int32_t* count, const int32_t* offset, int32_t E, int64_t N, int32_t dtype,
                   void* db) {
    const int adt = act_dtype_of(dtype);
    for (int32_t e = 0; e < E; ++e)
        for (int64_t n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int64_t r = offset[e]; r < offset[e] + (count[e] > 0 ? count[e] : 0); ++r) acc = acc + load_act(dy_rows, r * N + n, adt);
            store_act(db, (int64_t)e * N + n, adt, acc);
        }
}

void orc_combine_backward(const void* dout, const void* y_rows, const int32_t* pair_row, const float* topk_w, int32_t S,
                          int32_t k, int32_t H, int32_t dtype, void* dy_rows, float* dw) {
    const int adt = act_dtype_of(dtype);
#pragma omp parallel for schedule(static)
    for (int32_t t = 0; t < S; ++t)
        for (int32_t r = 0; r < k; ++r) {
            const int32_t row = pair_row[(int64_t)t * k + r];
            float acc = 0.0f;
            if (row >= 0) {
                const float w = topk_w[(int64_t)t * k + r];
                for (int32_t j = 0; j < H; ++j) {
                    const float d = load_act(dout, (int64_t)t * H + j, adt);
                    store_act(dy_rows, (int64_t)row * H + j, adt, w * d);
                    acc = fmaf(d, load_act(y_rows, (int64_t)row * H + j, adt), acc);
                }
            }
            dw[(int64_t)t * k + r] = acc;
        }
}

/* One expert FFN row: the two chained GEMMs of the reference's task graph (scheduling.cuh:212-222), the
 * intermediate rounded to the storage type between them (mma.cuh:108-109).  GELU is the exact erf form,
 * SwiGLU is silu(x.Wg^T + bg) * (x.Wu^T + bu); both are this build's extensions of hidden_act.
 * h must hold I floats. */
static void ffn_one_row(const orc_cfg* c, const float* xrow, const orc_weights* w, int32_t e, float* h,
                        void* y_row, int parallel_inner) {
    const int adt = act_dtype_of(c->dtype);
    const int64_t H = c->H, I = c->I;
    const int64_t kbH = (H + 127) / 128, kbI = (I + 127) / 128, nbI = (I + 127) / 128, nbH = (H + 127) / 128;
    const size_t wel = (c->dtype == ORC_F32 || c->dtype == ORC_TF32) ? 4 : (c->dtype == ORC_FP8 ? 1 : 2);
    const char* Wu = (const char*)w->w_up + (size_t)e * I * H * wel;
    const char* Wg = w->w_gate ? (const char*)w->w_gate + (size_t)e * I * H * wel : NULL;
    const char* Wd = (const char*)w->w_down + (size_t)e * H * I * wel;
    const float* su = w->s_up ? w->s_up + (int64_t)e * nbI * kbH : NULL;
    const float* sg = w->s_gate ? w->s_gate + (int64_t)e * nbI * kbH : NULL;
    const float* sd = w->s_down ? w->s_down + (int64_t)e * nbH * kbI : NULL;
#pragma omp parallel for schedule(static) if (parallel_inner)
    for (int64_t n = 0; n < I; ++n) {
        float u = dot_w(xrow, Wu, su, n, H, c->dtype);
        if (w->b_up) u = u + load_act(w->b_up, (int64_t)e * I + n, adt);
        float v;
        if (c->act == ORC_ACT_SWIGLU) {
            float g = dot_w(xrow, Wg, sg, n, H, c->dtype);
            if (w->b_gate) g = g + load_act(w->b_gate, (int64_t)e * I + n, adt);
            v = silu(g) * u;
        } else {
            v = act_apply(u, c->act);
        }
        h[n] = round_act(v, adt);
    }
#pragma omp parallel for schedule(static) if (parallel_inner)
    for (int64_t j = 0; j < H; ++j) {
        float v = dot_w(h, Wd, sd, j, I, c->dtype);
        if (w->b_down) v = v + load_act(w->b_down, (int64_t)e * H + j, adt);
        store_act(y_row, j, adt, v);
    }
}

void orc_ffn_rows(const orc_cfg* cfg, const void* x, const orc_weights* w, const int32_t* tokens,
                  const int32_t* experts, int64_t n_rows, void* y_rows) {
    const int adt = act_dtype_of(cfg->dtype);
    const size_t ael = adt == ORC_F32 ? 4 : 2;
    if (cfg->dtype == ORC_FP8) e4m3_lut_init();
    const int outer = n_rows >= 2 * (int64_t)orc_num_threads();
#pragma omp parallel if (outer)
    {
        float* xrow = (float*)malloc(sizeof(float) * (size_t)cfg->H);
        float* h = (float*)malloc(sizeof(float) * (size_t)cfg->I);
#pragma omp for schedule(dynamic, 1)
        for (int64_t r = 0; r < n_rows; ++r) {
            for (int32_t k = 0; k < cfg->H; ++k) xrow[k] = load_act(x, (int64_t)tokens[r] * cfg->H + k, adt);
            ffn_one_row(cfg, xrow, w, experts[r], h, (char*)y_rows + (size_t)r * cfg->H * ael, !outer);
        }
        free(xrow);
        free(h);
    }
}

/* ------------------------------------------------------------------------------------------------
 * Combine.  The reference scatters expert rows to activations[tokenIdx,:] by copy (top-1) or by atomic
 * add (top-k), unweighted (combine.cuh:170-186).  Build-defined: out[t,:] = sum over ranks r, ascending,
 * of w[t,r] * y[row(t,r),:] in fp32 with one rounding to the output type; dropped pairs contribute 0.
 * ---------------------------------------------------------------------------------------------- */
void orc_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w,
                 int32_t S, int32_t k, int32_t H, int32_t act_dtype, void* out) {
#pragma omp parallel for schedule(static)
    for (int32_t t = 0; t < S; ++t) {
        for (int32_t j = 0; j < H; ++j) {
            float acc = 0.0f;
            for (int32_t r = 0; r < k; ++r) {
                int32_t row = pair_row[(int64_t)t * k + r];
                if (row < 0) continue;
                acc = acc + topk_w[(int64_t)t * k + r] * load_act(y_rows, (int64_t)row * H + j, act_dtype);
            }
            store_act(out, (int64_t)t * H + j, act_dtype, acc);
        }
    }
}

/* The whole layer on all S tokens. */
void orc_forward(const orc_cfg* cfg, const void* x, const orc_weights* w, void* out,
                 int32_t* topk_idx, float* topk_w, int32_t* slot, int32_t* expert_count,
                 int32_t* expert_offset, int32_t* token_indices) {
    const int adt = act_dtype_of(cfg->dtype);
    const int64_t A = (int64_t)cfg->S * cfg->k;
    float* logits = (float*)malloc(sizeof(float) * (size_t)cfg->S * cfg->E);
    int32_t* pair_row = (int32_t*)malloc(sizeof(int32_t) * (size_t)A);
    int32_t* tok = (int32_t*)malloc(sizeof(int32_t) * (size_t)A);
    int32_t* exps = (int32_t*)malloc(sizeof(int32_t) * (size_t)A);
    orc_gate_logits(x, w->gate_w, w->gate_bias, cfg->S, cfg->H, cfg->E, adt, logits);
    orc_topk(logits, cfg->S, cfg->E, cfg->k, cfg->gate_fn, cfg->norm_topk, topk_idx, topk_w);
    orc_route(topk_idx, cfg->S, cfg->k, cfg->E, cfg->drop, cfg->capacity, slot, expert_count, expert_offset,
              tok, pair_row);
    int64_t kept = 0;
    for (int32_t e = 0; e < cfg->E; ++e) kept += expert_count[e];
    for (int32_t e = 0; e < cfg->E; ++e)
        for (int32_t i = 0; i < expert_count[e]; ++i) exps[expert_offset[e] + i] = e;
    void* y = malloc((size_t)(kept > 0 ? kept : 1) * cfg->H * (adt == ORC_F32 ? 4 : 2));
    orc_ffn_rows(cfg, x, w, tok, exps, kept, y);
    orc_combine(y, pair_row, topk_w, cfg->S, cfg->k, cfg->H, adt, out);
    if (token_indices) memcpy(token_indices, tok, sizeof(int32_t) * (size_t)A);
    free(y); free(exps); free(tok); free(pair_row); free(logits);
}

/* The layer output for a chosen subset of tokens, given the routing result: what a full-size parity check
 * can afford.  out_rows is [n_tokens, H] in the activation dtype. */
void orc_forward_tokens(const orc_cfg* cfg, const void* x, const orc_weights* w,
                        const int32_t* topk_idx, const float* topk_w, const int32_t* slot,
                        const int32_t* tokens, int64_t n_tokens, void* out_rows) {
    const int adt = act_dtype_of(cfg->dtype);
    const int64_t H = cfg->H;
    const size_t ael = adt == ORC_F32 ? 4 : 2;
    if (cfg->dtype == ORC_FP8) e4m3_lut_init();
    float* xrow = (float*)malloc(sizeof(float) * (size_t)H);
    float* h = (float*)malloc(sizeof(float) * (size_t)cfg->I);
    float* acc = (float*)malloc(sizeof(float) * (size_t)H);
    void* y = malloc((size_t)H * ael);
    for (int64_t i = 0; i < n_tokens; ++i) {
        const int32_t t = tokens[i];
        for (int64_t j = 0; j < H; ++j) { acc[j] = 0.0f; xrow[j] = load_act(x, (int64_t)t * H + j, adt); }
        for (int32_t r = 0; r < cfg->k; ++r) {
            const int64_t p = (int64_t)t * cfg->k + r;
            if (slot[p] < 0) continue;
            ffn_one_row(cfg, xrow, w, topk_idx[p], h, y, 1);
            for (int64_t j = 0; j < H; ++j) acc[j] = acc[j] + topk_w[p] * load_act(y, j, adt);
        }
        for (int64_t j = 0; j < H; ++j) store_act(out_rows, i * H + j, adt, acc[j]);
    }
    free(y); free(acc); free(h); free(xrow);
}
