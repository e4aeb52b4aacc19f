/*
 * CPU oracle for the fused MoE forward path (gate -> slot assignment -> expert FFN -> combine).
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product library links, loads or calls this file; it exists so
 * tests, the smoke check and the benchmark's CPU-baseline leg have an independent statement of the layer.
 *
 * The reference (osayamenja/cuPlayground) only fixes fragments of this path; each function below cites the
 * fragment it follows and says where the semantics are defined by this build instead.  Pinning status:
 *   - orc_philox4x32_10        pinned by the Random123 known-answer vectors (tests/test_oracle_rng.py)
 *   - bf16 / fp16 / e4m3 conversions  pinned by exhaustive code-point round trips and torch / numpy CPU casts
 *   - orc_gemm_bias_act        pinned by the reference driver's known-answer corner (mma.cuh:394-411)
 *                              and by float64 triple loops on random shapes
 *   - orc_gate_logits          pinned against float64 dot products (value) and against a pure-Python
 *                              restatement of the summation order (bit pattern)
 *   - orc_topk                 pinned by brute-force full sorts with key (score desc, index asc)
 *   - orc_router_stats         pinned by closed forms (uniform router: 1/E, 1/E, loss 1; one-hot router) and
 *                              a float64 numpy restatement
 *   - orc_route                pinned by a stable sort of the flattened expert ids and by its invariants
 *   - orc_combine              pinned by the reference driver's identity case (combine.cuh:220-231),
 *                              permutation and linearity properties
 *   - orc_forward*             pinned by the dense-mixture equivalence in float64
 *   - orc_expert_gemm / orc_expert_wgrad  pinned by float64 einsums per expert, by one-hot rows that select
 *                              single weight columns / operand rows, and by the adjoint identity
 *                              <dY, X.W^T> = <dY^T.X, W> = <dY.W, X> (tests/test_oracle_backward.py)
 *   - orc_act_backward / orc_bias_grad / orc_combine_backward  pinned by central differences of the float64
 *                              activations, float64 column sums, and the adjoint identity of the combine
 * Reference parity of gate / top-k / capacity / SwiGLU / fp8 scaling is unpinned by construction: the
 * reference holds no code for them.
 */
#ifndef MOE_ORACLE_H
#define MOE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* storage dtype codes: the reference's torch_dtype enum (aristos_config.schema.json:54-58) plus 4 = e4m3 */
enum { ORC_F32 = 0, ORC_TF32 = 1, ORC_BF16 = 2, ORC_F16 = 3, ORC_FP8 = 4 };
/* hidden_act codes (aristos_config.schema.json:24-28) plus 2 = SwiGLU; ORC_ACT_NONE is for the bare GEMM */
enum { ORC_ACT_RELU = 0, ORC_ACT_GELU = 1, ORC_ACT_SWIGLU = 2, ORC_ACT_NONE = 3 };
enum { ORC_GATE_SOFTMAX = 0, ORC_GATE_SIGMOID = 1 };

typedef struct orc_cfg {
    int32_t S, H, I, E, k;
    int32_t act;        /* ORC_ACT_* */
    int32_t dtype;      /* ORC_F32 / ORC_BF16 / ORC_FP8 */
    int32_t gate_fn;    /* ORC_GATE_* */
    int32_t norm_topk;  /* renormalise the k selected scores to sum 1 */
    int32_t drop;       /* drop pairs whose slot >= capacity */
    int64_t capacity;   /* rows per expert when drop != 0 */
} orc_cfg;

typedef struct orc_weights {
    const void* gate_w;     /* [E,H]  activation dtype (f32 or bf16) */
    const float* gate_bias; /* [E] or NULL */
    const void* w_up;       /* [E,I,H] storage dtype (f32 / bf16 / e4m3 bytes) */
    const void* w_gate;     /* [E,I,H] SwiGLU only */
    const void* w_down;     /* [E,H,I] */
    const void* b_up;       /* [E,I] activation dtype or NULL */
    const void* b_gate;     /* [E,I] or NULL */
    const void* b_down;     /* [E,H] or NULL */
    const float* s_up;      /* fp8 only: [E, I/128, H/128] */
    const float* s_gate;
    const float* s_down;    /* fp8 only: [E, H/128, I/128] */
} orc_weights;

/* ---- seeded synthetic data ---- */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
void orc_fill_normal(float* dst, int64_t n, uint64_t seed, uint64_t stream, float mean, float stddev);
void orc_fill_uniform(float* dst, int64_t n, uint64_t seed, uint64_t stream);

/* ---- storage formats ---- */
uint16_t orc_f32_to_bf16(float v);
float orc_bf16_to_f32(uint16_t v);
uint8_t orc_f32_to_e4m3(float v);
float orc_e4m3_to_f32(uint8_t v);
uint16_t orc_f32_to_f16(float v);
float orc_f16_to_f32(uint16_t v);
void orc_round_f16(const float* src, uint16_t* dst, int64_t n);
void orc_widen_f16(const uint16_t* src, float* dst, int64_t n);
void orc_round_bf16(const float* src, uint16_t* dst, int64_t n);
void orc_widen_bf16(const uint16_t* src, float* dst, int64_t n);
void orc_quant_block128(const float* w, int64_t N, int64_t K, uint8_t* q, float* scales);
void orc_dequant_block128(const uint8_t* q, const float* scales, int64_t N, int64_t K, float* w);
/* the same per (row, 128 columns): the activation operand of a product of two e4m3 matrices */
void orc_quant_rows128(const float* x, int64_t R, int64_t K, uint8_t* q, float* scales);
void orc_dequant_rows128(const uint8_t* q, const float* scales, int64_t R, int64_t K, float* x);

/* ---- the path ---- */
int orc_capacity(double capacity_factor, int64_t S, int64_t k, int64_t E, int64_t* out);
void orc_gate_logits(const void* x, const void* gate_w, const float* gate_bias,
                     int32_t S, int32_t H, int32_t E, int32_t act_dtype, float* logits);
void orc_topk(const float* logits, int32_t S, int32_t E, int32_t k, int32_t gate_fn, int32_t norm_topk,
              int32_t* topk_idx, float* topk_w);
void orc_router_stats(const float* logits, const int32_t* topk_idx, int32_t S, int32_t E, int32_t k, int32_t gate_fn,
                      float* load, float* mean_prob, float* aux_loss);
void orc_route(const int32_t* topk_idx, int32_t S, int32_t k, int32_t E, int32_t drop, int64_t capacity,
               int32_t* slot, int32_t* expert_count, int32_t* expert_offset, int32_t* token_indices,
               int32_t* pair_row);
void orc_gemm_bias_act(const void* A, const void* B, const void* bias, void* C,
                       int64_t M, int64_t N, int64_t K, int32_t dtype, int32_t act);
void orc_expert_gemm(const void* a_rows, const void* w, const void* bias, const int32_t* count, const int32_t* offset,
                     int32_t E, int64_t N, int64_t K, int32_t dtype, int32_t act, void* out_rows);
void orc_expert_wgrad(const void* dy_rows, const void* a_rows, const int32_t* count, const int32_t* offset, int32_t E,
                      int64_t N, int64_t K, int32_t dtype, void* dw);
void orc_act_backward(const void* dh, const void* u, const void* g, int64_t rows, int64_t I, int32_t dtype, int32_t act,
                      void* du, void* dg);
void orc_bias_grad(const void* dy_rows, const int32_t* count, const int32_t* offset, int32_t E, int64_t N, int32_t dtype,
                   void* db);
void orc_combine_backward(const void* dout, const void* y_rows, const int32_t* pair_row, const float* topk_w, int32_t S,
                          int32_t k, int32_t H, int32_t dtype, void* dy_rows, float* dw);
void orc_ffn_rows(const orc_cfg* cfg, const void* x, const orc_weights* w, const int32_t* tokens,
                  const int32_t* experts, int64_t n_rows, void* y_rows);
void orc_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w,
                 int32_t S, int32_t k, int32_t H, int32_t act_dtype, void* out);
void orc_forward(const orc_cfg* cfg, const void* x, const orc_weights* w, void* out,
                 int32_t* topk_idx, float* topk_w, int32_t* slot, int32_t* expert_count,
                 int32_t* expert_offset, int32_t* token_indices);
void orc_forward_tokens(const orc_cfg* cfg, const void* x, const orc_weights* w,
                        const int32_t* topk_idx, const float* topk_w, const int32_t* slot,
                        const int32_t* tokens, int64_t n_tokens, void* out_rows);
int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
