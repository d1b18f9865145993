/* CPU oracle for the quantized matvec / MoE hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing that ships (the HIP library, the host-side operator API) may include, link or
 * call this; only tests/, the smoke check and the CPU-baseline leg of the benchmark use it, as the checker.
 *
 * It restates, in plain C, the reference's CPU path for this computation:
 *   block geometry        src/kernels/quant_types.hpp:8-43
 *   dequant_row           tests/ref/dequant.cpp:34-120
 *   matvec_ref/ref_matvec tests/ref/dequant.cpp:122-131, tests/quant_test_util.hpp:29-42
 *   SwiGLU with clamps    tests/test_quant_moe.mm:14-18 (kernel form: src/kernels/quant_moe.metal:23-27)
 *   MoE decode reference  tests/test_quant_moe.mm:64-93
 *   MoE prefill reference tests/test_quant_moe_prefill.mm:25-47,186-212; reduce order
 *                         src/kernels/quant_moe_prefill.metal:330-344
 *   router, route lists   tests/ref/arch_ref.cpp:97-130 (kernels: src/kernels/arch_router.metal:26-160)
 *   rmsnorm               tests/ref/arch_ref.cpp:66-71
 *
 * Pinned by: bit-equality with the reference's own dequant.cpp compiled from /root/reference (oracle/_ref, and the
 * golden fixtures written from it under tests/golden/), closed-form known answers per format, codebook invariants,
 * and numpy float64 dots on tiny cases (tests/test_oracle.py). Router and route lists: equality with the reference's
 * arch_ref.cpp compiled the same way, softplus / tie / normalisation known answers, and a stable numpy argsort.
 */
#ifndef MSQ_ORACLE_H
#define MSQ_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (src/kernels/quant_types.hpp:9-11) */
enum {
  ORC_F32 = 0, ORC_F16 = 1, ORC_Q8_0 = 8, ORC_Q5_K = 13, ORC_Q6_K = 14, ORC_IQ2_XXS = 16, ORC_IQ1_S = 19,
  ORC_IQ4_NL = 20, ORC_BF16 = 30
};

int orc_block_elems(int t);
size_t orc_block_bytes(int t);
size_t orc_row_bytes(int t, int64_t cols);

float orc_fp16_to_f32(uint16_t h);
uint16_t orc_f32_to_fp16(float f); /* round to nearest even */
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f); /* round to nearest even */

/* codebook access (for invariant tests): writes 8 elements of entry i */
void orc_iq1s_entry(int i, int8_t out[8]);
void orc_iq2xxs_entry(int i, uint8_t out[8]);
uint8_t orc_ksign(int i);

/* dst[n] = dequantized elements; n multiple of the block size. Returns 0, or -1 for an unknown type. */
int orc_dequant_row(int t, const void* src, float* dst, int64_t n);

/* y[r] = sum_c (double)deq(W[r])[c] * x[c]; mag[r] = sum |w x|; wn2[r] = sum w^2 (any output may be NULL).
 * groups > 1: block-diagonal, row r reads x + (r / (rows/groups)) * cols. Rows are split over nthreads threads. */
int orc_matvec(int t, const void* W, int rows, int cols, const float* x, int groups, double* y, double* mag,
               double* wn2, int nthreads);

/* silu(min(g,10)) * clamp(u,-10,10) * w in double */
double orc_swiglu(double g, double u, double w);

/* One-token MoE layer reference. Expert e < n_routed uses (t_gu, t_down) and weight wts[e]; e == n_routed is the
 * shared expert (t_shared, weight 1) when has_shared. gate/up: inter rows x dim cols, down: dim rows x inter cols.
 * h_out[(n_routed+1) * inter] (float, as the kernel stores it), y[dim] += result, ymag[dim] = |y0| + sum |wd h|
 * (error scale), hscale[(n_routed+1)*inter] = |w| (sum|g terms| + sum|u terms|). Outputs other than y may be NULL. */
int orc_moe_decode(int t_gu, int t_down, int t_shared, int n_routed, int has_shared, int dim, int inter,
                   const void* const* gate, const void* const* up, const void* const* down, /* [n_routed+1] */
                   const float* wts, const float* x, double* y, double* ymag, float* h_out, double* hscale,
                   int nthreads);

/* Prefill MoE reference for a token subset. Routing is expert-sorted: expert j owns entries [offs[j], offs[j+1]) of
 * tok[] / wt[]. For each checked token chk[q] the function accumulates into Y[q*dim ..] (double, preloaded by the
 * caller with Y0) the shared expert (if any) and every routed entry of that token, and into Ymag the error scale.
 * x_round: 0 = pure F32 inputs, 1 = X and H rounded to fp16 (weights exact), 2 = X and H rounded to bf16. */
int orc_moe_prefill(int t_gu, int t_down, int t_shared, int n_tokens, int n_exp, int has_shared, int dim, int inter,
                    const void* const* gate, const void* const* up, const void* const* down, /* [n_exp+1] */
                    const int* offs, const int* tok, const float* wt, const float* X, const int* chk, int n_chk,
                    int x_round, double* Y, double* Ymag, int nthreads);

/* Seeded inputs (splitmix64 + Box-Muller in double; tests/dec_synth.hpp:25-31 uses the same integer generator).
 * Block filler follows ref::random_blocks' recipe (tests/ref/dequant.cpp:133-159): random bytes, then every block's
 * fp16 scale(s) overwritten with sc = scale*(0.5+0.5|N(0,1)|) (Q8_0 sc/16, Q5_K d=sc/8 dmin=sc/4, Q6_K sc/32). */
void orc_randn(float* out, int64_t n, uint64_t seed, float scale);
int orc_random_blocks(int t, int64_t n_elems, uint64_t seed, float scale, uint8_t* out);

/* MoE router for one token (tests/ref/arch_ref.cpp:97-113): score = sqrt(softplus(logit)) in double (softplus(x) = x
 * for x > 20, else log1p(exp(x))); key = (float)score + bias, rounded to float; the top_k experts by key, descending,
 * ties to the lower expert id; w[k] = (float)(score_k / (sum of the top_k scores + 1e-20) * route_scale). The reference
 * fixes n_exp = 384, top_k = 6, route_scale = 1.5. */
void orc_router(const float* logits, const float* bias, int n_exp, int top_k, float route_scale, int* ids, float* w);

/* y[i] = (float)(x[i] * r * w[i]) with r = 1 / sqrt(mean(x^2) + eps) in double; w may be NULL (tests/ref/arch_ref.cpp:66-71) */
void orc_rmsnorm(const float* x, const float* w, float* y, int dim, double eps);

/* Expert-sorted routing lists of n_entries = n_tokens * top_k entries (arch_ref.cpp:114-130): counts[n_exp],
 * offsets[n_exp + 1] (exclusive scan), and per sorted position p (expert-major, entry index ascending inside an expert)
 * entry[p] = i, tok[p] = i / top_k, lw[p] = w[i]; slot_of[i] = p. */
void orc_route_lists(const int* ids, const float* w, int n_entries, int n_exp, int top_k, uint32_t* counts,
                     uint32_t* offsets, uint32_t* entry, uint32_t* tok, float* lw, uint32_t* slot_of);

#ifdef __cplusplus
}
#endif
#endif
