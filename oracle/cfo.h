/*
 * cfo.h -- CPU oracle for the batched policy path.  TEST INFRASTRUCTURE ONLY:
 * nothing under oracle/ is linked into or called by the product library; only
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it, and
 * only as the checker / the timed CPU baseline.
 *
 * It restates, in plain C, the reference algorithms this repo reimplements in
 * HIP.  Each function cites the reference lines it follows.  Pinning status:
 *   cfo_encode_compact      pinned: golden records dumped from the compiled
 *                           reference (tests/golden/), incl. fuzzed states,
 *                           and live comparison against oracle/_ref when built
 *   cfo_expand_record       pinned: closed form (all 256 bytes, bit patterns)
 *   cfo_forward_f64 / _f32  pinned: independent numpy fp64 evaluation with
 *                           library matmuls, closed forms (zero weights,
 *                           terminal reset, gate saturation), brute-force carry
 *   cfo_backward_f64        pinned: central finite differences of cfo_loss_f64
 *                           (the reference's own gradcheck method,
 *                           craftax_full.cu:13854-13907) and closed forms
 *   cfo_sample_action       pinned: closed forms (equal logits, dominant logit,
 *                           normalisation of exp(logprob))
 *   cfo_philox4x32_10       pinned: the three known-answer vectors published with
 *                           the generator (Random123 kat_vectors, philox4x32 10)
 *   cfo_philox_draw         pinned: rocRAND's Philox4x32-10 engine on the host
 *                           (rocrand_init(seed, subsequence, offset) + rocrand), the
 *                           ROCm routine with curand_init's three arguments, over
 *                           thousands of triples (oracle/rocrand_check.cpp)
 *   cfo_philox_uniform      the draw through cuRAND's published conversion
 *                           x * 2^-32 + 2^-33 (rocRAND adds 2^-32, so the float
 *                           itself has no library to be held to: closed form only)
 */
#ifndef CFO_H_
#define CFO_H_

#include <stddef.h>
#include <stdint.h>

#include "../include/cfp.h"

#ifdef __cplusplus
extern "C" {
#endif

/* craftax_encode_compact_observation (craftax_full.c:2830-2844 with
 * :2721-2825, tail :2646-2703).  Planes are 48x48 u8; plane for level L starts
 * at base + L*level_stride. */
void cfo_encode_compact(const cfp_env_scalars* s, const uint8_t* map,
                        const uint8_t* item_map, const uint8_t* light_map,
                        size_t level_stride, uint8_t* obs /*[996]*/);
void cfo_encode_compact_batch(int n, const cfp_env_scalars* s, const uint8_t* map,
                              const uint8_t* item_map, const uint8_t* light_map,
                              size_t env_stride, size_t level_stride,
                              uint8_t* rec /*[n][996]*/);

/* k_expand_obs (craftax_full.cu:10028-10053). */
void cfo_expand_record(const uint8_t* rec /*[996]*/, float* x /*[843]*/);

/* fp64 evaluation of k_policy_ref_l3's math (craftax_full.cu:9778-9854) on
 * fp32 weights and inputs.  state_in/out [layers][n][256] (env-major, as the
 * production h_state, craftax_full.cu:9366).  Any output may be NULL. */
void cfo_forward_f64(const float* params, int layers, int n,
                     const float* x /*[n][843]*/, const double* state_in,
                     const float* prev_terminals /*[n] or NULL*/,
                     double* h_enc /*[n][256]*/, double* r_state /*[L][n][256]*/,
                     double* state_out, double* h3 /*[n][256]*/,
                     double* logits /*[n][43]*/, double* values /*[n]*/);

/* Classic-game policy (config 5): record expansion of encode_obs_kernel
 * (craftax_classic.cu:1714-1751) and the same forward with 1345 features /
 * 17 actions; logits [n][17].  Pinned like cfo_forward_f64 (numpy fp64
 * cross-check, one-hot closed form). */
void cfo_classic_expand(const uint8_t* rec /*[148]*/, float* x /*[1345]*/);
void cfo_classic_forward_f64(const float* params, int layers, int n,
                             const float* x /*[n][1345]*/, const double* state_in,
                             const float* prev_terminals, double* h_enc,
                             double* r_state, double* state_out, double* h3,
                             double* logits /*[n][17]*/, double* values);

/* Scalar fp32 forward following k_policy_ref_l3 literally (fmaf chains in
 * ascending feature order, exact-zero features skipped), from records, state
 * updated in place; OpenMP over envs with `threads` threads (<=0: default).
 * This is the CPU baseline that bench.py times. */
void cfo_forward_f32(const float* params, int layers, int n,
                     const uint8_t* rec /*[n][996]*/, float* state /*[L][n][256]*/,
                     const float* prev_terminals, float* av /*[n][44]*/,
                     int threads);

/* cf_nn_sample_action (craftax_full.cu:9147-9165) for a given uniform u; pinned
 * by closed forms (equal logits -> floor(u*A), dominant logit, exp(logprob) sums
 * to one). */
int cfo_sample_action(const float* logits, int actions, float u, float* logprob);
/* Philox4x32-10 and the uniform of the reference's sampler (k_value_sample,
 * craftax_full.cu:9732-9736: curand_init(seed ^ 0xA5A5.., env, step) + curand_uniform). */
void cfo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
uint32_t cfo_philox_draw(uint64_t seed, uint64_t subsequence, uint64_t offset);
float cfo_philox_uniform(uint64_t seed, uint64_t subsequence, uint64_t offset);
float cfo_sample_margin(const float* logits, int actions, float u);

int cfo_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
