/* PPO-update half of the CPU oracle.  TEST INFRASTRUCTURE ONLY (see cfo.h). */
#ifndef CFO_TRAIN_H_
#define CFO_TRAIN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One minibatch of a stored rollout: the reference's CuTrain slabs
 * (craftax_full.cu:12694-12700), all [T][n]-shaped, and the PPO coefficients
 * (cu_ppo_defaults, :12647-12655). */
typedef struct cfo_ppo_batch {
    int T, n;             /* rollout horizon and env count of the slabs   */
    int env_start, mb;    /* the minibatch is envs [env_start, env_start+mb) */
    int layers;
    int seg_len;          /* T / bptt_split                               */
    const uint8_t* r_obs;     /* [T][n][996]                              */
    const float* r_state;     /* [T][layers][n][256] post-zero state inputs */
    const int32_t* r_act;     /* [T][n]                                   */
    const float* r_logprob;
    const float* adv;
    const float* ret;
    const uint8_t* r_done;
    double adv_sum, adv_sumsq; /* over the whole [T][n] (k_adv_stats)     */
    float clip, vf, ent;
} cfo_ppo_batch;

double cfo_ppo_loss_f64(const float* params, const cfo_ppo_batch* b, double* loss3);
void cfo_ppo_backward_f64(const float* params, const cfo_ppo_batch* b, double* grads,
                          double* loss3);
/* cfo_ppo_backward_f64 with both operands of every matrix product rounded to bf16 and the
 * accumulation kept in fp64: the comparator of the bf16-input / fp32-accumulate update.
 * flags bit 0: also round what cfp_train_set_bf16_storage stores as bf16.
 * flags bit 1: the 768 leading map-byte rows of dW_enc multiply the unrounded encoder
 * gradient (the update with the split kernels switched off). */
void cfo_ppo_backward_bf16ops_f64(const float* params, const cfo_ppo_batch* b, double* grads,
                                  double* loss3, int flags);
/* min |zh| over the minibatch's recompute: the distance of the batch from the kink of the
 * candidate function, where the gradient is discontinuous. */
double cfo_ppo_min_abs_zh(const float* params, const cfo_ppo_batch* b, int bf16_ops);
void cfo_gae_f64(const float* values, const float* rewards, const uint8_t* dones,
                 const float* v_boot, double* adv, double* ret, int n, int T,
                 double gamma, double lam);
void cfo_adam_f64(double* params, const double* grads, double* m, double* v,
                  size_t count, int step, double lr, double beta1, double beta2,
                  double eps);

#ifdef __cplusplus
}
#endif
#endif
