// Launchers of the PPO update's streaming kernels (ppo_kernels.hip): reverse MinGRU
// sweep, head gradients, GAE with advantage moments, Adam with the weight mirrors
// written in the same pass.  Internal to the library.
#pragma once

#include "cfp_common.h"
#include "cfp_internal.h"

namespace cfp {

// Window addressing shared by these kernels: column c of a window is sample
// (step t0 + c / mb, env env_start + c % mb) of slabs laid out [T][n_all].
struct WindowMap {
    int t0, mb, n_all, env_start;
};

// Reverse sweep of one MinGRU layer over a window (the reference's
// k_mingru_window_bwd, craftax_full.cu:9510-9597).
struct ReverseArgs {
    float* gates;              // [cols][768]: zh | zg | zp in, their gradients out, in place
    const float* layer_in;     // [cols][256]: the layer's input (the highway branch)
    const float* grad_a;       // [cols][256]: gradient of the loss w.r.t. the layer's output ...
    const float* grad_b;       // ... plus this second term when not null
    float* highway_out;        // [cols][256]: gradient passed to the layer's input past the gates
    const float* slab_state;   // r_state [T][layers][n_all][256]: stored post-zero state inputs
    const uint8_t* slab_done;  // r_done  [T][n_all]
    float* carry;              // [mb][256]: gradient w.r.t. the recurrent state, live across windows
    WindowMap w;
    int steps;                 // steps in this window
    int layer, layers;
    int horizon, seg;          // rollout length, BPTT segment length
    int gates_bf16;            // gates, layer_in, grad_a/b and highway_out are bf16 arrays (the
                               // update's bf16 storage); carry stays fp32
    int state_bf16;            // slab_state is a bf16 array of the same shape (with gates_bf16 only)
};
int launch_gru_reverse(const ReverseArgs& a, hipStream_t st);

// Window recompute of one layer from the stored state (unfused chain only; the
// reference's k_mingru_epi_replay_win, craftax_full.cu:9460-9503).
int launch_gru_replay(const float* gates, const float* layer_in, const float* slab_state,
                      float* layer_out, const WindowMap& w, int cols, int layer, int layers,
                      hipStream_t st);

// PPO head: loss terms and, when grad_rows is not null, the gradient rows
// [43 dlogits | dvalue | 0 0 0 0] of every window column (k_head_bwd_win,
// craftax_full.cu:9603-9706; loss-only form k_loss_accum :10508-10560).
struct HeadArgs {
    const float* rows;          // [cols][ld]: 43 logits then the value
    int ld;                     // 44 or 48
    const float* bias_a;        // added to the logits / the value when not null
    const float* bias_v;
    const int32_t* act;         // slabs [T][n_all]
    const float* old_logp;
    const float* adv;
    const float* ret;
    const double* adv_moments;  // sum and sum of squares of adv over the whole rollout
    float* grad_rows;           // [cols][48] or null
    double* block_loss;         // [blocks][3] partial sums: -min(u1,u2), (v-ret)^2/2, entropy
    WindowMap w;
    int cols;
    int horizon;
    float clip, vf;
    const float* ent_coef;      // device scalar
};
constexpr int kHeadGradLd = 48;
int head_blocks(int cols);
int launch_head(const HeadArgs& a, hipStream_t st);
// acc[q] (+)= sum_b part[b * NQ + q] in a fixed order
int launch_fold_f64(const double* part, int blocks, int nq, double* acc, bool accumulate,
                    hipStream_t st);

// GAE(gamma, lambda) over [T][n] slabs and the sum / sum of squares of the advantages
// (k_gae :10617, k_adv_stats :10638).  part: 2 * gae_blocks(n) doubles.
int gae_blocks(int n);
int launch_gae(const float* values, const float* rewards, const uint8_t* dones,
               const float* v_boot, float* adv, float* ret, int n, int T, float gamma, float lam,
               double* part, double* moments, hipStream_t st);
constexpr int kMomentBlocks = 256;
int launch_adv_moments(const float* adv, size_t count, double* part, double* moments,
                       hipStream_t st);

// Adam step on the flat arena (k_adam :10668): params, moments updated, grads zeroed,
// and every weight mirror of the full-game policy rewritten from the new values in
// the same pass.  step_ctr is read, not bumped.
int launch_adam(cfp_policy* p, float* grads, float* m, float* v, const uint64_t* step_ctr,
                const float* lr, float beta1, float beta2, float eps, hipStream_t st);

// dW_enc from the records (enc_grad.hip) with the fp32 rows of its 75-feature remainder made
// ahead of time: the expansion depends on the records only, so the update asks for it at the
// start of a window, next to the recompute, instead of at the end of the dependent chain.
int dw_enc_tail_expand(const uint8_t* r_obs, float* tail_scratch, int t0, int cols, int mb, int n_all,
                       int env_start, hipStream_t st);
int dw_enc_records_tail_ready(const uint8_t* r_obs, const float* dh, float* dW, float* tail_scratch, int t0,
                              int cols, int mb, int n_all, int env_start, const SeamWork& sw, hipStream_t st,
                              bool dh_bf16, const SeamWork* sw_tail, hipStream_t st_tail);

}  // namespace cfp
