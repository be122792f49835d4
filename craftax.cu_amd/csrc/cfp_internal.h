// Library-internal definition of the policy object (opaque in include/cfp.h).
#pragma once

#include "cfp_common.h"

struct cfp_policy {
    int n = 0;
    int layers = 0;
    int variant = 0;   // 0 full game, 1 classic
    size_t param_count = 0;
    float* params = nullptr;
    float* we_pk = nullptr;
    uint16_t* we_s3 = nullptr;    // map rows of W_enc split in three bf16 terms
    float* wg_pk = nullptr;
    float* wav_pk = nullptr;
    uint16_t* we_bf = nullptr;    // bf16 mirrors (MFMA 32x32x16 order)
    uint16_t* wg_bf = nullptr;
    uint16_t* wav_bf = nullptr;
    int gemm_bf16 = 0;            // forward entry points run the bf16-input kernel
    int rs_bf16 = 0;              // r_state rows leave as bf16 (a trainer with a bf16 state slab)
    void* enc_x9 = nullptr;       // split mirror of W_enc for the forward from a feature matrix
    void* t16 = nullptr;          // mirrors of the 16-env-tile kernel (full game only)
    int small_tiles = 0;          // batches of at most 4096 envs run on 16-env tiles
    float* h_state = nullptr;
    uint8_t* rec = nullptr;
    float* h_enc = nullptr;
    float* h3 = nullptr;
    float* logits = nullptr;
    hipStream_t stream = nullptr;
};

namespace cfp {
// weight pointers, variant and action count of a policy into launch arguments
void fill_forward_weights(const cfp_policy* p, FwdArgs& a);

// Sampler behind cfp_value_sample.  From kSampleRowsFrom envs on it runs one thread per
// env; below, sixteen lanes per env, and there `ticket` (one zeroed word of device
// memory, or null) makes the launch bump *d_step_ctr itself once every workgroup has
// read it.
constexpr int kSampleRowsFrom = 16384;
int value_sample(const float* d_av, int n, int actions, float* d_env_actions, int32_t* d_actions,
                 float* d_logprobs, float* d_values, uint64_t seed, const uint64_t* d_step_ctr,
                 unsigned* ticket, hipStream_t st);

// launch_forward also draws the actions (FwdArgs::s_act ...) when this holds: full-game
// records in recording mode on 32-env tiles, one tile per workgroup (at most one per CU).
bool forward_draws(const FwdArgs& a);

// One rollout step's policy side for the trainer: records -> heads into the policy's
// live state and logits (r_state recorded), then the draw into act / logp / value
// (and env_actions when not null) with offset *step_ctr, then *step_ctr += 1.  One
// launch where the 16-env-tile kernel applies, forward + sampler otherwise.
struct SampleOut {
    int32_t* act;
    float* logp;
    float* value;
    float* env_actions;
    uint64_t seed;
    uint64_t* step_ctr;
    unsigned* ticket;   // one zeroed word, left zeroed
};
int forward_and_sample(cfp_policy* p, const uint8_t* d_rec_row, const float* d_terminals,
                       float* d_r_state_t, int n, const SampleOut& s, hipStream_t st);
}  // namespace cfp
