// Calls between the env, the record kernels and the trainer that are not part of the C ABI:
// the rollout step with the env in the loop folds two one-line kernels of its sequence
// (clearing the finished-env counter, copying rewards / done flags into the slabs) into the
// kernels next to them.
#pragma once
#include <cstddef>
#include <cstdint>

#include "../../include/cfp.h"
#include "../../include/cfp_env.h"

namespace cfp {

// cfp_record_obs_soa that also stores 0 to *d_zero (when not null) from its first thread.
int record_obs_soa_zero(const cfp_env_soa* soa, const uint8_t* d_map, const uint8_t* d_item_map,
                        const uint8_t* d_light_map, size_t env_stride, size_t level_stride,
                        uint8_t* d_rec_row, int n, int* d_zero, void* stream);

// cfp_env_record_obs that leaves the env's finished-env counter at zero: what cfp_env_step
// does with a launch of its own is done here by the record kernel.  Only for a sequence in
// which the counter has been consumed (reset) and env_step_rows follows.
int env_record_obs_zero(const cfp_env* e, uint8_t* d_rec_row, void* stream);

// cfp_env_step on the env's own action / reward / terminal slots, without the launch that
// clears the counter (env_record_obs_zero has), and with each env's reward and done flag
// also written to a trainer's slab rows (k_record_rd, craftax_full.cu:9758-9767).
int env_step_rows(cfp_env* e, float* d_r_reward_row, uint8_t* d_r_done_row, void* stream);

}  // namespace cfp
