// Rollout-side kernels of the policy path: categorical sampling from the fused
// head's outputs and reward/done extraction into the rollout slabs.
//
// Reference: k_value_sample (craftax_full.cu:9714-9741) with
// cf_nn_sample_action (:9147-9165), k_record_rd (:9758-9767).  The reference
// draws its uniform from cuRAND: curand_init(seed ^ 0xA5A5..., subsequence = env,
// offset = device step counter) of a Philox4_32_10 state, then curand_uniform.
// Here the same draw is computed directly (philox_uniform in cfp_common.h): the
// Philox4x32-10 block function is pinned by the published known-answer vectors,
// the mapping of (seed, subsequence, offset) onto key, counter and output word by
// rocRAND's engine (same three arguments; CPU test of the oracle's twin of
// philox_uniform), the conversion to a float is cuRAND's x * 2^-32 + 2^-33.  Given
// the uniform, the action and its log-probability follow the reference's
// arithmetic exactly (max-shifted expf, ascending cumulative sum, first index
// with target <= cum, last action as the fall-through).
#include "cfp_internal.h"
#include "sample_row.h"

namespace cfp {
namespace {

// Sixteen lanes per env, sixteen envs per workgroup.  The workgroup's logits rows are
// one contiguous piece of av and are staged through LDS with coalesced loads (a thread
// walking its own 176-byte row straight from memory touches 64 different lines per
// load instruction).  The order-independent parts -- the maximum and the
// exponentials -- are spread over the env's lanes; the two sums, whose rounding
// depends on their order, are then run by one lane in the reference's ascending
// order over the exponentials in LDS, so the draw is the sequential kernel's bit for bit.
constexpr int kSampleEnvs = 256 / kSampleLanes;

__global__ __launch_bounds__(256) void k_value_sample(
    const float* __restrict__ av, int avs, int actions, float* __restrict__ env_actions,
    int32_t* __restrict__ act, float* __restrict__ logprobs, float* __restrict__ values, int n,
    uint64_t seed, const uint64_t* step_ctr, unsigned* ticket) {
    __shared__ float logit[kSampleEnvs * (kMaxActions + 1)];
    __shared__ float expo[kSampleEnvs * kMaxActions];
    const int e0 = (int)blockIdx.x * kSampleEnvs;
    const int nb = n - e0 < kSampleEnvs ? n - e0 : kSampleEnvs;
    const float* src = av + (size_t)e0 * avs;
    for (int i = threadIdx.x; i < nb * avs; i += 256) logit[i] = src[i];
    __syncthreads();
    const int sub = threadIdx.x % kSampleLanes, slot = threadIdx.x / kSampleLanes;
    const bool live = slot < nb;
    const float* lp = logit + slot * avs;
    float* px = expo + slot * kMaxActions;
    const float m = sample_spread(lp, px, actions, sub, live);
    __syncthreads();
    if (live && sub == 0) {
        const uint64_t step = step_ctr ? *step_ctr : 0;
        if (actions == CFP_ACTIONS)
            sample_draw<CFP_ACTIONS>(lp, px, m, actions, e0 + slot, seed, step, env_actions, act,
                                     logprobs, values);
        else
            sample_draw(lp, px, m, actions, e0 + slot, seed, step, env_actions, act, logprobs,
                        values);
    }
    if (ticket) {   // the counter's bump rides on this launch (uniform branch)
        __syncthreads();
        if (threadIdx.x == 0)
            bump_by_last_group(ticket, const_cast<uint64_t*>(step_ctr), gridDim.x);
    }
}

// Large batches: one thread per env, 128 envs per workgroup (every lane busy through
// the sums; the sixteen-lane form above leaves fifteen of sixteen idle there and wins
// only while the launch is too small to fill the machine).  Same staging, rows of an
// odd stride so that the threads' rows start in different banks; the exponentials
// replace the logits in the row.  Same operations in the same order: same bits.
constexpr int kSampleRowEnvs = 128;

// ACTIONS > 0 fixes the action count at compile time: the row is read from LDS once into
// registers, and the partial sums of the total serve as the scan's cumulative sums (the
// reference adds the same terms up in the same order twice).
template <int ACTIONS>
__global__ __launch_bounds__(kSampleRowEnvs) void k_value_sample_rows(
    const float* __restrict__ av, int avs, int actions, float* __restrict__ env_actions,
    int32_t* __restrict__ act, float* __restrict__ logprobs, float* __restrict__ values, int n,
    uint64_t seed, const uint64_t* __restrict__ step_ctr) {
    __shared__ float rows[kSampleRowEnvs * (kMaxActions + 1)];
    const int stride = avs | 1;
    const int e0 = (int)blockIdx.x * kSampleRowEnvs;
    const int nb = n - e0 < kSampleRowEnvs ? n - e0 : kSampleRowEnvs;
    const float* src = av + (size_t)e0 * avs;
    const float inv = 1.0f / (float)avs;
    for (int i = threadIdx.x; i < nb * avs; i += kSampleRowEnvs) {
        // i / avs through the reciprocal: (i + 0.5) / avs keeps 0.5 / avs away from every
        // integer, far more than the rounding of this product for i < 2^14
        const int row = (int)(((float)i + 0.5f) * inv);
        rows[row * stride + (i - row * avs)] = src[i];
    }
    __syncthreads();
    const int e = e0 + (int)threadIdx.x;
    if (e >= n) return;
    float* lp = rows + threadIdx.x * stride;
    if (values) values[e] = lp[actions];
    const uint64_t step = step_ctr ? *step_ctr : 0;
    const float u = philox_uniform(seed ^ 0xA5A5A5A5A5A5A5A5ULL, (uint64_t)e, step);
    float m, total = 0.0f, chosen;
    int action = actions - 1;
    if (ACTIONS > 0) {
        float z[ACTIONS > 0 ? ACTIONS : 1], cum[ACTIONS > 0 ? ACTIONS : 1];
#pragma unroll
        for (int a = 0; a < ACTIONS; a++) z[a] = lp[a];
        m = z[0];
#pragma unroll
        for (int a = 1; a < ACTIONS; a++) m = fmaxf(m, z[a]);
#pragma unroll
        for (int a = 0; a < ACTIONS; a++) {
            total += expf(z[a] - m);
            cum[a] = total;
        }
        const float target = u * total;
        chosen = z[ACTIONS - 1];
#pragma unroll
        for (int a = ACTIONS - 1; a >= 0; a--)
            if (target <= cum[a]) {   // descending: the smallest hit is kept
                action = a;
                chosen = z[a];
            }
    } else {
        m = lp[0];
        for (int a = 1; a < actions; a++) m = fmaxf(m, lp[a]);
        for (int a = 0; a < actions; a++) {
            const float p = expf(lp[a] - m);
            lp[a] = p;
            total += p;
        }
        const float target = u * total;
        float cum = 0.0f;
        for (int a = 0; a < actions; a++) {
            cum += lp[a];
            if (target <= cum) { action = a; break; }
        }
        chosen = av[(size_t)e * avs + action];
    }
    if (env_actions) env_actions[e] = (float)action;
    act[e] = action;
    logprobs[e] = chosen - m - logf(total);
}

__global__ void k_record_rd(const float* __restrict__ rewards, const float* __restrict__ terminals,
                            float* __restrict__ r_reward_row, uint8_t* __restrict__ r_done_row,
                            int n) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    r_reward_row[e] = rewards[e];
    r_done_row[e] = terminals[e] != 0.0f ? 1 : 0;
}

}  // namespace

// ticket not null (batches below kSampleRowsFrom envs only): the launch also bumps
// *d_step_ctr once every workgroup has read it; *ticket is zero before and after.
int value_sample(const float* d_av, int n, int actions, float* d_env_actions, int32_t* d_actions,
                 float* d_logprobs, float* d_values, uint64_t seed, const uint64_t* d_step_ctr,
                 unsigned* ticket, hipStream_t st) {
    CFP_REQUIRE(d_av && d_actions && d_logprobs && n > 0, "cfp_value_sample: bad argument");
    CFP_REQUIRE(actions > 0 && actions <= kMaxActions, "cfp_value_sample: actions must be in 1..%d",
                kMaxActions);
    CFP_REQUIRE(!ticket || (d_step_ctr && n < kSampleRowsFrom),
                "value_sample: the in-launch counter bump covers batches below %d envs",
                kSampleRowsFrom);
    if (n >= kSampleRowsFrom && actions == CFP_ACTIONS)
        hipLaunchKernelGGL(k_value_sample_rows<CFP_ACTIONS>,
                           dim3((n + kSampleRowEnvs - 1) / kSampleRowEnvs), dim3(kSampleRowEnvs), 0,
                           st, d_av, actions + 1, actions, d_env_actions, d_actions, d_logprobs,
                           d_values, n, seed, d_step_ctr);
    else if (n >= kSampleRowsFrom)
        hipLaunchKernelGGL(k_value_sample_rows<0>, dim3((n + kSampleRowEnvs - 1) / kSampleRowEnvs),
                           dim3(kSampleRowEnvs), 0, st, d_av, actions + 1, actions, d_env_actions,
                           d_actions, d_logprobs, d_values, n, seed, d_step_ctr);
    else
        hipLaunchKernelGGL(k_value_sample, dim3((n + kSampleEnvs - 1) / kSampleEnvs), dim3(256), 0,
                           st, d_av, actions + 1, actions, d_env_actions, d_actions, d_logprobs,
                           d_values, n, seed, d_step_ctr, ticket);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace cfp

using namespace cfp;

extern "C" {

int cfp_value_sample(const float* d_av, int n, int actions, float* d_env_actions,
                     int32_t* d_actions, float* d_logprobs, float* d_values, uint64_t seed,
                     const uint64_t* d_step_ctr, void* stream) {
    return value_sample(d_av, n, actions, d_env_actions, d_actions, d_logprobs, d_values, seed,
                        d_step_ctr, nullptr, (hipStream_t)stream);
}

int cfp_record_rd(const float* d_rewards, const float* d_terminals, float* d_r_reward_row,
                  uint8_t* d_r_done_row, int n, void* stream) {
    CFP_REQUIRE(d_rewards && d_terminals && d_r_reward_row && d_r_done_row && n > 0,
                "cfp_record_rd: bad argument");
    hipLaunchKernelGGL(k_record_rd, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       d_rewards, d_terminals, d_r_reward_row, d_r_done_row, n);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // extern "C"
