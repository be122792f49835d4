// Categorical draw from one env's staged head row (actions logits, then the value),
// shared by the stand-alone sampler (rollout.hip) and the small-batch forward kernel
// that samples behind its heads (policy_forward_t16.hip): the same operations in the
// same order in both, so both give the reference's draw (k_value_sample with
// cf_nn_sample_action, craftax_full.cu:9714-9741, :9147-9165) bit for bit.
#pragma once

#include "cfp_common.h"

namespace cfp {

constexpr int kMaxActions = 64;
constexpr int kSampleLanes = 16;   // lanes that share one env's row

// Order-independent part, spread over the env's sixteen lanes (consecutive lanes of one
// wave): the row maximum, returned to each of them, and px[a] = expf(lp[a] - max).
// A workgroup barrier must follow before sample_draw reads px.
__device__ __forceinline__ float sample_spread(const float* lp, float* px, int actions, int sub,
                                               bool live) {
    float m = -INFINITY;
    if (live)
        for (int a = sub; a < actions; a += kSampleLanes) m = fmaxf(m, lp[a]);
#pragma unroll
    for (int d = kSampleLanes / 2; d > 0; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, kSampleLanes));
    if (live)
        for (int a = sub; a < actions; a += kSampleLanes) px[a] = expf(lp[a] - m);
    return m;
}

// Order-dependent part, run by one lane of the env: the sum of the exponentials in
// ascending action order, the uniform of (seed, env, step), the first action whose
// cumulative sum reaches the target (the last action as the fall-through), and the outputs.
// The reference adds the exponentials up twice in the same order (once for the total, once
// for the scan: cf_nn_sample_action, craftax_full.cu:9147-9165), so the scan's cumulative sums
// are the partial sums of the total.  ACTIONS > 0 fixes the action count at compile time:
// the partial sums are then kept (one chain of additions instead of two, the exponentials
// read from LDS once, in one batch) and the scan is 43 independent comparisons.
template <int ACTIONS = 0>
__device__ __forceinline__ void sample_draw(const float* lp, const float* px, float m, int actions,
                                            int e, uint64_t seed, uint64_t step,
                                            float* __restrict__ env_actions,
                                            int32_t* __restrict__ act,
                                            float* __restrict__ logprobs,
                                            float* __restrict__ values) {
    const int na = ACTIONS > 0 ? ACTIONS : actions;
    if (values) values[e] = lp[na];
    const float u = philox_uniform(seed ^ 0xA5A5A5A5A5A5A5A5ULL, (uint64_t)e, step);
    float total = 0.0f;
    int action = na - 1;
    if (ACTIONS > 0) {
        float cum[ACTIONS > 0 ? ACTIONS : 1];
#pragma unroll
        for (int a = 0; a < ACTIONS; a++) {
            total += px[a];
            cum[a] = total;
        }
        const float target = u * total;
#pragma unroll
        for (int a = ACTIONS - 1; a >= 0; a--)
            if (target <= cum[a]) action = a;   // descending: the smallest hit is kept
    } else {
        for (int a = 0; a < na; a++) total += px[a];
        const float target = u * total;
        float cum = 0.0f;
        for (int a = 0; a < na; a++) {
            cum += px[a];
            if (target <= cum) { action = a; break; }
        }
    }
    if (env_actions) env_actions[e] = (float)action;
    act[e] = action;
    logprobs[e] = lp[action] - m - logf(total);
}

// The step counter's bump without a launch of its own: every workgroup takes a ticket
// once its lanes have used the counter, and the one that takes the last ticket writes
// counter + 1 and clears the tickets for the next launch.  Called by one thread of
// each workgroup, after a barrier that follows the workgroup's last read of the
// counter.  Meant for launches of at most a few thousand workgroups (the tickets are
// atomics on one word).
__device__ __forceinline__ void bump_by_last_group(unsigned* ticket, uint64_t* ctr, unsigned groups) {
    // The counter is unchanged until every ticket, this one included, is taken.  No fence
    // is needed in front of the ticket: the workgroup's reads of the counter have
    // returned (their values were used before the barrier), and the two stores below
    // become visible to the next launch at the end of this one.
    const uint64_t step = *ctr;
    if (atomicAdd(ticket, 1u) == groups - 1) {
        *ctr = step + 1;
        *ticket = 0u;
    }
}
// The same in two halves, for a workgroup that holds the counter's value in registers
// (`step`): the ticket can be taken as soon as all its reads of the counter have returned,
// and the atomic's round trip then runs under whatever work is left.
__device__ __forceinline__ unsigned take_ticket(unsigned* ticket) { return atomicAdd(ticket, 1u); }
__device__ __forceinline__ void bump_if_last(unsigned no, unsigned groups, unsigned* ticket,
                                             uint64_t* ctr, uint64_t step) {
    if (no == groups - 1) {
        *ctr = step + 1;
        *ticket = 0u;
    }
}

}  // namespace cfp
