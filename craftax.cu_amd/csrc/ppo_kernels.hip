// Streaming kernels of the on-device PPO update for gfx950.  The mathematics is the
// reference's (craftax_full.cu: k_mingru_window_bwd :9510, k_head_bwd_win :9603,
// k_mingru_epi_replay_win :9460, k_loss_accum :10508, k_gae :10617, k_adv_stats :10638,
// k_adam :10668); the kernels are laid out for 64-wide wavefronts and 16-byte accesses:
//
//   reverse sweep   one wavefront per env, a lane owns four hidden units: every stream
//                   of a step (three gate rows, two gradient rows, stored state, layer
//                   input in; three gate gradients and the highway gradient out) is one
//                   coalesced 1 KiB row per wavefront, requested two steps before the
//                   step that consumes it, so that only the four-float carry is
//                   serial in time
//   head            the window's head rows are contiguous: 64 of them are staged
//                   through LDS with 16-byte loads, four lanes share a column (eleven
//                   actions each, reductions by cross-lane adds in a fixed pattern),
//                   gradient rows leave through LDS as 16-byte stores
//   GAE             one lane per env walking time backwards with the loads of eight
//                   steps in flight; the advantage moments are accumulated in the same
//                   pass (double) and folded in a fixed order
//   Adam            four parameters per lane; the lane that updates a weight also
//                   writes it into every MFMA-ordered mirror the forward kernels read
//                   (fp32, three-term bf16 split, bf16), so no repack pass follows
// Every reduction runs in a fixed order: results are bitwise reproducible run to run.
#include "ppo_kernels.h"

#include "policy_tile.h"

namespace cfp {
namespace {

constexpr int H = CFP_HIDDEN, G = CFP_GRU, A = CFP_ACTIONS;
constexpr int H4 = H / 4, G4 = G / 4;

__device__ __forceinline__ f4 ld_stream(const f4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st_stream(f4* p, const f4& v) { __builtin_nontemporal_store(v, p); }

// sum over the 64 lanes of a wavefront, the same bits in every lane (butterfly of
// commutative adds)
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
    return v;
}

// ---- reverse MinGRU sweep --------------------------------------------------------
// The loads and stores of a step are issued from inline assembly and the wait that
// makes a step's operands readable is an explicit s_waitcnt vmcnt(N): the compiler's own
// wait insertion drains the whole queue (vmcnt(0)) in front of every store, which leaves
// nothing in flight while a wavefront computes.  Vector-memory operations complete in
// issue order, so "the set fetched three stages ago has landed" is "at most N younger
// operations are outstanding".  Three register sets rotate through a loop unrolled by
// three (a set is never copied: a copy would read registers whose loads are in flight).
// G16: the gate rows, the layer input, the incoming gradients and the highway term are
// stored as bf16 (8 bytes per lane and row); the recorded state stays fp32 unless G16 = 2.
typedef unsigned int u2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// G16 = 2: the recorded state is a bf16 slab as well (cfp_train_set_bf16_rstate).
template <int G16>
struct StepIn;
template <>
struct StepIn<0> {
    f4 zh, zg, zp, x, ga, gb, s;
    unsigned done;
};
template <>
struct StepIn<1> {
    u2 zh, zg, zp, x, ga, gb;
    f4 s;
    unsigned done;
};
template <>
struct StepIn<2> {
    u2 zh, zg, zp, x, ga, gb, s;
    unsigned done;
};

__device__ __forceinline__ f4 widen(const f4& v) { return v; }
__device__ __forceinline__ f4 widen(const u2& v) {   // four bf16 -> four fp32
    return f4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
              __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u)};
}
__device__ __forceinline__ u2 narrow(const f4& v) {   // round to nearest even
    return __builtin_bit_cast(u2, __builtin_convertvector(v, bf16x4));
}

// lo: byte offset of the lane inside an fp32 row (16 q), lo8: inside a bf16 row (8 q)
template <bool TWO_GRADS, int G16>
__device__ __forceinline__ void sweep_fetch(StepIn<G16>& r, unsigned lo, unsigned lo8,
                                            const void* gates, const void* ga, const void* gb,
                                            const void* state, const void* xin, const uint8_t* done) {
    const unsigned zero = 0u;
    if (G16 == 2 && TWO_GRADS)
        asm volatile(
            "global_load_dwordx2 %0, %9, %11 nt\n\t"
            "global_load_dwordx2 %1, %9, %11 offset:512 nt\n\t"
            "global_load_dwordx2 %2, %9, %11 offset:1024 nt\n\t"
            "global_load_dwordx2 %3, %9, %12 nt\n\t"
            "global_load_dwordx2 %4, %9, %13 nt\n\t"
            "global_load_dwordx2 %5, %9, %14 nt\n\t"
            "global_load_dwordx2 %6, %9, %15 nt\n\t"
            "global_load_ubyte %7, %10, %16"
            : "=&v"(r.zh), "=&v"(r.zg), "=&v"(r.zp), "=&v"(r.ga), "=&v"(r.gb), "=&v"(r.s),
              "=&v"(r.x), "=&v"(r.done)
            : "v"(lo), "v"(lo8), "v"(zero), "s"(gates), "s"(ga), "s"(gb), "s"(state), "s"(xin),
              "s"(done)
            : "memory");
    else if (G16 == 2)
        asm volatile(
            "global_load_dwordx2 %0, %8, %10 nt\n\t"
            "global_load_dwordx2 %1, %8, %10 offset:512 nt\n\t"
            "global_load_dwordx2 %2, %8, %10 offset:1024 nt\n\t"
            "global_load_dwordx2 %3, %8, %11 nt\n\t"
            "global_load_dwordx2 %4, %8, %12 nt\n\t"
            "global_load_dwordx2 %5, %8, %13 nt\n\t"
            "global_load_ubyte %6, %9, %14"
            : "=&v"(r.zh), "=&v"(r.zg), "=&v"(r.zp), "=&v"(r.ga), "=&v"(r.s), "=&v"(r.x),
              "=&v"(r.done)
            : "v"(lo), "v"(lo8), "v"(zero), "s"(gates), "s"(ga), "s"(state), "s"(xin), "s"(done)
            : "memory");
    else if (G16 && TWO_GRADS)
        asm volatile(
            "global_load_dwordx2 %0, %9, %11 nt\n\t"
            "global_load_dwordx2 %1, %9, %11 offset:512 nt\n\t"
            "global_load_dwordx2 %2, %9, %11 offset:1024 nt\n\t"
            "global_load_dwordx2 %3, %9, %12 nt\n\t"
            "global_load_dwordx2 %4, %9, %13 nt\n\t"
            "global_load_dwordx4 %5, %8, %14 nt\n\t"
            "global_load_dwordx2 %6, %9, %15 nt\n\t"
            "global_load_ubyte %7, %10, %16"
            : "=&v"(r.zh), "=&v"(r.zg), "=&v"(r.zp), "=&v"(r.ga), "=&v"(r.gb), "=&v"(r.s),
              "=&v"(r.x), "=&v"(r.done)
            : "v"(lo), "v"(lo8), "v"(zero), "s"(gates), "s"(ga), "s"(gb), "s"(state), "s"(xin),
              "s"(done)
            : "memory");
    else if (G16)
        asm volatile(
            "global_load_dwordx2 %0, %8, %10 nt\n\t"
            "global_load_dwordx2 %1, %8, %10 offset:512 nt\n\t"
            "global_load_dwordx2 %2, %8, %10 offset:1024 nt\n\t"
            "global_load_dwordx2 %3, %8, %11 nt\n\t"
            "global_load_dwordx4 %4, %7, %12 nt\n\t"
            "global_load_dwordx2 %5, %8, %13 nt\n\t"
            "global_load_ubyte %6, %9, %14"
            : "=&v"(r.zh), "=&v"(r.zg), "=&v"(r.zp), "=&v"(r.ga), "=&v"(r.s), "=&v"(r.x),
              "=&v"(r.done)
            : "v"(lo), "v"(lo8), "v"(zero), "s"(gates), "s"(ga), "s"(state), "s"(xin), "s"(done)
            : "memory");
    else if (TWO_GRADS)
        asm volatile(
            "global_load_dwordx4 %0, %8, %10 nt\n\t"
            "global_load_dwordx4 %1, %8, %10 offset:1024 nt\n\t"
            "global_load_dwordx4 %2, %8, %10 offset:2048 nt\n\t"
            "global_load_dwordx4 %3, %8, %11 nt\n\t"
            "global_load_dwordx4 %4, %8, %12 nt\n\t"
            "global_load_dwordx4 %5, %8, %13 nt\n\t"
            "global_load_dwordx4 %6, %8, %14 nt\n\t"
            "global_load_ubyte %7, %9, %15"
            : "=&v"(r.zh), "=&v"(r.zg), "=&v"(r.zp), "=&v"(r.ga), "=&v"(r.gb), "=&v"(r.s),
              "=&v"(r.x), "=&v"(r.done)
            : "v"(lo), "v"(zero), "s"(gates), "s"(ga), "s"(gb), "s"(state), "s"(xin), "s"(done)
            : "memory");
    else
        asm volatile(
            "global_load_dwordx4 %0, %7, %9 nt\n\t"
            "global_load_dwordx4 %1, %7, %9 offset:1024 nt\n\t"
            "global_load_dwordx4 %2, %7, %9 offset:2048 nt\n\t"
            "global_load_dwordx4 %3, %7, %10 nt\n\t"
            "global_load_dwordx4 %4, %7, %11 nt\n\t"
            "global_load_dwordx4 %5, %7, %12 nt\n\t"
            "global_load_ubyte %6, %8, %13"
            : "=&v"(r.zh), "=&v"(r.zg), "=&v"(r.zp), "=&v"(r.ga), "=&v"(r.s), "=&v"(r.x),
              "=&v"(r.done)
            : "v"(lo), "v"(zero), "s"(gates), "s"(ga), "s"(state), "s"(xin), "s"(done)
            : "memory");
}

// Every later use of the set depends on this statement's outputs, so none can be moved
// in front of the wait.
template <int N, bool TWO_GRADS, int G16>
__device__ __forceinline__ void sweep_wait(StepIn<G16>& r) {
    if (TWO_GRADS)
        asm volatile("s_waitcnt vmcnt(%8)"
                     : "+v"(r.zh), "+v"(r.zg), "+v"(r.zp), "+v"(r.ga), "+v"(r.gb), "+v"(r.s),
                       "+v"(r.x), "+v"(r.done)
                     : "n"(N));
    else
        asm volatile("s_waitcnt vmcnt(%7)"
                     : "+v"(r.zh), "+v"(r.zg), "+v"(r.zp), "+v"(r.ga), "+v"(r.s), "+v"(r.x),
                       "+v"(r.done)
                     : "n"(N));
}

// Drain the queue; every set is an output, so nothing of any set is read before it.
template <bool TWO_GRADS, int G16>
__device__ __forceinline__ void sweep_drain(StepIn<G16>& p, StepIn<G16>& q, StepIn<G16>& r) {
    if (TWO_GRADS)
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(p.zh), "+v"(p.zg), "+v"(p.zp), "+v"(p.ga), "+v"(p.gb), "+v"(p.s),
                       "+v"(p.x), "+v"(p.done), "+v"(q.zh), "+v"(q.zg), "+v"(q.zp), "+v"(q.ga),
                       "+v"(q.gb), "+v"(q.s), "+v"(q.x), "+v"(q.done), "+v"(r.zh), "+v"(r.zg),
                       "+v"(r.zp), "+v"(r.ga), "+v"(r.gb), "+v"(r.s), "+v"(r.x), "+v"(r.done));
    else
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(p.zh), "+v"(p.zg), "+v"(p.zp), "+v"(p.ga), "+v"(p.s), "+v"(p.x),
                       "+v"(p.done), "+v"(q.zh), "+v"(q.zg), "+v"(q.zp), "+v"(q.ga), "+v"(q.s),
                       "+v"(q.x), "+v"(q.done), "+v"(r.zh), "+v"(r.zg), "+v"(r.zp), "+v"(r.ga),
                       "+v"(r.s), "+v"(r.x), "+v"(r.done));
}

// the trailing s_nop keeps the next instruction clear of the store data registers
template <bool HIGHWAY>
__device__ __forceinline__ void sweep_store(unsigned lo, unsigned, void* gates, void* hw,
                                            const f4& dzh, const f4& dzg, const f4& dzp,
                                            const f4& hwv) {
    if (HIGHWAY)
        asm volatile(
            "global_store_dwordx4 %0, %1, %5 nt\n\t"
            "global_store_dwordx4 %0, %2, %5 offset:1024 nt\n\t"
            "global_store_dwordx4 %0, %3, %5 offset:2048 nt\n\t"
            "global_store_dwordx4 %0, %4, %6 nt\n\t"
            "s_nop 0"
            :
            : "v"(lo), "v"(dzh), "v"(dzg), "v"(dzp), "v"(hwv), "s"(gates), "s"(hw)
            : "memory");
    else
        asm volatile(
            "global_store_dwordx4 %0, %1, %4 nt\n\t"
            "global_store_dwordx4 %0, %2, %4 offset:1024 nt\n\t"
            "global_store_dwordx4 %0, %3, %4 offset:2048 nt\n\t"
            "s_nop 0"
            :
            : "v"(lo), "v"(dzh), "v"(dzg), "v"(dzp), "s"(gates)
            : "memory");
}
template <bool HIGHWAY>
__device__ __forceinline__ void sweep_store(unsigned, unsigned lo8, void* gates, void* hw,
                                            const u2& dzh, const u2& dzg, const u2& dzp,
                                            const u2& hwv) {
    if (HIGHWAY)
        asm volatile(
            "global_store_dwordx2 %0, %1, %5 nt\n\t"
            "global_store_dwordx2 %0, %2, %5 offset:512 nt\n\t"
            "global_store_dwordx2 %0, %3, %5 offset:1024 nt\n\t"
            "global_store_dwordx2 %0, %4, %6 nt\n\t"
            "s_nop 0"
            :
            : "v"(lo8), "v"(dzh), "v"(dzg), "v"(dzp), "v"(hwv), "s"(gates), "s"(hw)
            : "memory");
    else
        asm volatile(
            "global_store_dwordx2 %0, %1, %4 nt\n\t"
            "global_store_dwordx2 %0, %2, %4 offset:512 nt\n\t"
            "global_store_dwordx2 %0, %3, %4 offset:1024 nt\n\t"
            "s_nop 0"
            :
            : "v"(lo8), "v"(dzh), "v"(dzg), "v"(dzp), "s"(gates)
            : "memory");
}

constexpr int kSweepEnvs = 1;   // envs (wavefronts) per workgroup: the best of 1 / 2 / 4
template <bool TWO_GRADS, bool HIGHWAY, int G16>
__global__ __launch_bounds__(64 * kSweepEnvs, 4) void k_gru_reverse(ReverseArgs a) {
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int env = (int)blockIdx.x * kSweepEnvs + wave;   // one wavefront per env of the minibatch
    const unsigned lane_off = (threadIdx.x & 63u) * 16u;   // units 4q .. 4q+3 of a 1 KiB fp32 row
    const unsigned lane_off8 = (threadIdx.x & 63u) * 8u;   // ... of a 512-byte bf16 row
    // wavefront-uniform row pointers of this env; a step back in time is one stride
    const size_t mbz = (size_t)a.w.mb;
    constexpr size_t kGateRow = G16 ? G * 2 : G * 4, kInRow = G16 ? H * 2 : H * 4;   // bytes
    char* const gates = reinterpret_cast<char*>(a.gates) + (size_t)env * kGateRow;
    const char* const xin = reinterpret_cast<const char*>(a.layer_in) + (size_t)env * kInRow;
    const char* const ga = reinterpret_cast<const char*>(a.grad_a) + (size_t)env * kInRow;
    const char* const gb =
        TWO_GRADS ? reinterpret_cast<const char*>(a.grad_b) + (size_t)env * kInRow : nullptr;
    char* const hw = HIGHWAY ? reinterpret_cast<char*>(a.highway_out) + (size_t)env * kInRow : nullptr;
    const size_t slab_env = (size_t)a.w.env_start + env;
    // the recorded state: rows of 256 fp32, or of 256 bf16 (G16 = 2); a step back is one stride
    constexpr size_t kStateRow = G16 == 2 ? H * 2 : H * 4;   // bytes
    const size_t state_step = (size_t)a.layers * a.w.n_all * kStateRow;
    const char* const state = reinterpret_cast<const char*>(a.slab_state) +
                              (((size_t)a.w.t0 * a.layers + a.layer) * a.w.n_all + slab_env) * kStateRow;
    const uint8_t* const done = a.slab_done + (size_t)a.w.t0 * a.w.n_all + slab_env;
    // Every stage fetches, so that the number of operations in flight is the same at
    // every wait; a stage with no step left to fetch reads rows of the carry array
    // instead (cache-resident, never used).  Three consecutive rows must exist.
    const f4* const idle = reinterpret_cast<const f4*>(a.carry) +
                           (size_t)(env < a.w.mb - 2 ? env : a.w.mb - 3) * H4;

    auto fetch = [&](int s, StepIn<G16>& r) {   // s < 0: nothing left, an idle fetch
        const bool real = s >= 0;
        const size_t c = (size_t)(real ? s : 0) * mbz;
        sweep_fetch<TWO_GRADS, G16>(
            r, lane_off, lane_off8, real ? (const void*)(gates + c * kGateRow) : (const void*)idle,
            real ? (const void*)(ga + c * kInRow) : (const void*)idle,
            TWO_GRADS ? (real ? (const void*)(gb + c * kInRow) : (const void*)idle) : nullptr,
            real ? (const void*)(state + (size_t)s * state_step) : (const void*)idle,
            real ? (const void*)(xin + c * kInRow) : (const void*)idle,
            done + (size_t)(real ? s : 0) * a.w.n_all);
    };

    f4* const carry_p = reinterpret_cast<f4*>(a.carry) + (size_t)env * H4 + (threadIdx.x & 63u);
    f4 carry = *carry_p;
    // the recurrence is cut behind the last step of the rollout and of every BPTT
    // segment: `phase` = (t + 1) % seg of the step about to be consumed
    const int last = a.steps - 1;
    int phase = (a.w.t0 + last + 1) % a.seg;

    auto consume = [&](int s, const StepIn<G16>& in) {
        if (a.w.t0 + s == a.horizon - 1 || phase == 0) carry = f4{0.0f, 0.0f, 0.0f, 0.0f};
        phase = (phase == 0 ? a.seg : phase) - 1;
        const float pass = (in.done & 0xffu) ? 0.0f : 1.0f;   // a terminal step hands nothing back
        const f4 zh = widen(in.zh), zg = widen(in.zg), zp = widen(in.zp), x = widen(in.x);
        const f4 sv = widen(in.s);
        const f4 ga_v = widen(in.ga);
        f4 gb_v = f4{0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (TWO_GRADS) gb_v = widen(in.gb);
        f4 dzh, dzg, dzp, hwv;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float sg = sigmoid_fast(zg[j]);
            const float mix = sigmoid_fast(zp[j]);
            const float sh = sigmoid_fast(zh[j]);
            const bool lin = zh[j] >= 0.0f;
            const float cand = lin ? zh[j] + 0.5f : sh;              // g(zh)
            const float dcand = lin ? 1.0f : sh * (1.0f - sh);       // g'(zh)
            const float gap = cand - sv[j];
            const float h_new = sv[j] + sg * gap;
            const float g_top = TWO_GRADS ? ga_v[j] + gb_v[j] : ga_v[j];
            const float g_h = g_top * mix + pass * carry[j];
            dzp[j] = g_top * (h_new - x[j]) * mix * (1.0f - mix);
            hwv[j] = g_top * (1.0f - mix);
            carry[j] = g_h * (1.0f - sg);
            dzg[j] = g_h * gap * sg * (1.0f - sg);
            dzh[j] = g_h * sg * dcand;
        }
        const size_t c = (size_t)s * mbz;
        if constexpr (G16)
            sweep_store<HIGHWAY>(lane_off, lane_off8, gates + c * kGateRow,
                                 HIGHWAY ? hw + c * kInRow : nullptr, narrow(dzh), narrow(dzg),
                                 narrow(dzp), narrow(hwv));
        else
            sweep_store<HIGHWAY>(lane_off, lane_off8, gates + c * kGateRow,
                                 HIGHWAY ? hw + c * kInRow : nullptr, dzh, dzg, dzp, hwv);
    };

    // Operations per stage: NL loads then (after the step's arithmetic) NS stores.
    // When a set is waited for, the younger operations are the two fetches behind it and
    // the stores of the stages in between: two stages' worth in the steady state, fewer
    // stores in the first round.  A round is straight-line code: no control flow ever
    // merges registers whose loads are in flight.
    constexpr int NL = TWO_GRADS ? 8 : 7, NS = HIGHWAY ? 4 : 3;
    StepIn<G16> b0, b1, b2;
    fetch(last, b0);
    fetch(last - 1, b1);
    fetch(last - 2, b2);
#define CFP_SWEEP_ROUND(s_, N0, N1, N2)                      \
    do {                                                     \
        sweep_wait<(N0), TWO_GRADS, G16>(b0);                \
        consume((s_), b0);                                   \
        fetch((s_) - 3, b0);                                 \
        sweep_wait<(N1), TWO_GRADS, G16>(b1);                \
        consume((s_) - 1, b1);                               \
        fetch((s_) - 4, b1);                                 \
        sweep_wait<(N2), TWO_GRADS, G16>(b2);                \
        consume((s_) - 2, b2);                               \
        fetch((s_) - 5, b2);                                 \
    } while (0)
    int s = last;
    if (s >= 2) {
        CFP_SWEEP_ROUND(s, 2 * NL, 2 * NL + NS, 2 * NL + 2 * NS);
        for (s -= 3; s >= 2; s -= 3)
            CFP_SWEEP_ROUND(s, 2 * NL + 2 * NS, 2 * NL + 2 * NS, 2 * NL + 2 * NS);
    }
#undef CFP_SWEEP_ROUND
    // at most two steps are left, in b0 then b1; everything in flight lands first
    sweep_drain<TWO_GRADS, G16>(b0, b1, b2);
    if (s >= 0) consume(s, b0);
    if (s >= 1) consume(s - 1, b1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    *carry_p = carry;
}

// ---- window recompute of one layer from the stored state (unfused chain) -----------
__global__ __launch_bounds__(256) void k_gru_replay(const f4* __restrict__ gates,
                                                    const f4* __restrict__ xin,
                                                    const f4* __restrict__ slab_state,
                                                    f4* __restrict__ xout, WindowMap w,
                                                    size_t total4, int layer, int layers) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total4) return;
    const int q = (int)(i & (H4 - 1));
    const size_t col = i / H4;
    const size_t tr = col / (size_t)w.mb, el = col - tr * (size_t)w.mb;
    const size_t so = ((((size_t)w.t0 + tr) * layers + layer) * w.n_all + w.env_start + el) * H4 + q;
    const f4 s = ld_stream(slab_state + so);
    const f4 zh = ld_stream(gates + col * G4 + q);
    const f4 zg = ld_stream(gates + col * G4 + H4 + q);
    const f4 zp = ld_stream(gates + col * G4 + 2 * H4 + q);
    const f4 x = ld_stream(xin + i);
    f4 o;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float cand = zh[j] >= 0.0f ? zh[j] + 0.5f : sigmoid_fast(zh[j]);
        const float h_new = s[j] + sigmoid_fast(zg[j]) * (cand - s[j]);
        const float mix = sigmoid_fast(zp[j]);
        o[j] = mix * h_new + (1.0f - mix) * x[j];
    }
    xout[i] = o;
}

// ---- PPO head ------------------------------------------------------------------------
constexpr int kHeadCols = 64;      // columns per workgroup, four lanes each
constexpr int kHeadStride = 49;    // LDS row stride of the staged rows (odd)
constexpr int kHeadSlots = 11;     // actions per lane: a = q + 4 i

template <bool GRAD>
__global__ __launch_bounds__(256) void k_ppo_head(HeadArgs a) {
    __shared__ float rows_s[kHeadCols * kHeadStride];
    __shared__ __attribute__((aligned(16))) float grad_s[kHeadCols * kHeadGradLd];
    __shared__ double loss_s[4][3];
    const int tid = threadIdx.x;
    const int col0 = (int)blockIdx.x * kHeadCols;
    const int nb = min(kHeadCols, a.cols - col0);
    {   // rows of this workgroup: one contiguous piece, 16 bytes per lane
        const int ld4 = a.ld / 4;
        const f4* src = reinterpret_cast<const f4*>(a.rows + (size_t)col0 * a.ld);
        for (int i = tid; i < nb * ld4; i += 256) {
            const f4 v = src[i];
            const int r = i / ld4, c4 = i - r * ld4;
            float* d = rows_s + r * kHeadStride + 4 * c4;
            d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
        }
    }
    __syncthreads();
    const int cl = min(tid >> 2, nb - 1), q = tid & 3;   // lanes past the end shadow the last column
    const bool live = (tid >> 2) < nb;
    const int col = col0 + cl;
    const int step = col / a.w.mb;
    const size_t o = (size_t)(a.w.t0 + step) * a.w.n_all + a.w.env_start + (col - step * a.w.mb);
    const float* row = rows_s + cl * kHeadStride;

    float lg[kHeadSlots];
    float top = -INFINITY;
#pragma unroll
    for (int i = 0; i < kHeadSlots; i++) {
        const int act = q + 4 * i;
        lg[i] = act < A ? row[act] + (a.bias_a ? a.bias_a[act] : 0.0f) : -INFINITY;
        top = fmaxf(top, lg[i]);
    }
    top = fmaxf(top, __shfl_xor(top, 1, 4));
    top = fmaxf(top, __shfl_xor(top, 2, 4));
    float ex[kHeadSlots];
    float mass = 0.0f;
#pragma unroll
    for (int i = 0; i < kHeadSlots; i++) {
        ex[i] = expf(lg[i] - top);   // exp(-inf) = 0 for the one slot past the actions
        mass += ex[i];
    }
    mass += __shfl_xor(mass, 1, 4);
    mass += __shfl_xor(mass, 2, 4);
    const float lse = top + logf(mass);
    const float inv_mass = 1.0f / mass;
    const int taken = a.act[o];
    float lp_taken = 0.0f, ent = 0.0f;
    float lp[kHeadSlots], pi[kHeadSlots];
#pragma unroll
    for (int i = 0; i < kHeadSlots; i++) {
        const int act = q + 4 * i;
        lp[i] = act < A ? lg[i] - lse : 0.0f;
        pi[i] = ex[i] * inv_mass;
        ent -= pi[i] * lp[i];
        lp_taken += act == taken ? lp[i] : 0.0f;
    }
    ent += __shfl_xor(ent, 1, 4);
    ent += __shfl_xor(ent, 2, 4);
    lp_taken += __shfl_xor(lp_taken, 1, 4);   // three of the four terms are zero: exact
    lp_taken += __shfl_xor(lp_taken, 2, 4);

    // advantage normalised with the moments of the whole rollout
    const double inv_count = 1.0 / ((double)a.w.n_all * (double)a.horizon);
    const double mean = a.adv_moments[0] * inv_count;
    const double var = a.adv_moments[1] * inv_count - mean * mean;
    const float inv_std = 1.0f / ((float)sqrt(var > 0.0 ? var : 0.0) + 1e-8f);
    const float adv = (a.adv[o] - (float)mean) * inv_std;
    const float ratio = expf(lp_taken - a.old_logp[o]);
    const float plain = ratio * adv;
    const float clipped = fminf(fmaxf(ratio, 1.0f - a.clip), 1.0f + a.clip) * adv;
    const float value = row[A] + (a.bias_v ? a.bias_v[0] : 0.0f);
    const float verr = value - a.ret[o];

    if (GRAD) {
        // d(-min(plain, clipped)) / d log pi(taken): zero where the clipped branch is active
        const float w_taken = plain <= clipped ? -adv * ratio : 0.0f;
        const float ent_coef = a.ent_coef[0];
        const float scale = 1.0f / ((float)a.horizon * (float)a.w.mb);
        float* out = grad_s + cl * kHeadGradLd;
        if (live) {
#pragma unroll
            for (int i = 0; i < kHeadSlots; i++) {
                const int act = q + 4 * i;
                const float d = w_taken * ((act == taken ? 1.0f : 0.0f) - pi[i]) +
                                ent_coef * pi[i] * (lp[i] + ent);
                out[act] = act < A ? d * scale : scale * a.vf * verr;   // slot 43: the value
            }
            out[A + 1 + q] = 0.0f;
        }
        __syncthreads();
        f4* dst = reinterpret_cast<f4*>(a.grad_rows + (size_t)col0 * kHeadGradLd);
        const f4* g4 = reinterpret_cast<const f4*>(grad_s);
        for (int i = tid; i < nb * (kHeadGradLd / 4); i += 256) dst[i] = g4[i];
    }

    // loss terms: one lane per column contributes, fixed-order sums over the workgroup
    const bool counts = live && q == 0;
    const double t0 = wave_sum(counts ? (double)(-fminf(plain, clipped)) : 0.0);
    const double t1 = wave_sum(counts ? (double)(0.5f * verr * verr) : 0.0);
    const double t2 = wave_sum(counts ? (double)ent : 0.0);
    if ((tid & 63) == 0) {
        loss_s[tid >> 6][0] = t0; loss_s[tid >> 6][1] = t1; loss_s[tid >> 6][2] = t2;
    }
    __syncthreads();
    if (tid < 3)
        a.block_loss[3 * (size_t)blockIdx.x + tid] =
            (loss_s[0][tid] + loss_s[1][tid]) + (loss_s[2][tid] + loss_s[3][tid]);
}

// acc[q] (+)= sum_b part[b*NQ + q]: lane c of row q adds its contiguous chunk of the
// blocks in ascending order, then lane 0 adds the 64 chunk sums in ascending order.
template <int NQ>
__global__ __launch_bounds__(64 * NQ) void k_fold_f64(const double* __restrict__ part, int blocks,
                                                      double* __restrict__ acc, int accumulate) {
    __shared__ double chunk[NQ][64];
    const int q = threadIdx.x >> 6, c = threadIdx.x & 63;
    const int per = (blocks + 63) / 64;
    const int b1 = min(blocks, (c + 1) * per);
    double s = 0.0;
    for (int b = c * per; b < b1; b++) s += part[(size_t)b * NQ + q];
    chunk[q][c] = s;
    __syncthreads();
    if (c == 0) {
        double t = 0.0;
        for (int i = 0; i < 64; i++) t += chunk[q][i];
        acc[q] = accumulate ? acc[q] + t : t;
    }
}

// ---- GAE and advantage moments ---------------------------------------------------------
constexpr int kGaeLanes = 64;

__global__ __launch_bounds__(kGaeLanes) void k_gae_moments(
    const float* __restrict__ values, const float* __restrict__ rewards,
    const uint8_t* __restrict__ dones, const float* __restrict__ v_boot, float* __restrict__ adv,
    float* __restrict__ ret, int n, int T, float gamma, float lam, double* __restrict__ part) {
    const int e = (int)blockIdx.x * kGaeLanes + (int)threadIdx.x;
    const bool live = e < n;
    const int ec = live ? e : n - 1;
    double m1 = 0.0, m2 = 0.0;
    float ahead = v_boot[ec];   // V(s_{t+1})
    float run = 0.0f;           // A_{t+1}
    const float decay = gamma * lam;
    constexpr int B = 8;        // steps whose loads are in flight together
    for (int hi = T; hi > 0; hi -= B) {
        const int cnt = hi < B ? hi : B;
        float v[B], r[B];
        uint8_t d[B];
#pragma unroll
        for (int i = 0; i < B; i++) {
            const size_t o = (size_t)(i < cnt ? hi - 1 - i : 0) * n + ec;
            v[i] = values[o]; r[i] = rewards[o]; d[i] = dones[o];
        }
#pragma unroll
        for (int i = 0; i < B; i++) {
            if (i >= cnt) break;
            const size_t o = (size_t)(hi - 1 - i) * n + ec;
            const float keep = d[i] ? 0.0f : 1.0f;
            const float td = r[i] + gamma * ahead * keep - v[i];
            run = td + decay * keep * run;
            if (live) { adv[o] = run; ret[o] = run + v[i]; }
            m1 += run; m2 += (double)run * (double)run;
            ahead = v[i];
        }
    }
    const double s1 = wave_sum(live ? m1 : 0.0), s2 = wave_sum(live ? m2 : 0.0);
    if (threadIdx.x == 0) { part[2 * blockIdx.x] = s1; part[2 * blockIdx.x + 1] = s2; }
}

// moments alone, for advantages the caller filled in: 16-byte loads, a grid-stride walk
__global__ __launch_bounds__(256) void k_adv_moments(const f4* __restrict__ adv4, size_t count4,
                                                     const float* __restrict__ adv, size_t count,
                                                     double* __restrict__ part) {
    __shared__ double ws[4][2];
    double m1 = 0.0, m2 = 0.0;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count4; i += stride) {
        const f4 v = adv4[i];
#pragma unroll
        for (int j = 0; j < 4; j++) { m1 += v[j]; m2 += (double)v[j] * (double)v[j]; }
    }
    if (blockIdx.x == 0)   // the up to three values past the last whole group
        for (size_t i = 4 * count4 + threadIdx.x; i < count; i += 256) {
            m1 += adv[i]; m2 += (double)adv[i] * (double)adv[i];
        }
    m1 = wave_sum(m1); m2 = wave_sum(m2);
    if ((threadIdx.x & 63) == 0) { ws[threadIdx.x >> 6][0] = m1; ws[threadIdx.x >> 6][1] = m2; }
    __syncthreads();
    if (threadIdx.x < 2)
        part[2 * blockIdx.x + threadIdx.x] = (ws[0][threadIdx.x] + ws[1][threadIdx.x]) +
                                             (ws[2][threadIdx.x] + ws[3][threadIdx.x]);
}

// ---- Adam with the weight mirrors written in the same pass ------------------------------
// Positions of a weight inside the MFMA-ordered mirrors: the inverse of the index maps of
// k_pack_enc / k_pack_gru / k_pack_av (policy_forward.hip), k_pack_enc_split and the bf16
// packers (policy_forward_bf16.hip).  A K block is 8 wide in the fp32 mirrors (lane
// half h carries k = 8 kb + 4 h + j) and 16 wide in the bf16 ones (k = 16 kb + 8 h + j).
struct AdamArgs {
    float* params; float* grads; float* m; float* v;
    const uint64_t* step_ctr; const float* lr;
    float beta1, beta2, eps;
    float* we_pk; __bf16* we_s3; __bf16* we_bf;
    float* wg_pk; __bf16* wg_bf;
    float* wav_pk; __bf16* wav_bf;
    int layers;
    int enc_items, mid_items, tail_items;   // lanes of the three ranges below
    int off_b_enc, off_w_gru, off_w_a, off_b_a, off_w_v, off_b_v;
};

struct AdamCoef { float lr, c1, c2; };

__device__ __forceinline__ float adam_one(const AdamArgs& a, const AdamCoef& k, size_t i) {
    const float g = a.grads[i];
    a.grads[i] = 0.0f;
    const float m = a.beta1 * a.m[i] + (1.0f - a.beta1) * g;
    const float v = a.beta2 * a.v[i] + (1.0f - a.beta2) * g * g;
    a.m[i] = m;
    a.v[i] = v;
    const float w = a.params[i] - k.lr * (m / k.c1) / (sqrtf(v / k.c2) + a.eps);
    a.params[i] = w;
    return w;
}

__device__ __forceinline__ f4 adam_four(const AdamArgs& a, const AdamCoef& k, size_t i) {
    f4* g4 = reinterpret_cast<f4*>(a.grads + i);
    f4* m4 = reinterpret_cast<f4*>(a.m + i);
    f4* v4 = reinterpret_cast<f4*>(a.v + i);
    f4* p4 = reinterpret_cast<f4*>(a.params + i);
    const f4 g = *g4;
    f4 m = *m4, v = *v4, w = *p4;
    *g4 = f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        m[j] = a.beta1 * m[j] + (1.0f - a.beta1) * g[j];
        v[j] = a.beta2 * v[j] + (1.0f - a.beta2) * g[j] * g[j];
        w[j] -= k.lr * (m[j] / k.c1) / (sqrtf(v[j] / k.c2) + a.eps);
    }
    *m4 = m; *v4 = v; *p4 = w;
    return w;
}

__device__ __forceinline__ void put_bf16x4(__bf16* dst, const f4& w) {
    *reinterpret_cast<bf16x4*>(dst) = __builtin_convertvector(w, bf16x4);
}

__global__ __launch_bounds__(256) void k_adam_mirrors(AdamArgs a) {
    AdamCoef k;
    k.lr = a.lr[0];
    const float step = (float)((int)a.step_ctr[0] + 1);
    k.c1 = 1.0f - powf(a.beta1, step);
    k.c2 = 1.0f - powf(a.beta2, step);
    int it = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (it < a.enc_items) {
        // W_enc[f][u]: four consecutive features 4 fq .. 4 fq + 3 of one unit (a wavefront
        // covers 64 consecutive units of each of the four rows)
        const int fq = it >> 8, u = it & 255;
        const int wave = u >> 6, ut = (u >> 5) & 1, l32 = u & 31;
        f4 w;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int f = 4 * fq + j;
            w[j] = f < CFP_OBS ? adam_one(a, k, (size_t)f * H + u) : 0.0f;
        }
        {   // fp32 mirror: K block fq / 2, lane half fq % 2
            const int kb = fq >> 1, lane = (fq & 1) * 32 + l32;
            reinterpret_cast<f4*>(a.we_pk)[((kb * 4 + wave) * 2 + ut) * 64 + lane] = w;
        }
        const int kb16 = fq >> 2, lane16 = ((fq >> 1) & 1) * 32 + l32, j8 = (fq & 1) * 4;
        put_bf16x4(a.we_bf + ((size_t)((kb16 * 4 + wave) * 2 + ut) * 64 + lane16) * 8 + j8, w);
        if (4 * fq < CFP_OBS_MAP) {   // the byte-valued features: hi + mid + lo = w exactly
            f4 hi, mid, lo;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const __bf16 h = (__bf16)w[j];
                const float r1 = w[j] - (float)h;
                const __bf16 md = (__bf16)r1;
                hi[j] = (float)h; mid[j] = (float)md; lo[j] = r1 - (float)md;
            }
            __bf16* s3 = a.we_s3 + ((size_t)(((kb16 * 4 + wave) * 2 + ut) * 3) * 64 + lane16) * 8 + j8;
            put_bf16x4(s3, hi);
            put_bf16x4(s3 + 64 * 8, mid);
            put_bf16x4(s3 + 2 * 64 * 8, lo);
        }
        return;
    }
    it -= a.enc_items;
    if (it < a.mid_items) {
        // [b_enc | W_gru | W_a]: four consecutive floats of the arena
        const int o = a.off_b_enc + 4 * it;
        const f4 w = adam_four(a, k, (size_t)o);
        if (o < a.off_w_gru) return;   // b_enc is read from the arena
        if (o < a.off_w_a) {
            const int i = o - a.off_w_gru;
            const int layer = i / (G * H), r = (i / H) % G, k0 = i % H;
            const int gate = r >> 8, u = r & 255, wave = u >> 6, t = 2 * gate + ((u >> 5) & 1);
            const int l32 = u & 31;
            {
                const int kb = k0 >> 3, lane = ((k0 >> 2) & 1) * 32 + l32;
                reinterpret_cast<f4*>(a.wg_pk)[(size_t)layer * (G * H / 4) +
                                               ((kb * 4 + wave) * 6 + t) * 64 + lane] = w;
            }
            const int kb16 = k0 >> 4, lane16 = ((k0 >> 3) & 1) * 32 + l32, j8 = k0 & 4;
            put_bf16x4(a.wg_bf + (size_t)layer * (G * H) +
                           ((size_t)((kb16 * 4 + wave) * 6 + t) * 64 + lane16) * 8 + j8, w);
        } else {
            const int i = o - a.off_w_a;
            const int arow = i / H, k0 = i % H, nt = arow >> 5, l32 = arow & 31;
            {
                const int kb = k0 >> 3, lane = ((k0 >> 2) & 1) * 32 + l32;
                reinterpret_cast<f4*>(a.wav_pk)[(kb * 2 + nt) * 64 + lane] = w;
            }
            const int kb16 = k0 >> 4, lane16 = ((k0 >> 3) & 1) * 32 + l32, j8 = k0 & 4;
            put_bf16x4(a.wav_bf + ((size_t)(kb16 * 2 + nt) * 64 + lane16) * 8 + j8, w);
        }
        return;
    }
    it -= a.mid_items;
    if (it < a.tail_items) {
        // [b_a | W_v | b_v]: not 16-byte aligned in the arena, one float per lane
        const int o = a.off_b_a + it;
        const float w = adam_one(a, k, (size_t)o);
        if (o >= a.off_w_v && o < a.off_b_v) {   // W_v is row 43 of the fused head mirror
            const int k0 = o - a.off_w_v, nt = A >> 5, l32 = A & 31;
            a.wav_pk[((size_t)((k0 >> 3) * 2 + nt) * 64 + ((k0 >> 2) & 1) * 32 + l32) * 4 + (k0 & 3)] = w;
            a.wav_bf[((size_t)((k0 >> 4) * 2 + nt) * 64 + ((k0 >> 3) & 1) * 32 + l32) * 8 + (k0 & 7)] =
                (__bf16)w;
        }
    }
}

}  // namespace

int launch_gru_reverse(const ReverseArgs& a, hipStream_t st) {
    CFP_REQUIRE(a.gates && a.layer_in && a.grad_a && a.slab_state && a.slab_done && a.carry &&
                    a.steps > 0 && a.w.mb > 0 && a.w.mb % kSweepEnvs == 0 && a.seg > 0,
                "reverse MinGRU sweep: bad arguments");
    const dim3 grid(a.w.mb / kSweepEnvs), blk(64 * kSweepEnvs);
    CFP_REQUIRE(a.w.mb >= 3, "reverse MinGRU sweep: at least three envs");
#define CFP_SWEEP_LAUNCH(G16)                                                                         \
    do {                                                                                              \
        if (a.grad_b && a.highway_out)                                                                \
            hipLaunchKernelGGL((k_gru_reverse<true, true, G16>), grid, blk, 0, st, a);                \
        else if (a.grad_b) hipLaunchKernelGGL((k_gru_reverse<true, false, G16>), grid, blk, 0, st, a); \
        else if (a.highway_out)                                                                       \
            hipLaunchKernelGGL((k_gru_reverse<false, true, G16>), grid, blk, 0, st, a);               \
        else hipLaunchKernelGGL((k_gru_reverse<false, false, G16>), grid, blk, 0, st, a);             \
    } while (0)
    CFP_REQUIRE(!a.state_bf16 || a.gates_bf16, "a bf16 state slab goes with the bf16 storage of the window");
    if (a.gates_bf16 && a.state_bf16) CFP_SWEEP_LAUNCH(2);
    else if (a.gates_bf16) CFP_SWEEP_LAUNCH(1);
    else CFP_SWEEP_LAUNCH(0);
#undef CFP_SWEEP_LAUNCH
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int launch_gru_replay(const float* gates, const float* layer_in, const float* slab_state,
                      float* layer_out, const WindowMap& w, int cols, int layer, int layers,
                      hipStream_t st) {
    const size_t total4 = (size_t)cols * H4;
    hipLaunchKernelGGL(k_gru_replay, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const f4*>(gates), reinterpret_cast<const f4*>(layer_in),
                       reinterpret_cast<const f4*>(slab_state), reinterpret_cast<f4*>(layer_out), w,
                       total4, layer, layers);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int head_blocks(int cols) { return (cols + kHeadCols - 1) / kHeadCols; }

int launch_head(const HeadArgs& a, hipStream_t st) {
    CFP_REQUIRE(a.rows && a.cols > 0 && (a.ld == 44 || a.ld == 48) && a.block_loss && a.w.mb > 0 &&
                    (reinterpret_cast<uintptr_t>(a.rows) & 15u) == 0 &&
                    (reinterpret_cast<uintptr_t>(a.grad_rows) & 15u) == 0,
                "PPO head: rows must be 44 or 48 floats wide and 16-byte aligned");
    const dim3 grid(head_blocks(a.cols)), blk(256);
    if (a.grad_rows) hipLaunchKernelGGL(k_ppo_head<true>, grid, blk, 0, st, a);
    else hipLaunchKernelGGL(k_ppo_head<false>, grid, blk, 0, st, a);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int launch_fold_f64(const double* part, int blocks, int nq, double* acc, bool accumulate,
                    hipStream_t st) {
    CFP_REQUIRE(nq == 2 || nq == 3, "fold: 2 or 3 sums");
    if (nq == 2)
        hipLaunchKernelGGL(k_fold_f64<2>, dim3(1), dim3(128), 0, st, part, blocks, acc, accumulate ? 1 : 0);
    else
        hipLaunchKernelGGL(k_fold_f64<3>, dim3(1), dim3(192), 0, st, part, blocks, acc, accumulate ? 1 : 0);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int gae_blocks(int n) { return (n + kGaeLanes - 1) / kGaeLanes; }

int launch_gae(const float* values, const float* rewards, const uint8_t* dones,
               const float* v_boot, float* adv, float* ret, int n, int T, float gamma, float lam,
               double* part, double* moments, hipStream_t st) {
    hipLaunchKernelGGL(k_gae_moments, dim3(gae_blocks(n)), dim3(kGaeLanes), 0, st, values, rewards,
                       dones, v_boot, adv, ret, n, T, gamma, lam, part);
    CFP_HIP_TRY(hipGetLastError());
    return launch_fold_f64(part, gae_blocks(n), 2, moments, false, st);
}

int launch_adv_moments(const float* adv, size_t count, double* part, double* moments,
                       hipStream_t st) {
    const size_t count4 = (reinterpret_cast<uintptr_t>(adv) & 15u) == 0 ? count / 4 : 0;
    hipLaunchKernelGGL(k_adv_moments, dim3(kMomentBlocks), dim3(256), 0, st,
                       reinterpret_cast<const f4*>(adv), count4, adv, count, part);
    CFP_HIP_TRY(hipGetLastError());
    return launch_fold_f64(part, kMomentBlocks, 2, moments, false, st);
}

int launch_adam(cfp_policy* p, float* grads, float* m, float* v, const uint64_t* step_ctr,
                const float* lr, float beta1, float beta2, float eps, hipStream_t st) {
    CFP_REQUIRE(p && p->variant == 0, "Adam with mirrors covers the full-game policy");
    const int L = p->layers;
    AdamArgs a{};
    a.params = p->params; a.grads = grads; a.m = m; a.v = v;
    a.step_ctr = step_ctr; a.lr = lr;
    a.beta1 = beta1; a.beta2 = beta2; a.eps = eps;
    a.we_pk = p->we_pk; a.we_s3 = reinterpret_cast<__bf16*>(p->we_s3);
    a.we_bf = reinterpret_cast<__bf16*>(p->we_bf);
    a.wg_pk = p->wg_pk; a.wg_bf = reinterpret_cast<__bf16*>(p->wg_bf);
    a.wav_pk = p->wav_pk; a.wav_bf = reinterpret_cast<__bf16*>(p->wav_bf);
    a.layers = L;
    a.off_b_enc = CFP_OFF_B_ENC; a.off_w_gru = CFP_OFF_W_GRU; a.off_w_a = CFP_OFF_W_A(L);
    a.off_b_a = CFP_OFF_B_A(L); a.off_w_v = CFP_OFF_W_V(L); a.off_b_v = CFP_OFF_B_V(L);
    static_assert(CFP_OFF_B_ENC % 4 == 0 && CFP_OFF_W_GRU % 4 == 0 && (CFP_GRU * CFP_HIDDEN) % 4 == 0 &&
                      (CFP_ACTIONS * CFP_HIDDEN) % 4 == 0,
                  "the middle range walks the arena in aligned groups of four");
    a.enc_items = ((CFP_OBS + 3) / 4) * H;
    a.mid_items = (a.off_b_a - a.off_b_enc) / 4;
    a.tail_items = (int)p->param_count - a.off_b_a;
    const int items = a.enc_items + a.mid_items + a.tail_items;
    hipLaunchKernelGGL(k_adam_mirrors, dim3((items + 255) / 256), dim3(256), 0, st, a);
    CFP_HIP_TRY(hipGetLastError());
    // the 16-env-tile kernel's mirrors take one more pack launch.  Always, not only while that
    // mode is on: the switch can be flipped after this step (or after a capture of it), and a
    // forward on 16-env tiles must never see weights from before an update
    if (p->t16) return launch_pack_weights_t16(p->params, L, p->t16, st);
    return 0;
}

}  // namespace cfp
