// On-device PPO update: rollout slabs, windowed recompute backward, GAE,
// Adam.  Host-side mirror of the reference's CuTrain layer
// (craftax_full.cu:12637-13480).  The streaming kernels (reverse MinGRU sweep, head
// gradients, GAE, Adam) live in ppo_kernels.hip, the GEMMs behind the seam of
// gemm.hip / gemm_x9.hip; here: the window loop, the two-stream schedule, graph
// capture and the column sums (the reference's k_colsum family, :10442).
//   k_add_dv_wv :10224 is folded into the head's 48-wide gradient rows, k_vadd
//   :10069 into the layer-0 dh GEMM, which accumulates onto the highway term.
// All reductions are done in a fixed order (no float atomics), so a backward pass
// is bitwise reproducible run to run.
#include <chrono>
#include <vector>

#include "cfp_common.h"
#include "cfp_internal.h"
#include "ppo_kernels.h"
#include "../../include/cfp_env.h"
#include "env_internal.h"

namespace cfp {
namespace {

constexpr int H = CFP_HIDDEN, G = CFP_GRU, A = CFP_ACTIONS;

__global__ void k_fill(float* p, size_t count, float v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = v;
}
__global__ void k_fill_f64(double* p, int count) {
    if ((int)threadIdx.x < count) p[threadIdx.x] = 0.0;
}

// The head's gradient rows are 48 floats wide: [43 dlogits | dvalue | 0 0 0 0], and the
// head weights are mirrored as one [48][256] matrix [W_a ; W_v ; 0].  dh3 = rows . mirror
// then carries the value head's share (the reference's k_add_dv_wv pass,
// craftax_full.cu:10224), K = 48 suits the 16-wide MFMA steps, and one dW GEMM over 44
// rows yields dW_a and dW_v together (cu_gemv_dwv, :11655, needs no pass of its own).
constexpr int kHeadLd = kHeadGradLd;
__global__ void k_head_mirror(const float* __restrict__ W_a, const float* __restrict__ W_v,
                              float* __restrict__ out) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= kHeadLd * H) return;
    const int r = idx / H, k = idx - r * H;
    out[idx] = r < A ? W_a[idx] : (r == A ? W_v[k] : 0.0f);
}

// out[r] += sum_c src[c*ld + r]: partial sums over `slices` column ranges
// (grid.x), then folded in slice order by k_colsum_fold.  A workgroup covers RB rows
// with CL = 256 / RB threads each; a thread walks every CL-th column of the slice with
// four independent running sums (loads in flight instead of one dependent chain) and
// the CL sums of a row are added in thread order: a fixed order throughout.
// S16: src is a bf16 array (ld counts its elements).
template <bool S16>
__device__ __forceinline__ float colsum_at(const float* src, size_t i) {
    if (S16)
        return __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(src)[i] << 16);
    return src[i];
}
template <int RB, bool S16 = false>
__global__ __launch_bounds__(256) void k_colsum_partial(
    const float* __restrict__ src, int ld, float* __restrict__ part, int rows, int cols,
    int cols_per_slice) {
    constexpr int CL = 256 / RB;
    __shared__ float red[CL][RB];
    const int rl = threadIdx.x % RB, cl = threadIdx.x / RB;
    const int r = blockIdx.y * RB + rl;
    const int c0 = blockIdx.x * cols_per_slice;
    const int c1 = min(cols, c0 + cols_per_slice);
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    if (r < rows) {
        int c = c0 + cl;
        for (; c + 3 * CL < c1; c += 4 * CL) {
            s0 += colsum_at<S16>(src, (size_t)c * ld + r);
            s1 += colsum_at<S16>(src, (size_t)(c + CL) * ld + r);
            s2 += colsum_at<S16>(src, (size_t)(c + 2 * CL) * ld + r);
            s3 += colsum_at<S16>(src, (size_t)(c + 3 * CL) * ld + r);
        }
        for (; c < c1; c += CL) s0 += colsum_at<S16>(src, (size_t)c * ld + r);
    }
    red[cl][rl] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (cl == 0 && r < rows) {
        float t = red[0][rl];
#pragma unroll
        for (int i = 1; i < CL; i++) t += red[i][rl];
        part[(size_t)blockIdx.x * rows + r] = t;
    }
}
// Fixed order: thread (row, c) of 4 x 64 sums the slices of chunk c in ascending
// order, thread (row, 0) then adds the 64 chunk sums in ascending order.
__global__ __launch_bounds__(256) void k_colsum_fold(const float* __restrict__ part,
                                                     float* __restrict__ out, int rows,
                                                     int slices) {
    __shared__ float red[4][64];
    const int rl = threadIdx.x >> 6, c = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + rl;
    const int per = (slices + 63) / 64;
    float s = 0.0f;
    if (r < rows) {
        const int z1 = min(slices, (c + 1) * per);
        for (int z = c * per; z < z1; z++) s += part[(size_t)z * rows + r];
    }
    red[rl][c] = s;
    __syncthreads();
    if (c == 0 && r < rows) {
        float t = 0.0f;
        for (int i = 0; i < 64; i++) t += red[rl][i];
        out[r] += t;
    }
}

__global__ void k_bump_ctr(uint64_t* ctr) { *ctr += 1; }

__global__ void k_take_value(const float* __restrict__ av, float* __restrict__ value_row,
                             int n) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n) value_row[e] = av[(size_t)e * CFP_AV + A];
}
__global__ void k_done_to_float(const uint8_t* __restrict__ d, float* __restrict__ f, int n) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n) f[e] = d[e] ? 1.0f : 0.0f;
}

inline unsigned grid1(size_t total, int block = 256) {
    return (unsigned)((total + block - 1) / block);
}

}  // namespace
}  // namespace cfp

using namespace cfp;

struct cfp_trainer {
    cfp_policy* p = nullptr;
    cfp_ppo_config cfg{};
    int n = 0, T = 0, L = 0, mb = 0, win = 0;
    size_t cols_cap = 0;
    std::vector<void*> owned;
    // slabs
    uint8_t* r_obs = nullptr; float* r_state = nullptr; int32_t* r_act = nullptr;
    float *r_logprob = nullptr, *r_value = nullptr, *r_reward = nullptr;
    uint8_t* r_done = nullptr;
    float *adv = nullptr, *ret = nullptr, *v_boot = nullptr;
    double *stats = nullptr, *loss_acc = nullptr, *block_loss = nullptr, *stats_part = nullptr;
    float *grads = nullptr, *adam_m = nullptr, *adam_v = nullptr;
    uint64_t* adam_ctr = nullptr;
    uint64_t* step_ctr = nullptr;   // rollout steps taken (the sampler's offset), device side
    unsigned* ticket = nullptr;     // workgroup tickets of the in-launch counter bump; zero between launches
    float* boot_state = nullptr;    // [L][n][256] copy of the live state for the bootstrap value
    float *d_lr = nullptr, *d_ent = nullptr;
    // window workspace
    float* xobs = nullptr; float* x[CFP_MAX_LAYERS + 1] = {}; float* preb[CFP_MAX_LAYERS] = {};
    float *logitsb = nullptr, *dlogits = nullptr, *w_head = nullptr;
    float *dh3b = nullptr, *dhG = nullptr, *dhX = nullptr;
    float* dcarry[CFP_MAX_LAYERS] = {};
    float* colsum_part = nullptr;
    float* live = nullptr;     // [L][n][256] live state for the loss replay
    float* termf = nullptr;    // [n]
    float* av_tmp = nullptr;   // [n][44]
    // second stream of the backward pass (the layers' dependent chain alternates between
    // it and the caller's, see cfp_train_backward)
    hipStream_t st2 = nullptr;
    hipEvent_t ev_dh[CFP_MAX_LAYERS] = {};
    hipEvent_t ev_join = nullptr, ev_head = nullptr;
    // GEMM scratch owned by this trainer: `sw` for the chain's GEMMs, and a split
    // workspace per layer for the gate dW GEMMs that run beside the chain
    SeamWork sw;
    SeamWork sw_layer[CFP_MAX_LAYERS];
    float* dw_work2 = nullptr;
    size_t dw_work2_floats = 0;
    // cfp_train_update's captured iteration (epochs x minibatches x (backward, Adam)) and
    // the process-wide GEMM modes it was captured under
    hipGraph_t tgraph = nullptr;
    hipGraphExec_t texec = nullptr;
    int graph_split = -1, graph_bf16 = -1, graph_pol_bf16 = -1, graph_store16 = -1;
    // bf16 storage of the window's gate pre-activations / their gradients and of the
    // layer inputs (in effect with bf16 GEMM inputs on the split kernels only)
    int bf16_store = 0;
    // the r_state slab holds bf16 (cfp_train_set_bf16_rstate): written by the bf16-input forward
    // of the rollout, read by the bf16 window recompute and the bf16-storage sweep
    int rs16 = 0;
    int prof = 0;             // phase timers on: eager update, a sync at every phase boundary
    double prof_ms[4] = {0.0, 0.0, 0.0, 0.0};   // rollout, gae (+ bootstrap), backward, adam
    // GEMM mode of this trainer's update (cfp_train_set_gemm_mode); -1: the process-wide switch
    int gemm_bf16 = -1, gemm_split = -1;
    hipStream_t st_own = nullptr;   // capture stream when the caller passes the null stream
};

static constexpr int kColsumSlices = 1024;

extern "C" {

void cfp_train_destroy(cfp_trainer* tr) {
    if (!tr) return;
    if (tr->rs16 && tr->p) tr->p->rs_bf16 = 0;   // the policy no longer writes rows of a bf16 slab
    for (void* q : tr->owned) (void)hipFree(q);
    seam_work_destroy(&tr->sw);
    for (hipEvent_t e : tr->ev_dh)
        if (e) (void)hipEventDestroy(e);
    if (tr->ev_join) (void)hipEventDestroy(tr->ev_join);
    if (tr->ev_head) (void)hipEventDestroy(tr->ev_head);
    if (tr->texec) (void)hipGraphExecDestroy(tr->texec);
    if (tr->tgraph) (void)hipGraphDestroy(tr->tgraph);
    if (tr->st2) (void)hipStreamDestroy(tr->st2);
    if (tr->st_own) (void)hipStreamDestroy(tr->st_own);
    delete tr;
}

int cfp_ppo_defaults(cfp_ppo_config* cfg) {
    CFP_REQUIRE(cfg, "cfp_ppo_defaults: NULL");
    cfg->lr = 3e-4f; cfg->gamma = 0.99f; cfg->lam = 0.95f; cfg->clip = 0.2f;
    cfg->ent = 0.01f; cfg->vf = 0.5f; cfg->epochs = 1; cfg->minibatches = 1;
    cfg->bptt_split = 1; cfg->bwd_win = 0;
    return 0;
}

int cfp_train_create(cfp_trainer** out, cfp_policy* p, int T, const cfp_ppo_config* cfg) {
    CFP_REQUIRE(out && p && cfg, "cfp_train_create: NULL argument");
    *out = nullptr;
    CFP_REQUIRE(p->variant == 0, "the trainer covers the full-game policy only");
    CFP_REQUIRE(T > 0, "horizon must be positive (got %d)", T);
    CFP_REQUIRE(cfg->minibatches >= 1 && p->n % cfg->minibatches == 0,
                "minibatches must divide num_envs (%d %% %d != 0)", p->n,
                cfg->minibatches);
    const int mb = p->n / cfg->minibatches;
    CFP_REQUIRE(cfg->bptt_split >= 1 && T % cfg->bptt_split == 0 && mb % 32 == 0,
                "bptt_split must divide the horizon (%d %% %d != 0), and "
                "envs/minibatch must be a multiple of 32", T, cfg->bptt_split);
    cfp_trainer* tr = new cfp_trainer();
    tr->p = p; tr->cfg = *cfg; tr->n = p->n; tr->T = T; tr->L = p->layers; tr->mb = mb;
    // Window: the reference keeps 16 steps so that the workspace fits a 24-32 GB
    // card (craftax_full.cu:12657-12686); with 288 GB the default is the whole
    // horizon up to 262 144 window columns (~5.3 GB of fp32 workspace).
    int win = cfg->bwd_win > 0 ? cfg->bwd_win : (int)(262144 / mb);
    if (win < 1) win = 1;
    if (win > T) win = T;
    tr->win = win;
    tr->cols_cap = (size_t)win * mb;
    const size_t nt = (size_t)tr->n * T, hn = (size_t)H * tr->n, cc = tr->cols_cap;
    const size_t pc = p->param_count;
    auto alloc = [&](void** ptr, size_t bytes) -> bool {
        hipError_t e = hipMalloc(ptr, bytes);
        if (e != hipSuccess) {
            set_error("hipMalloc(%zu bytes) failed in cfp_train_create: %s", bytes,
                      hipGetErrorString(e));
            return false;
        }
        tr->owned.push_back(*ptr);
        return hipMemset(*ptr, 0, bytes) == hipSuccess;
    };
    bool ok = true;
#define TA(field, bytes) ok = ok && alloc((void**)&tr->field, (bytes))
    TA(r_obs, nt * CFP_REC_BYTES);
    TA(r_state, nt * tr->L * H * sizeof(float));
    TA(r_act, nt * sizeof(int32_t));
    TA(r_logprob, nt * sizeof(float));
    TA(r_value, nt * sizeof(float));
    TA(r_reward, nt * sizeof(float));
    TA(r_done, nt);
    TA(adv, nt * sizeof(float));
    TA(ret, nt * sizeof(float));
    TA(v_boot, (size_t)tr->n * sizeof(float));
    TA(stats, 2 * sizeof(double));
    TA(loss_acc, 3 * sizeof(double));
    TA(block_loss, 3 * sizeof(double) * (size_t)head_blocks((int)(cc > (size_t)tr->n ? cc : tr->n)));
    TA(stats_part, 2 * sizeof(double) * (size_t)(gae_blocks(tr->n) > kMomentBlocks ? gae_blocks(tr->n) : kMomentBlocks));
    TA(grads, pc * sizeof(float));
    TA(adam_m, pc * sizeof(float));
    TA(adam_v, pc * sizeof(float));
    TA(adam_ctr, sizeof(uint64_t));
    TA(step_ctr, sizeof(uint64_t));
    TA(ticket, sizeof(unsigned));
    TA(boot_state, (size_t)tr->L * hn * sizeof(float));
    TA(d_lr, sizeof(float));
    TA(d_ent, sizeof(float));
    TA(xobs, cc * kObsPad * sizeof(float));   // rows widened 843 -> 848: 16-byte aligned
    for (int l = 0; l <= tr->L; l++) TA(x[l], cc * H * sizeof(float));
    for (int l = 0; l < tr->L; l++) TA(preb[l], cc * G * sizeof(float));
    for (int l = 0; l < tr->L; l++) TA(dcarry[l], (size_t)mb * H * sizeof(float));
    TA(logitsb, cc * kHeadLd * sizeof(float));   // [cols][44] from the fused recompute, [cols][48] unfused
    TA(dlogits, cc * kHeadLd * sizeof(float));
    TA(w_head, (size_t)kHeadLd * H * sizeof(float));
    TA(dh3b, cc * H * sizeof(float));
    TA(dhG, cc * H * sizeof(float));
    TA(dhX, cc * H * sizeof(float));
    TA(colsum_part, (size_t)kColsumSlices * H * sizeof(float));
    TA(live, (size_t)tr->L * hn * sizeof(float));
    TA(termf, (size_t)tr->n * sizeof(float));
    TA(av_tmp, (size_t)tr->n * CFP_AV * sizeof(float));
    tr->dw_work2_floats = (size_t)48 * G * H;   // per layer: 48 splits of a gate dW
    TA(dw_work2, (size_t)tr->L * tr->dw_work2_floats * sizeof(float));
#undef TA
    if (ok) ok = seam_work_create(&tr->sw) == 0;
    for (int l = 0; ok && l < tr->L; l++) {
        tr->sw_layer[l].dw_part = tr->dw_work2 + (size_t)l * tr->dw_work2_floats;
        tr->sw_layer[l].dw_part_floats = tr->dw_work2_floats;
    }
    // default priority, as every stream of this library
    if (ok) ok = hipStreamCreateWithFlags(&tr->st2, hipStreamNonBlocking) == hipSuccess &&
                 hipEventCreateWithFlags(&tr->ev_join, hipEventDisableTiming) == hipSuccess &&
                 hipEventCreateWithFlags(&tr->ev_head, hipEventDisableTiming) == hipSuccess;
    for (int l = 0; ok && l < tr->L; l++)
        ok = hipEventCreateWithFlags(&tr->ev_dh[l], hipEventDisableTiming) == hipSuccess;
    if (ok) ok = hipMemcpy(tr->d_lr, &cfg->lr, 4, hipMemcpyHostToDevice) == hipSuccess &&
                 hipMemcpy(tr->d_ent, &cfg->ent, 4, hipMemcpyHostToDevice) == hipSuccess;
    if (!ok) {
        if (!*cfp_last_error()) set_error("cfp_train_create: device setup failed");
        cfp_train_destroy(tr);
        return 1;
    }
    *out = tr;
    return 0;
}

void* cfp_train_buffer(cfp_trainer* tr, int which) {
    if (!tr) return nullptr;
    switch (which) {
        case CFP_BUF_R_OBS: return tr->r_obs;
        case CFP_BUF_R_STATE: return tr->r_state;
        case CFP_BUF_R_ACT: return tr->r_act;
        case CFP_BUF_R_LOGPROB: return tr->r_logprob;
        case CFP_BUF_R_VALUE: return tr->r_value;
        case CFP_BUF_R_REWARD: return tr->r_reward;
        case CFP_BUF_R_DONE: return tr->r_done;
        case CFP_BUF_ADV: return tr->adv;
        case CFP_BUF_RET: return tr->ret;
        case CFP_BUF_V_BOOT: return tr->v_boot;
        case CFP_BUF_STATS: return tr->stats;
        case CFP_BUF_LOSS_ACC: return tr->loss_acc;
        case CFP_BUF_GRADS: return tr->grads;
        case CFP_BUF_ADAM_M: return tr->adam_m;
        case CFP_BUF_ADAM_V: return tr->adam_v;
        case CFP_BUF_LR: return tr->d_lr;
        case CFP_BUF_ENT: return tr->d_ent;
        case CFP_BUF_STEP_CTR: return tr->step_ctr;
        default: return nullptr;
    }
}

int cfp_train_set_bf16_storage(cfp_trainer* tr, int on) {
    CFP_REQUIRE(tr, "cfp_train_set_bf16_storage: NULL trainer");
    tr->bf16_store = on ? 1 : 0;
    return 0;
}
int cfp_train_bf16_storage(const cfp_trainer* tr) { return tr ? tr->bf16_store : -1; }

int cfp_train_set_bf16_rstate(cfp_trainer* tr, int on) {
    CFP_REQUIRE(tr, "cfp_train_set_bf16_rstate: NULL trainer");
    tr->rs16 = on ? 1 : 0;
    tr->p->rs_bf16 = tr->rs16;   // the policy's forward writes the rows of this trainer's slab
    return 0;
}
int cfp_train_bf16_rstate(const cfp_trainer* tr) { return tr ? tr->rs16 : -1; }

int cfp_train_set_profile(cfp_trainer* tr, int on) {
    CFP_REQUIRE(tr, "cfp_train_set_profile: NULL trainer");
    tr->prof = on ? 1 : 0;
    return 0;
}

int cfp_train_profile(cfp_trainer* tr, double* ms4, int reset) {
    CFP_REQUIRE(tr && ms4, "cfp_train_profile: NULL argument");
    for (int i = 0; i < 4; i++) {
        ms4[i] = tr->prof_ms[i];
        if (reset) tr->prof_ms[i] = 0.0;
    }
    return 0;
}

int cfp_train_set_gemm_mode(cfp_trainer* tr, int bf16, int split) {
    CFP_REQUIRE(tr, "cfp_train_set_gemm_mode: NULL trainer");
    CFP_REQUIRE(bf16 >= -1 && bf16 <= 1 && split >= -1 && split <= 3,
                "cfp_train_set_gemm_mode: bf16 must be -1, 0 or 1 and split -1, 0, 1 or 2 (got %d, %d)", bf16, split);
    tr->gemm_bf16 = bf16;
    tr->gemm_split = split;
    return 0;
}
int cfp_train_gemm_mode(const cfp_trainer* tr, int* bf16, int* split) {
    CFP_REQUIRE(tr && bf16 && split, "cfp_train_gemm_mode: NULL argument");
    *bf16 = tr->gemm_bf16 >= 0 ? tr->gemm_bf16 : cfp_get_gemm_bf16();
    *split = tr->gemm_split >= 0 ? tr->gemm_split : cfp_get_gemm_split();
    return 0;
}

int cfp_train_window(const cfp_trainer* tr) { return tr ? tr->win : 0; }
int cfp_train_minibatch(const cfp_trainer* tr) { return tr ? tr->mb : 0; }

// r_state rows of step t: [layers][n][256] fp32, or bf16 in a slab of 2-byte elements
static float* state_rows(cfp_trainer* tr, int t) {
    const size_t el = (size_t)t * tr->L * tr->n * H;
    return tr->rs16 ? reinterpret_cast<float*>(reinterpret_cast<uint16_t*>(tr->r_state) + el) : tr->r_state + el;
}

int cfp_train_record_step(cfp_trainer* tr, int t, const uint8_t* d_rec_row,
                          const float* d_terminals, void* stream) {
    CFP_REQUIRE(tr && d_rec_row, "cfp_train_record_step: NULL argument");
    CFP_REQUIRE(t >= 0 && t < tr->T, "step %d outside the horizon %d", t, tr->T);
    hipStream_t st = (hipStream_t)stream;
    const size_t n = tr->n;
    uint8_t* row = tr->r_obs + (size_t)t * n * CFP_REC_BYTES;
    if (d_rec_row != row)
        CFP_HIP_TRY(hipMemcpyAsync(row, d_rec_row, n * CFP_REC_BYTES,
                                   hipMemcpyDeviceToDevice, st));
    if (cfp_policy_forward(tr->p, row, d_terminals, nullptr, state_rows(tr, t), nullptr, nullptr,
                           nullptr, tr->n, 0, stream) != 0)
        return 1;
    hipLaunchKernelGGL(k_take_value, dim3(grid1(n)), dim3(256), 0, st, tr->p->logits,
                       tr->r_value + (size_t)t * n, tr->n);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_rollout_step(cfp_trainer* tr, int t, const uint8_t* d_rec_row,
                     const float* d_prev_terminals, uint64_t seed, float* d_env_actions,
                     void* stream) {
    CFP_REQUIRE(tr && d_rec_row, "cfp_rollout_step: NULL argument");
    CFP_REQUIRE(t >= 0 && t < tr->T, "step %d outside the horizon %d", t, tr->T);
    hipStream_t st = (hipStream_t)stream;
    const size_t n = tr->n, hn = (size_t)H * n, o = (size_t)t * n;
    uint8_t* row = tr->r_obs + o * CFP_REC_BYTES;
    if (d_rec_row != row)
        CFP_HIP_TRY(hipMemcpyAsync(row, d_rec_row, n * CFP_REC_BYTES, hipMemcpyDeviceToDevice,
                                   st));
    const SampleOut so{tr->r_act + o,  tr->r_logprob + o, tr->r_value + o, d_env_actions,
                       seed,           tr->step_ctr,      tr->ticket};
    (void)hn;
    return forward_and_sample(tr->p, row, d_prev_terminals, state_rows(tr, t), tr->n, so, st);
}

int cfp_env_rollout_step(cfp_trainer* tr, cfp_env* e, int t, uint64_t seed, void* stream) {
    CFP_REQUIRE(tr && e, "cfp_env_rollout_step: NULL argument");
    CFP_REQUIRE(cfp_env_num_envs(e) == tr->n, "cfp_env_rollout_step: the env object holds %d envs, the trainer %d",
                cfp_env_num_envs(e), tr->n);
    CFP_REQUIRE(t >= 0 && t < tr->T, "step %d outside the horizon %d", t, tr->T);
    const size_t o = (size_t)t * tr->n;
    uint8_t* row = tr->r_obs + o * CFP_REC_BYTES;
    // cfp_env_record_obs, cfp_rollout_step, cfp_env_step, cfp_record_rd, reset -- with the two
    // one-line kernels of that sequence folded into their neighbours: the record kernel leaves the
    // finished-env counter at zero for the step, the step writes rewards and done flags into the
    // slab rows as well (two launches of ~5 us less per step, 6 % of a step at 4096 envs)
    if (cfp::env_record_obs_zero(e, row, stream)) return 1;
    if (cfp_rollout_step(tr, t, row, cfp_env_terminals(e), seed, cfp_env_actions(e), stream)) return 1;
    if (cfp::env_step_rows(e, tr->r_reward + o, tr->r_done + o, stream)) return 1;
    return cfp_env_pool_size(e) > 0 ? cfp_env_reset_from_pool(e, stream) : cfp_env_reset(e, stream);
}

// cu_prof_mark (craftax_full.cu:12973-12980): with the timers on, the work queued so far is
// waited for and the host clock read; off, nothing happens.  A failed wait reads as -1.
static double prof_mark(cfp_trainer* tr, void* stream) {
    if (!tr->prof) return 0.0;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return -1.0;
    using clk = std::chrono::steady_clock;
    return std::chrono::duration<double, std::milli>(clk::now().time_since_epoch()).count();
}
static void prof_add(cfp_trainer* tr, int phase, double t0, double t1) {
    if (tr->prof && t0 >= 0.0 && t1 >= 0.0) tr->prof_ms[phase] += t1 - t0;
}

// The reference overlaps the regeneration of finished envs (side stream, then a list-form
// record) with the recording of the others (cu_encode_step, craftax_full.cu:11931-11955).
// Measured here at 65 536 envs that costs time: next to the record kernel's 2048 workgroups
// the world generator's workgroups wait for CU slots (48 -> 180 us) and the step grows by
// 80 us, so the steps run in sequence.
int cfp_train_collect(cfp_trainer* tr, cfp_env* e, uint64_t seed, void* stream) {
    CFP_REQUIRE(tr && e, "cfp_train_collect: NULL argument");
    const double t0 = prof_mark(tr, stream);
    for (int t = 0; t < tr->T; t++)
        if (cfp_env_rollout_step(tr, e, t, seed, stream)) return 1;
    const double t1 = prof_mark(tr, stream);
    if (cfp_env_record_obs(e, tr->p->rec, stream)) return 1;
    if (cfp_train_bootstrap(tr, tr->p->rec, cfp_env_terminals(e), stream)) return 1;
    if (cfp_train_gae(tr, stream)) return 1;
    prof_add(tr, 0, t0, t1);
    prof_add(tr, 1, t1, prof_mark(tr, stream));
    return 0;
}

int cfp_train_bootstrap(cfp_trainer* tr, const uint8_t* d_rec_row, const float* d_terminals,
                        void* stream) {
    CFP_REQUIRE(tr && d_rec_row, "cfp_train_bootstrap: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    const size_t n = tr->n, hn = (size_t)H * n;
    CFP_HIP_TRY(hipMemcpyAsync(tr->boot_state, tr->p->h_state, (size_t)tr->L * hn * sizeof(float),
                               hipMemcpyDeviceToDevice, st));
    if (cfp_policy_forward(tr->p, d_rec_row, d_terminals, tr->boot_state, nullptr, nullptr,
                           nullptr, tr->av_tmp, tr->n, 0, stream) != 0)
        return 1;
    hipLaunchKernelGGL(k_take_value, dim3(grid1(n)), dim3(256), 0, st, tr->av_tmp, tr->v_boot,
                       tr->n);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_train_gae(cfp_trainer* tr, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_gae: NULL trainer");
    hipStream_t st = (hipStream_t)stream;
    // one pass: advantages, returns and the advantage moments
    return launch_gae(tr->r_value, tr->r_reward, tr->r_done, tr->v_boot, tr->adv, tr->ret, tr->n,
                      tr->T, tr->cfg.gamma, tr->cfg.lam, tr->stats_part, tr->stats, st);
}

int cfp_train_adv_stats(cfp_trainer* tr, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_adv_stats: NULL trainer");
    hipStream_t st = (hipStream_t)stream;
    return launch_adv_moments(tr->adv, (size_t)tr->n * tr->T, tr->stats_part, tr->stats, st);
}

static int colsum_into(cfp_trainer* tr, const float* src, int ld, float* out, int rows,
                       int cols, hipStream_t st, bool src_bf16 = false) {
    int slices = kColsumSlices;
    if (slices > cols) slices = cols;
    const int per = (cols + slices - 1) / slices;
    slices = (cols + per - 1) / per;
    if (src_bf16)
        hipLaunchKernelGGL((k_colsum_partial<256, true>), dim3(slices, (rows + 255) / 256), dim3(256),
                           0, st, src, ld, tr->colsum_part, rows, cols, per);
    else if (rows <= 64)
        hipLaunchKernelGGL(k_colsum_partial<64>, dim3(slices, 1), dim3(256), 0, st, src, ld,
                           tr->colsum_part, rows, cols, per);
    else
        hipLaunchKernelGGL(k_colsum_partial<256>, dim3(slices, (rows + 255) / 256), dim3(256), 0,
                           st, src, ld, tr->colsum_part, rows, cols, per);
    hipLaunchKernelGGL(k_colsum_fold, dim3((rows + 3) / 4), dim3(256), 0, st,
                       tr->colsum_part, out, rows, slices);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_train_backward(cfp_trainer* tr, int env_start, int env_count, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_backward: NULL trainer");
    CFP_REQUIRE(env_start >= 0 && env_count > 0 && env_start + env_count <= tr->n &&
                    env_count <= tr->mb,
                "minibatch [%d, %d) outside the %d envs / minibatch size %d", env_start,
                env_start + env_count, tr->n, tr->mb);
    hipStream_t st = (hipStream_t)stream;
    cfp_policy* p = tr->p;
    const GemmModeScope mode(tr->gemm_bf16, tr->gemm_split);   // the trainer's own mode, if it has one
    const int T = tr->T, n = tr->n, L = tr->L, mb = env_count;
    const int seg = T / tr->cfg.bptt_split;
    const float* W_enc = p->params + CFP_OFF_W_ENC;
    const float* b_enc = p->params + CFP_OFF_B_ENC;
    const float* W_gru = p->params + CFP_OFF_W_GRU;
    const float* W_a = p->params + CFP_OFF_W_A(L);
    const float* b_a = p->params + CFP_OFF_B_A(L);
    const float* W_v = p->params + CFP_OFF_W_V(L);
    const float* b_v = p->params + CFP_OFF_B_V(L);
    float* g = tr->grads;
    const WindowMap wm_all{0, mb, n, env_start};

    for (int l = 0; l < L; l++)
        hipLaunchKernelGGL(k_fill, dim3(grid1((size_t)H * mb)), dim3(256), 0, st,
                           tr->dcarry[l], (size_t)H * mb, 0.0f);

    hipLaunchKernelGGL(k_head_mirror, dim3((kHeadLd * H + 255) / 256), dim3(256), 0, st, W_a, W_v,
                       tr->w_head);

    for (int t_end = T; t_end > 0; t_end -= tr->win) {
        const int t0 = t_end - tr->win > 0 ? t_end - tr->win : 0;
        const int Tw = t_end - t0;
        const int cols = Tw * mb;
        WindowMap wm = wm_all;
        wm.t0 = t0;
        // ---- forward recompute of the window into tight columns: one launch of the
        // fused forward kernel (fp32, or the bf16-input one) in its window mode: stored
        // state in, pre-activations and layer outputs out.  The unfused chain below is
        // what bf16 inputs run with the split kernels switched off.
        const bool fused = gemm_mode_bf16() == 0 || gemm_mode_split() != 0;
        // bf16 storage: pre / dpre, the layer inputs x[0..L] and the three dh buffers are
        // bf16 arrays inside the same buffers; needs the record-fed dW_enc and the split
        // kernels (whole 32-column blocks); a window that does not fit runs with fp32
        // storage
        const bool st16 = tr->bf16_store && gemm_mode_bf16() != 0 && gemm_mode_split() != 0 &&
                          dw_enc_records_ok(mb) && cols % 32 == 0;
        CFP_REQUIRE(!tr->rs16 || st16,
                    "a bf16 state slab needs the update in its bf16 mode: bf16 GEMM inputs, the split "
                    "kernels, bf16 storage, and a window of whole 32-column blocks");
        if (fused) {
            FwdArgs fa{};
            fill_forward_weights(p, fa);
            fa.bf16 = gemm_mode_bf16();
            fa.rec = tr->r_obs;
            fa.state = tr->r_state;
            fa.h_enc_out = tr->x[0];
            fa.av_out = tr->logitsb;
            fa.n = cols;
            fa.layers = L;
            fa.do_head = 1;
            fa.train = 1;
            fa.tr_bf16 = st16 ? 1 : 0;
            fa.rs_bf16 = tr->rs16;
            fa.tr_t0 = t0; fa.tr_mb = mb; fa.tr_n_all = n; fa.tr_env_start = env_start;
            for (int l = 0; l < L; l++) fa.tr_pre[l] = tr->preb[l];
            for (int l = 0; l <= L; l++) fa.tr_x[l] = tr->x[l];
            // the fp32 rows of dW_enc's 75-feature remainder depend on the records only: made here
            // (40 us alone) instead of behind the last GEMMs of the chain, where the same kernel
            // shares the GPU and takes 190 us on the critical path; xobs is free in this mode
            if (dw_enc_records_ok(mb) &&
                dw_enc_tail_expand(tr->r_obs, tr->xobs, t0, cols, mb, n, env_start, st))
                return 1;
            if (launch_forward(fa, st)) return 1;
            // without the record-fed dW_enc kernel the reverse pass reads the fp32
            // feature matrix
            if (!dw_enc_records_ok(mb) &&
                launch_expand_obs(tr->r_obs, tr->xobs, t0, cols, mb, n, env_start, kObsPad, st))
                return 1;
        } else {
            if (launch_expand_obs(tr->r_obs, tr->xobs, t0, cols, mb, n, env_start, kObsPad, st))
                return 1;
            if (gemm_enc_fwd_ld(cols, W_enc, tr->xobs, kObsPad, tr->x[0], st)) return 1;
            if (cfp_add_bias(tr->x[0], b_enc, cols, stream)) return 1;
            for (int l = 0; l < L; l++) {
                if (cfp_gemm_fwd(G, cols, H, W_gru + (size_t)l * G * H, tr->x[l], tr->preb[l],
                                 stream))
                    return 1;
                if (launch_gru_replay(tr->preb[l], tr->x[l], tr->r_state, tr->x[l + 1], wm, cols, l,
                                      L, st))
                    return 1;
            }
            // 48-row head against the [W_a ; W_v ; 0] mirror: logits and value, no biases
            if (cfp_gemm_fwd(kHeadLd, cols, H, tr->w_head, tr->x[L], tr->logitsb, stream)) return 1;
        }
        // ---- head gradients
        HeadArgs ha{};
        ha.rows = tr->logitsb;
        ha.ld = fused ? A + 1 : kHeadLd;     // the fused forward's rows carry the biases
        ha.bias_a = fused ? nullptr : b_a;
        ha.bias_v = fused ? nullptr : b_v;
        ha.act = tr->r_act; ha.old_logp = tr->r_logprob; ha.adv = tr->adv; ha.ret = tr->ret;
        ha.adv_moments = tr->stats;
        ha.grad_rows = tr->dlogits;
        ha.block_loss = tr->block_loss;
        ha.w = wm; ha.cols = cols; ha.horizon = T;
        ha.clip = tr->cfg.clip; ha.vf = tr->cfg.vf; ha.ent_coef = tr->d_ent;
        if (launch_head(ha, st)) return 1;
        if (launch_fold_f64(tr->block_loss, head_blocks(cols), 3, tr->loss_acc, true, st)) return 1;
        // dh3 = [dlogits | dvalue] . [W_a ; W_v]; dW_a and dW_v from one GEMM; bias sums.
        // Only dh3 is on the way to the layers: with the split kernels the heads' own
        // gradients go to the second stream and run beside the top layer's sweep.
        const int terms = gemm_split_terms();
        const bool overlap = terms >= 1 && gemm_dw_x9_ok(G, cols);
        hipStream_t hs = st;
        // (bf16 storage: the three dh buffers hold bf16 as well)
        if (st16) {
            if (gemm_dh_x9(kHeadLd, cols, tr->w_head, tr->dlogits, tr->dh3b, false, 1,
                           tr->sw.w_mirror, st, false, true))
                return 1;
        } else if (gemm_dh_acc(kHeadLd, cols, tr->w_head, tr->dlogits, tr->dh3b, false, tr->sw, st)) {
            return 1;
        }
        // the second stream starts behind dh3: next to it the heads' dW doubled its time (90 ->
        // 190 us) with the top layer's sweep waiting; under that sweep, which is bound by memory,
        // the same GEMM costs little
        if (overlap) {
            CFP_HIP_TRY(hipEventRecord(tr->ev_head, st));
            CFP_HIP_TRY(hipStreamWaitEvent(tr->st2, tr->ev_head, 0));
            hs = tr->st2;
        }
        if (st16) {
            if (gemm_dw_x9(A + 1, cols, tr->x[L], tr->dlogits, kHeadLd, g + CFP_OFF_W_A(L), 1, tr->sw,
                           hs, A, g + CFP_OFF_W_V(L), false, true))
                return 1;
        } else if (gemm_dw_two(A, 1, cols, tr->x[L], tr->dlogits, kHeadLd, g + CFP_OFF_W_A(L),
                               g + CFP_OFF_W_V(L), tr->sw, hs)) {
            return 1;
        }
        if (colsum_into(tr, tr->dlogits, kHeadLd, g + CFP_OFF_B_A(L), A, cols, hs)) return 1;
        if (colsum_into(tr, tr->dlogits + A, kHeadLd, g + CFP_OFF_B_V(L), 1, cols, hs)) return 1;
        // ---- reverse MinGRU layers
        // With the split kernels the dependent chain  reverse(l) -> dh(l) -> reverse(l-1)
        // hops between two streams: dW(l) is enqueued right behind dh(l) on the stream
        // that ran it, and the next layer's chain on the other stream behind an event.
        // dW(l) so starts first and takes its one workgroup per CU; the HBM-bound
        // reverse kernel of the next layer then fills the wave slots that are left and
        // runs under it.  Every dW has a split workspace of its own.  (The heads' gradients
        // above share the trainer's workspace and column-sum scratch with dW_enc and
        // db_enc below: whichever stream those end up on has by then waited for an event
        // recorded on the second stream behind them.)
        hipStream_t chain = st, other = tr->st2;
        const float* dh_gemm = tr->dh3b;
        const float* dh_extra = nullptr;
        for (int l = L - 1; l >= 0; l--) {
            ReverseArgs ra{};
            ra.gates = tr->preb[l]; ra.layer_in = tr->x[l];
            ra.grad_a = dh_gemm; ra.grad_b = dh_extra; ra.highway_out = tr->dhX;
            ra.slab_state = tr->r_state; ra.slab_done = tr->r_done; ra.carry = tr->dcarry[l];
            ra.w = wm; ra.steps = Tw; ra.layer = l; ra.layers = L; ra.horizon = T; ra.seg = seg;
            ra.gates_bf16 = st16 ? 1 : 0;
            ra.state_bf16 = tr->rs16;
            if (launch_gru_reverse(ra, chain)) return 1;
            if (!overlap &&
                gemm_dw_ld(G, cols, tr->x[l], tr->preb[l], G, g + CFP_OFF_W_GRU + (size_t)l * G * H,
                           tr->sw, chain))
                return 1;
            // layer 0: dh_enc = W_0^T dpre + highway, accumulated onto the highway term
            if (st16) {
                if (gemm_dh_x9(G, cols, W_gru + (size_t)l * G * H, tr->preb[l],
                               l == 0 ? tr->dhX : tr->dhG, l == 0, 1, tr->sw.w_mirror, chain, true,
                               true))
                    return 1;
            } else if (gemm_dh_acc(G, cols, W_gru + (size_t)l * G * H, tr->preb[l],
                                   l == 0 ? tr->dhX : tr->dhG, l == 0, tr->sw, chain)) {
                return 1;
            }
            if (overlap) {
                CFP_HIP_TRY(hipEventRecord(tr->ev_dh[l], chain));
                if (gemm_dw_x9(G, cols, tr->x[l], tr->preb[l], G,
                               g + CFP_OFF_W_GRU + (size_t)l * G * H, terms, tr->sw_layer[l], chain, 0,
                               nullptr, st16, st16))
                    return 1;
                CFP_HIP_TRY(hipStreamWaitEvent(other, tr->ev_dh[l], 0));
                hipStream_t t = chain; chain = other; other = t;
            }
            dh_gemm = tr->dhG;
            dh_extra = tr->dhX;
        }
        // ---- encoder: db_enc; dW_enc += xobs^T dh_enc (dh_enc sits in dhX)
        if (colsum_into(tr, tr->dhX, H, g + CFP_OFF_B_ENC, H, cols, chain, st16)) return 1;
        if (dw_enc_records_ok(mb)) {
            // map bytes straight from the records; xobs is free by now and takes the
            // 76-float rows of the fp32 remainder
            if (fused ? dw_enc_records_tail_ready(tr->r_obs, tr->dhX, g + CFP_OFF_W_ENC, tr->xobs, t0, cols, mb, n,
                                                  env_start, tr->sw, chain, st16,
                                                  overlap ? &tr->sw_layer[0] : nullptr, other)
                      : dw_enc_records(tr->r_obs, tr->dhX, g + CFP_OFF_W_ENC, tr->xobs, t0, cols, mb, n,
                                       env_start, tr->sw, chain, st16, overlap ? &tr->sw_layer[0] : nullptr,
                                       other))
                return 1;
        } else if (gemm_dw_ld(CFP_OBS, cols, tr->dhX, tr->xobs, kObsPad, g + CFP_OFF_W_ENC, tr->sw,
                              chain)) {
            return 1;
        }
        if (overlap) {
            // both streams meet on the caller's: the window's buffers are free again and
            // the gradients complete once it has passed this point
            CFP_HIP_TRY(hipEventRecord(tr->ev_join, tr->st2));
            CFP_HIP_TRY(hipStreamWaitEvent(st, tr->ev_join, 0));
        }
    }
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_train_zero_loss(cfp_trainer* tr, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_zero_loss: NULL trainer");
    hipLaunchKernelGGL(k_fill_f64, dim3(1), dim3(64), 0, (hipStream_t)stream, tr->loss_acc, 3);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_train_adam(cfp_trainer* tr, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_adam: NULL trainer");
    hipStream_t st = (hipStream_t)stream;
    // parameters, moments and every weight mirror of the forward kernels in one pass
    if (launch_adam(tr->p, tr->grads, tr->adam_m, tr->adam_v, tr->adam_ctr, tr->d_lr, 0.9f, 0.999f,
                    1e-8f, st))
        return 1;
    hipLaunchKernelGGL(k_bump_ctr, dim3(1), dim3(1), 0, st, tr->adam_ctr);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

// cu_train_body without its collect (craftax_full.cu:13348-13366): per epoch the loss
// sums start at zero, then every minibatch's backward is followed by its Adam step.
static int train_body(cfp_trainer* tr, void* stream) {
    for (int e = 0; e < tr->cfg.epochs; e++) {
        int rc = cfp_train_zero_loss(tr, stream);
        for (int m = 0; m < tr->cfg.minibatches && rc == 0; m++) {
            const double t0 = prof_mark(tr, stream);
            rc = cfp_train_backward(tr, m * tr->mb, tr->mb, stream);
            const double t1 = prof_mark(tr, stream);
            if (rc == 0) rc = cfp_train_adam(tr, stream);
            prof_add(tr, 2, t0, t1);
            prof_add(tr, 3, t1, prof_mark(tr, stream));
        }
        if (rc != 0) return rc;
    }
    return 0;
}

int cfp_train_update(cfp_trainer* tr, int use_graph, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_update: NULL trainer");
    hipStream_t st = (hipStream_t)stream;
    if (!use_graph || tr->prof) {   // the timers wait between the phases, which a capture cannot
        const int rc = train_body(tr, st);
        if (rc != 0) return rc;
        CFP_HIP_TRY(hipStreamSynchronize(st));
        return 0;
    }
    if (!st) {   // the null stream cannot be captured
        if (!tr->st_own) CFP_HIP_TRY(hipStreamCreate(&tr->st_own));
        st = tr->st_own;
    }
    const int split = tr->gemm_split >= 0 ? tr->gemm_split : cfp_get_gemm_split(),
              bf = tr->gemm_bf16 >= 0 ? tr->gemm_bf16 : cfp_get_gemm_bf16(),
              pbf = cfp_policy_gemm_bf16(tr->p);
    if (tr->texec && (split != tr->graph_split || bf != tr->graph_bf16 ||
                      pbf != tr->graph_pol_bf16 || tr->bf16_store + 2 * tr->rs16 != tr->graph_store16)) {
        (void)hipGraphExecDestroy(tr->texec);
        (void)hipGraphDestroy(tr->tgraph);
        tr->texec = nullptr;
        tr->tgraph = nullptr;
    }
    if (!tr->texec) {
        // No warm-up pass (the reference runs one, :13379-13386, to get cuBLAS's lazy
        // workspaces allocated before the capture): every buffer the iteration touches,
        // GEMM scratch included, was allocated by cfp_train_create.
        CFP_HIP_TRY(hipStreamSynchronize(st));
        CFP_HIP_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        const int rc = train_body(tr, st);
        hipGraph_t g = nullptr;
        const hipError_t ec = hipStreamEndCapture(st, &g);   // always leaves capture mode
        if (rc != 0) {
            if (g) (void)hipGraphDestroy(g);
            return rc;
        }
        CFP_HIP_TRY(ec);
        hipGraphExec_t ex = nullptr;
        const hipError_t ei = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
        if (ei != hipSuccess) {
            (void)hipGraphDestroy(g);
            CFP_HIP_TRY(ei);
        }
        tr->tgraph = g;
        tr->texec = ex;
        tr->graph_split = split;
        tr->graph_bf16 = bf;
        tr->graph_pol_bf16 = pbf;
        tr->graph_store16 = tr->bf16_store + 2 * tr->rs16;
    }
    CFP_HIP_TRY(hipGraphLaunch(tr->texec, st));
    CFP_HIP_TRY(hipStreamSynchronize(st));
    return 0;
}

int cfp_train_loss(cfp_trainer* tr, double* host_loss4, void* stream) {
    CFP_REQUIRE(tr && host_loss4, "cfp_train_loss: NULL argument");
    CFP_REQUIRE(!tr->rs16, "cfp_train_loss replays from an fp32 state slab (cfp_train_set_bf16_rstate is on)");
    hipStream_t st = (hipStream_t)stream;
    const int T = tr->T, n = tr->n, L = tr->L;
    const int seg = T / tr->cfg.bptt_split;
    const size_t hn = (size_t)H * n;
    if (cfp_train_zero_loss(tr, stream)) return 1;
    HeadArgs ha{};
    ha.rows = tr->av_tmp; ha.ld = A + 1;
    ha.act = tr->r_act; ha.old_logp = tr->r_logprob; ha.adv = tr->adv; ha.ret = tr->ret;
    ha.adv_moments = tr->stats;
    ha.block_loss = tr->block_loss;
    ha.cols = n; ha.horizon = T;
    ha.clip = tr->cfg.clip; ha.vf = tr->cfg.vf; ha.ent_coef = tr->d_ent;
    for (int t = 0; t < T; t++) {
        const bool segstart = (t % seg) == 0;
        const float* term = nullptr;
        if (segstart) {
            CFP_HIP_TRY(hipMemcpyAsync(tr->live, tr->r_state + (size_t)t * L * hn,
                                       L * hn * sizeof(float), hipMemcpyDeviceToDevice, st));
        } else {
            hipLaunchKernelGGL(k_done_to_float, dim3(grid1(n)), dim3(256), 0, st,
                               tr->r_done + (size_t)(t - 1) * n, tr->termf, n);
            term = tr->termf;
        }
        if (cfp_policy_forward(tr->p, tr->r_obs + (size_t)t * n * CFP_REC_BYTES, term,
                               tr->live, nullptr, nullptr, nullptr, tr->av_tmp, n, 0, stream))
            return 1;
        ha.w = WindowMap{t, n, n, 0};
        if (launch_head(ha, st)) return 1;
        if (launch_fold_f64(tr->block_loss, head_blocks(n), 3, tr->loss_acc, true, st)) return 1;
    }
    CFP_HIP_TRY(hipGetLastError());
    CFP_HIP_TRY(hipStreamSynchronize(st));
    double h3[3];
    CFP_HIP_TRY(hipMemcpy(h3, tr->loss_acc, sizeof(h3), hipMemcpyDeviceToHost));
    const double count = (double)n * T;
    host_loss4[0] = h3[0]; host_loss4[1] = h3[1]; host_loss4[2] = h3[2];
    host_loss4[3] = (h3[0] + (double)tr->cfg.vf * h3[1] - (double)tr->cfg.ent * h3[2]) / count;
    return 0;
}

}  // extern "C"
