// On-device PPO update: rollout slabs, windowed recompute backward, GAE,
// Adam.  Host-side mirror of the reference's CuTrain layer
// (craftax_full.cu:12637-13480); kernels follow
//   k_mingru_epi_replay_win :9460   k_head_bwd_win      :9603
//   k_mingru_window_bwd     :9510   k_colsum / 256 / small  :10442
//   (k_add_dv_wv :10224 is folded into the top layer's reverse kernel, k_vadd
//    :10069 into the layer-0 dh GEMM, which accumulates onto the highway term)
//   k_gae :10617  k_adv_stats :10638  k_adam :10668  k_loss_accum :10508
// The GEMMs go through the fp32 MFMA seam in gemm.hip.  All reductions are
// done in a fixed order (no float atomics), so a backward pass is bitwise
// reproducible run to run.
#include <vector>

#include "cfp_common.h"
#include "cfp_internal.h"

namespace cfp {
namespace {

constexpr int H = CFP_HIDDEN, G = CFP_GRU, A = CFP_ACTIONS;

__device__ __forceinline__ float sigm(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float gfun(float z) { return z >= 0.0f ? z + 0.5f : sigm(z); }
__device__ __forceinline__ float dgfun(float z) {
    if (z >= 0.0f) return 1.0f;
    const float s = sigm(z);
    return s * (1.0f - s);
}

__global__ void k_fill(float* p, size_t count, float v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = v;
}
__global__ void k_fill_f64(double* p, int count) {
    if ((int)threadIdx.x < count) p[threadIdx.x] = 0.0;
}

// Window recompute epilogue: column w = (t0 + w/mb, env_start + w%mb) reloads
// the stored post-zero state for every step (no live carry).
__global__ void k_mingru_epi_replay_win(const float* __restrict__ pre,
                                        const float* __restrict__ x,
                                        const float* __restrict__ r_state,
                                        float* __restrict__ x_next, int t0,
                                        size_t total, int mb, int n,
                                        int env_start, int layer, int layers) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int k = (int)(idx & (H - 1));
    const size_t w = idx / H;
    const size_t tr = w / (size_t)mb;
    const size_t el = w - tr * (size_t)mb;
    const size_t t = (size_t)t0 + tr;
    const size_t rs = ((t * layers + layer) * (size_t)n + env_start + el) * H + k;
    const float st = r_state[rs];
    const size_t o3 = w * G + k;
    const float zh = pre[o3], zg = pre[o3 + H], zp = pre[o3 + 2 * H];
    const float out = st + sigm(zg) * (gfun(zh) - st);
    const float p = sigm(zp);
    x_next[idx] = p * out + (1.0f - p) * x[idx];
}

// PPO head gradients for one window column per thread; loss terms are reduced
// per block in a fixed order and written to block_loss[3*blockIdx] (double).
// The head's gradient rows are 48 floats wide: [43 dlogits | dvalue | 0 0 0 0], and the
// head weights are mirrored as one [48][256] matrix [W_a ; W_v ; 0].  dh3 = rows . mirror
// then carries the value head's share (the reference's k_add_dv_wv pass,
// craftax_full.cu:10224), K = 48 suits the 16-wide MFMA steps, and one dW GEMM over 44
// rows yields dW_a and dW_v together (cu_gemv_dwv, :11655, needs no pass of its own).
constexpr int kHeadLd = 48;
__global__ void k_head_mirror(const float* __restrict__ W_a, const float* __restrict__ W_v,
                              float* __restrict__ out) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= kHeadLd * H) return;
    const int r = idx / H, k = idx - r * H;
    out[idx] = r < A ? W_a[idx] : (r == A ? W_v[k] : 0.0f);
}

__global__ __launch_bounds__(128) void k_head_bwd_win(
    const float* __restrict__ logits, const float* __restrict__ h3,
    const float* __restrict__ b_a, const float* __restrict__ W_v,
    const float* __restrict__ b_v, const int32_t* __restrict__ r_act,
    const float* __restrict__ r_logprob, const float* __restrict__ adv,
    const float* __restrict__ ret, const double* __restrict__ adv_stats,
    float* __restrict__ dlogits,
    double* __restrict__ block_loss, int t0, int cols, int mb, int n, int n_all,
    int T_all, float clip_eps, float vf_coef, const float* __restrict__ ent_coef_p,
    int logits_ld) {   // b_a == nullptr: rows of the fused forward, 43 logits + value, biases included
    __shared__ double s_l[3][128];
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    double l_pg = 0.0, l_v = 0.0, l_e = 0.0;
    if (c < cols) {
        const int t_rel = c / mb;
        const int el = c - t_rel * mb;
        const size_t o = (size_t)(t0 + t_rel) * n + el;
        const float ent_coef = *ent_coef_p;
        const double inv_count = 1.0 / ((double)n_all * (double)T_all);
        const double m = adv_stats[0] * inv_count;
        const float adv_mean = (float)m;
        const double var = adv_stats[1] * inv_count - m * m;
        const float adv_inv_std = 1.0f / ((float)sqrt(var > 0.0 ? var : 0.0) + 1e-8f);
        const float inv_batch = 1.0f / (float)(T_all * mb);
        const float* lp = logits + (size_t)c * logits_ld;
        float lg[A], pi[A];
        float mx = -1e30f;
#pragma unroll
        for (int a = 0; a < A; a++) { lg[a] = lp[a] + (b_a ? b_a[a] : 0.0f); mx = fmaxf(mx, lg[a]); }
        float total = 0.0f;
#pragma unroll
        for (int a = 0; a < A; a++) { pi[a] = expf(lg[a] - mx); total += pi[a]; }
        const float inv_total = 1.0f / total;
#pragma unroll
        for (int a = 0; a < A; a++) pi[a] *= inv_total;
        const float lse = mx + logf(total);
        const int act = r_act[o];
        float lg_act = 0.0f;
#pragma unroll
        for (int a = 0; a < A; a++) lg_act = (a == act) ? lg[a] : lg_act;
        const float ratio = expf((lg_act - lse) - r_logprob[o]);
        const float Ad = (adv[o] - adv_mean) * adv_inv_std;
        const float u1 = ratio * Ad;
        const float u2 = fminf(fmaxf(ratio, 1.0f - clip_eps), 1.0f + clip_eps) * Ad;
        const float dlogp = (u1 <= u2) ? -Ad * ratio : 0.0f;
        float Hent = 0.0f;
#pragma unroll
        for (int a = 0; a < A; a++) Hent -= pi[a] * (lg[a] - lse);
        float v;
        if (b_a) {
            v = b_v[0];
            const float* hc = h3 + (size_t)c * H;
#pragma unroll 4
            for (int j = 0; j < H; j++) v = fmaf(W_v[j], hc[j], v);
        } else {
            v = lp[A];   // the fused forward leaves the value (bias included) behind the logits
        }
        const float dret = v - ret[o];
        // one 48-float row per column: 43 logit gradients, the value gradient, zeros
        float* dq = dlogits + (size_t)c * kHeadLd;
#pragma unroll
        for (int a = 0; a < A; a++) {
            float d = dlogp * ((a == act ? 1.0f : 0.0f) - pi[a]);
            d += ent_coef * pi[a] * ((lg[a] - lse) + Hent);
            dq[a] = d * inv_batch;
        }
        dq[A] = inv_batch * vf_coef * dret;
#pragma unroll
        for (int a = A + 1; a < kHeadLd; a++) dq[a] = 0.0f;
        l_pg = (double)(-fminf(u1, u2));
        l_v = (double)(0.5f * dret * dret);
        l_e = (double)Hent;
    }
    s_l[0][threadIdx.x] = l_pg; s_l[1][threadIdx.x] = l_v; s_l[2][threadIdx.x] = l_e;
    __syncthreads();
    for (int w = 64; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w)
            for (int q = 0; q < 3; q++) s_l[q][threadIdx.x] += s_l[q][threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x < 3) block_loss[3 * blockIdx.x + threadIdx.x] = s_l[threadIdx.x][0];
}

// loss_acc[q] += sum_b block_loss[3b+q].  Fixed order: thread (q, c) of 3 x 64 sums
// the blocks of chunk c in ascending order, then thread (q, 0) adds the 64 chunk
// sums in ascending order.
__global__ __launch_bounds__(256) void k_loss_fold(const double* __restrict__ block_loss,
                                                   int blocks, double* __restrict__ loss_acc) {
    __shared__ double red[3][64];
    const int q = threadIdx.x >> 6, c = threadIdx.x & 63;
    if (q < 3) {
        const int per = (blocks + 63) / 64;
        const int b1 = min(blocks, (c + 1) * per);
        double s = 0.0;
        for (int b = c * per; b < b1; b++) s += block_loss[3 * b + q];
        red[q][c] = s;
    }
    __syncthreads();
    if (q < 3 && c == 0) {
        double s = 0.0;
        for (int i = 0; i < 64; i++) s += red[q][i];
        loss_acc[q] += s;
    }
}

// out[r] += sum_c src[c*ld + r]: partial sums over `slices` column ranges
// (grid.x), then folded in slice order by k_colsum_fold.  A workgroup covers RB rows
// with CL = 256 / RB threads each; a thread walks every CL-th column of the slice with
// four independent running sums (loads in flight instead of one dependent chain) and
// the CL sums of a row are added in thread order: a fixed order throughout.
template <int RB>
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
        const float* p = src + r;
        int c = c0 + cl;
        for (; c + 3 * CL < c1; c += 4 * CL) {
            s0 += p[(size_t)c * ld];
            s1 += p[(size_t)(c + CL) * ld];
            s2 += p[(size_t)(c + 2 * CL) * ld];
            s3 += p[(size_t)(c + 3 * CL) * ld];
        }
        for (; c < c1; c += CL) s0 += p[(size_t)c * ld];
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

// Reverse MinGRU over one window: thread per (unit, env), t descending, live
// dcarry across windows; dpre overwrites pre in place.
__global__ void k_mingru_window_bwd(
    float* __restrict__ pre, const float* __restrict__ x,
    const float* __restrict__ dhGEMM, const float* __restrict__ dhExtra,
    const float* __restrict__ r_state, const uint8_t* __restrict__ r_done,
    float* __restrict__ dhExtraOut, float* __restrict__ dcarry, int t0, int Tw,
    int mb, int n, int env_start, int layer, int layers, int T_all, int seg_len) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)H * mb) return;
    const int k = (int)(idx & (H - 1));
    const size_t el = idx / H;
    float dc = dcarry[idx];
    for (int tr = Tw - 1; tr >= 0; tr--) {
        const int t = t0 + tr;
        if (t == T_all - 1 || ((t + 1) % seg_len) == 0) dc = 0.0f;
        const size_t w = (size_t)tr * mb + el;
        const size_t o = w * H + k;
        const size_t o3 = w * G + k;
        const float zh = __builtin_nontemporal_load(pre + o3);
        const float zg = __builtin_nontemporal_load(pre + o3 + H);
        const float zp = __builtin_nontemporal_load(pre + o3 + 2 * H);
        float dhout = __builtin_nontemporal_load(dhGEMM + o);
        if (dhExtra) dhout += __builtin_nontemporal_load(dhExtra + o);
        const size_t rs = (((size_t)t * layers + layer) * (size_t)n + env_start + el) * H + k;
        const float s_in = __builtin_nontemporal_load(r_state + rs);
        const float xv = __builtin_nontemporal_load(x + o);
        const bool done_t = r_done[(size_t)t * n + env_start + el] != 0;
        const float sg = sigm(zg);
        const float gh = gfun(zh);
        const float p = sigm(zp);
        const float out_k = s_in + sg * (gh - s_in);
        const float dout = dhout * p + (done_t ? 0.0f : dc);
        const float dzp = dhout * (out_k - xv) * p * (1.0f - p);
        if (dhExtraOut) dhExtraOut[o] = dhout * (1.0f - p);
        dc = dout * (1.0f - sg);
        const float dzg = dout * (gh - s_in) * sg * (1.0f - sg);
        const float dzh = dout * sg * dgfun(zh);
        pre[o3] = dzh;
        pre[o3 + H] = dzg;
        pre[o3 + 2 * H] = dzp;
    }
    dcarry[idx] = dc;
}

__global__ void k_gae(const float* __restrict__ values, const float* __restrict__ rewards,
                      const uint8_t* __restrict__ dones, const float* __restrict__ v_boot,
                      float* __restrict__ adv, float* __restrict__ ret, int n, int T,
                      float gamma, float lam) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    float Aacc = 0.0f;
    for (int t = T - 1; t >= 0; t--) {
        const size_t o = (size_t)t * n + e;
        const float vnext = (t == T - 1) ? v_boot[e] : values[o + n];
        const float nonterm = dones[o] ? 0.0f : 1.0f;
        const float delta = rewards[o] + gamma * vnext * nonterm - values[o];
        Aacc = delta + gamma * lam * nonterm * Aacc;
        adv[o] = Aacc;
        ret[o] = Aacc + values[o];
    }
}

// (sum, sum of squares) in double; 256 blocks of partials, folded in order.
__global__ __launch_bounds__(256) void k_adv_stats_partial(
    const float* __restrict__ adv, size_t count, double* __restrict__ part) {
    __shared__ double s_sum[256], s_sq[256];
    double sum = 0.0, sq = 0.0;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (size_t)gridDim.x * blockDim.x) {
        const double a = adv[i];
        sum += a; sq += a * a;
    }
    s_sum[threadIdx.x] = sum; s_sq[threadIdx.x] = sq;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + w];
            s_sq[threadIdx.x] += s_sq[threadIdx.x + w];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) { part[2 * blockIdx.x] = s_sum[0]; part[2 * blockIdx.x + 1] = s_sq[0]; }
}
__global__ void k_adv_stats_fold(const double* __restrict__ part, int blocks,
                                 double* __restrict__ stats) {
    if (threadIdx.x >= 2) return;
    double s = 0.0;
    for (int b = 0; b < blocks; b++) s += part[2 * b + threadIdx.x];
    stats[threadIdx.x] = s;
}

__global__ void k_adam(float* __restrict__ params, float* __restrict__ grads,
                       float* __restrict__ m, float* __restrict__ v,
                       const uint64_t* __restrict__ step_ctr,
                       const float* __restrict__ lr_ptr, float beta1, float beta2,
                       float eps, int count) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const float lr = *lr_ptr;
    const int step = (int)(*step_ctr) + 1;
    const float g = grads[i];
    grads[i] = 0.0f;
    const float mi = beta1 * m[i] + (1.0f - beta1) * g;
    const float vi = beta2 * v[i] + (1.0f - beta2) * g * g;
    m[i] = mi; v[i] = vi;
    const float mhat = mi / (1.0f - powf(beta1, (float)step));
    const float vhat = vi / (1.0f - powf(beta2, (float)step));
    params[i] -= lr * mhat / (sqrtf(vhat) + eps);
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

// Loss terms of one step from biased logits/value rows [n][44] (k_loss_accum).
__global__ __launch_bounds__(128) void k_loss_accum(
    const float* __restrict__ av, const int32_t* __restrict__ r_act,
    const float* __restrict__ r_logprob, const float* __restrict__ adv,
    const float* __restrict__ ret, const double* __restrict__ adv_stats,
    double* __restrict__ block_loss, int t, int n, int T_all, float clip_eps) {
    __shared__ double s_l[3][128];
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    double l_pg = 0.0, l_v = 0.0, l_e = 0.0;
    if (e < n) {
        const size_t o = (size_t)t * n + e;
        const double inv_count = 1.0 / ((double)n * (double)T_all);
        const double m = adv_stats[0] * inv_count;
        const double var = adv_stats[1] * inv_count - m * m;
        const float amean = (float)m;
        const float ainv = 1.0f / ((float)sqrt(var > 0.0 ? var : 0.0) + 1e-8f);
        const float* lg = av + (size_t)e * CFP_AV;
        float mx = -1e30f;
        for (int a = 0; a < A; a++) mx = fmaxf(mx, lg[a]);
        float total = 0.0f;
        for (int a = 0; a < A; a++) total += expf(lg[a] - mx);
        const float lse = mx + logf(total);
        float Hent = 0.0f;
        for (int a = 0; a < A; a++) Hent -= (expf(lg[a] - mx) / total) * (lg[a] - lse);
        const float Ad = (adv[o] - amean) * ainv;
        const float ratio = expf((lg[r_act[o]] - lse) - r_logprob[o]);
        const float u1 = ratio * Ad;
        const float u2 = fminf(fmaxf(ratio, 1.0f - clip_eps), 1.0f + clip_eps) * Ad;
        const float dret = lg[A] - ret[o];
        l_pg = (double)(-fminf(u1, u2));
        l_v = (double)(0.5f * dret * dret);
        l_e = (double)Hent;
    }
    s_l[0][threadIdx.x] = l_pg; s_l[1][threadIdx.x] = l_v; s_l[2][threadIdx.x] = l_e;
    __syncthreads();
    for (int w = 64; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w)
            for (int q = 0; q < 3; q++) s_l[q][threadIdx.x] += s_l[q][threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x < 3) block_loss[3 * blockIdx.x + threadIdx.x] = s_l[threadIdx.x][0];
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
    // it and the caller's, see cfp_train_backward) and the dW GEMMs' own split workspaces
    hipStream_t st2 = nullptr;
    hipEvent_t ev_dh[CFP_MAX_LAYERS] = {};
    hipEvent_t ev_join = nullptr;
    float* dw_work2 = nullptr;
    size_t dw_work2_floats = 0;
    // cfp_train_update's captured iteration (epochs x minibatches x (backward, Adam)) and
    // the process-wide GEMM modes it was captured under
    hipGraph_t tgraph = nullptr;
    hipGraphExec_t texec = nullptr;
    int graph_split = -1, graph_bf16 = -1, graph_pol_bf16 = -1;
    hipStream_t st_own = nullptr;   // capture stream when the caller passes the null stream
};

static constexpr int kColsumSlices = 1024;

extern "C" {

void cfp_train_destroy(cfp_trainer* tr) {
    if (!tr) return;
    for (void* q : tr->owned) (void)hipFree(q);
    for (hipEvent_t e : tr->ev_dh)
        if (e) (void)hipEventDestroy(e);
    if (tr->ev_join) (void)hipEventDestroy(tr->ev_join);
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
    TA(block_loss, 3 * sizeof(double) * ((cc > (size_t)tr->n ? cc : tr->n) / 128 + 1));
    TA(stats_part, 2 * 256 * sizeof(double));
    TA(grads, pc * sizeof(float));
    TA(adam_m, pc * sizeof(float));
    TA(adam_v, pc * sizeof(float));
    TA(adam_ctr, sizeof(uint64_t));
    TA(step_ctr, sizeof(uint64_t));
    TA(boot_state, (size_t)tr->L * hn * sizeof(float));
    TA(d_lr, sizeof(float));
    TA(d_ent, sizeof(float));
    TA(xobs, cc * kObsPad * sizeof(float));   // rows widened 843 -> 848: 16-byte aligned
    for (int l = 0; l <= tr->L; l++) TA(x[l], cc * H * sizeof(float));
    for (int l = 0; l < tr->L; l++) TA(preb[l], cc * G * sizeof(float));
    for (int l = 0; l < tr->L; l++) TA(dcarry[l], (size_t)mb * H * sizeof(float));
    TA(logitsb, cc * (A + 1) * sizeof(float));   // [cols][44] from the fused recompute, [cols][43] unfused
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
    // default priority, as every stream of this library
    if (ok) ok = hipStreamCreateWithFlags(&tr->st2, hipStreamNonBlocking) == hipSuccess &&
                 hipEventCreateWithFlags(&tr->ev_join, hipEventDisableTiming) == hipSuccess;
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

int cfp_train_window(const cfp_trainer* tr) { return tr ? tr->win : 0; }
int cfp_train_minibatch(const cfp_trainer* tr) { return tr ? tr->mb : 0; }

int cfp_train_record_step(cfp_trainer* tr, int t, const uint8_t* d_rec_row,
                          const float* d_terminals, void* stream) {
    CFP_REQUIRE(tr && d_rec_row, "cfp_train_record_step: NULL argument");
    CFP_REQUIRE(t >= 0 && t < tr->T, "step %d outside the horizon %d", t, tr->T);
    hipStream_t st = (hipStream_t)stream;
    const size_t n = tr->n, hn = (size_t)H * n;
    uint8_t* row = tr->r_obs + (size_t)t * n * CFP_REC_BYTES;
    if (d_rec_row != row)
        CFP_HIP_TRY(hipMemcpyAsync(row, d_rec_row, n * CFP_REC_BYTES,
                                   hipMemcpyDeviceToDevice, st));
    if (cfp_policy_forward(tr->p, row, d_terminals, nullptr,
                           tr->r_state + (size_t)t * tr->L * hn, nullptr, nullptr,
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
    if (cfp_policy_forward(tr->p, row, d_prev_terminals, nullptr, tr->r_state + o * tr->L * H,
                           nullptr, nullptr, nullptr, tr->n, 0, stream) != 0)
        return 1;
    if (cfp_value_sample(tr->p->logits, tr->n, A, d_env_actions, tr->r_act + o, tr->r_logprob + o,
                         tr->r_value + o, seed, tr->step_ctr, stream) != 0)
        return 1;
    hipLaunchKernelGGL(k_bump_ctr, dim3(1), dim3(1), 0, st, tr->step_ctr);
    CFP_HIP_TRY(hipGetLastError());
    (void)hn;
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
    hipLaunchKernelGGL(k_gae, dim3(grid1(tr->n)), dim3(256), 0, st, tr->r_value,
                       tr->r_reward, tr->r_done, tr->v_boot, tr->adv, tr->ret, tr->n,
                       tr->T, tr->cfg.gamma, tr->cfg.lam);
    return cfp_train_adv_stats(tr, stream);
}

int cfp_train_adv_stats(cfp_trainer* tr, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_adv_stats: NULL trainer");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_adv_stats_partial, dim3(256), dim3(256), 0, st, tr->adv,
                       (size_t)tr->n * tr->T, tr->stats_part);
    hipLaunchKernelGGL(k_adv_stats_fold, dim3(1), dim3(64), 0, st, tr->stats_part, 256,
                       tr->stats);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

static int colsum_into(cfp_trainer* tr, const float* src, int ld, float* out, int rows,
                       int cols, hipStream_t st) {
    int slices = kColsumSlices;
    if (slices > cols) slices = cols;
    const int per = (cols + slices - 1) / slices;
    slices = (cols + per - 1) / per;
    if (rows <= 64)
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

    for (int l = 0; l < L; l++)
        hipLaunchKernelGGL(k_fill, dim3(grid1((size_t)H * mb)), dim3(256), 0, st,
                           tr->dcarry[l], (size_t)H * mb, 0.0f);

    hipLaunchKernelGGL(k_head_mirror, dim3((kHeadLd * H + 255) / 256), dim3(256), 0, st, W_a, W_v,
                       tr->w_head);

    for (int t_end = T; t_end > 0; t_end -= tr->win) {
        const int t0 = t_end - tr->win > 0 ? t_end - tr->win : 0;
        const int Tw = t_end - t0;
        const int cols = Tw * mb;
        const size_t hc = (size_t)H * cols;
        // ---- forward recompute of the window into tight columns: one launch of the
        // fused forward kernel (fp32, or the bf16-input one) in its window mode: stored
        // state in, pre-activations and layer outputs out.  The unfused chain below is
        // what bf16 inputs run with the split kernels switched off.
        const bool fused = cfp_get_gemm_bf16() == 0 || cfp_get_gemm_split() != 0;
        if (fused) {
            FwdArgs fa{};
            fill_forward_weights(p, fa);
            fa.bf16 = cfp_get_gemm_bf16();
            fa.rec = tr->r_obs;
            fa.state = tr->r_state;
            fa.h_enc_out = tr->x[0];
            fa.av_out = tr->logitsb;
            fa.n = cols;
            fa.layers = L;
            fa.do_head = 1;
            fa.train = 1;
            fa.tr_t0 = t0; fa.tr_mb = mb; fa.tr_n_all = n; fa.tr_env_start = env_start;
            for (int l = 0; l < L; l++) fa.tr_pre[l] = tr->preb[l];
            for (int l = 0; l <= L; l++) fa.tr_x[l] = tr->x[l];
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
                hipLaunchKernelGGL(k_mingru_epi_replay_win, dim3(grid1(hc)), dim3(256), 0, st,
                                   tr->preb[l], tr->x[l], tr->r_state, tr->x[l + 1], t0, hc,
                                   mb, n, env_start, l, L);
            }
            if (cfp_gemm_fwd(A, cols, H, W_a, tr->x[L], tr->logitsb, stream)) return 1;
        }
        // ---- head gradients
        const int hb = (cols + 127) / 128;
        hipLaunchKernelGGL(k_head_bwd_win, dim3(hb), dim3(128), 0, st, tr->logitsb, tr->x[L],
                           fused ? nullptr : b_a, W_v, b_v, tr->r_act + env_start, tr->r_logprob + env_start,
                           tr->adv + env_start, tr->ret + env_start, tr->stats, tr->dlogits,
                           tr->block_loss, t0, cols, mb, n, n, T, tr->cfg.clip,
                           tr->cfg.vf, tr->d_ent, fused ? A + 1 : A);
        hipLaunchKernelGGL(k_loss_fold, dim3(1), dim3(256), 0, st, tr->block_loss, hb,
                           tr->loss_acc);
        // dh3 = [dlogits | dvalue] . [W_a ; W_v]; dW_a and dW_v from one GEMM; bias sums
        if (gemm_dh_acc(kHeadLd, cols, tr->w_head, tr->dlogits, tr->dh3b, false, st)) return 1;
        if (gemm_dw_two(A, 1, cols, tr->x[L], tr->dlogits, kHeadLd, g + CFP_OFF_W_A(L),
                        g + CFP_OFF_W_V(L), st))
            return 1;
        if (colsum_into(tr, tr->dlogits, kHeadLd, g + CFP_OFF_B_A(L), A, cols, st)) return 1;
        if (colsum_into(tr, tr->dlogits + A, kHeadLd, g + CFP_OFF_B_V(L), 1, cols, st)) return 1;
        // ---- reverse MinGRU layers
        // With the split kernels the dependent chain  reverse(l) -> dh(l) -> reverse(l-1)
        // hops between two streams: dW(l) is enqueued right behind dh(l) on the stream
        // that ran it, and the next layer's chain on the other stream behind an event.
        // dW(l) so starts first and takes its one workgroup per CU; the HBM-bound
        // reverse kernel of the next layer then fills the wave slots that are left and
        // runs under it.  Every dW has a split workspace of its own.
        const int terms = gemm_split_terms();
        const bool overlap = terms > 1 && gemm_dw_x9_ok(G, cols);
        hipStream_t chain = st, other = tr->st2;
        const float* dh_gemm = tr->dh3b;
        const float* dh_extra = nullptr;
        for (int l = L - 1; l >= 0; l--) {
            hipLaunchKernelGGL(k_mingru_window_bwd, dim3(grid1((size_t)H * mb)), dim3(256),
                               0, chain, tr->preb[l], tr->x[l], dh_gemm, dh_extra, tr->r_state,
                               tr->r_done, tr->dhX, tr->dcarry[l], t0, Tw, mb, n, env_start,
                               l, L, T, seg);
            if (!overlap &&
                gemm_dw_ld(G, cols, tr->x[l], tr->preb[l], G, g + CFP_OFF_W_GRU + (size_t)l * G * H,
                           chain))
                return 1;
            // layer 0: dh_enc = W_0^T dpre + highway, accumulated onto the highway term
            if (gemm_dh_acc(G, cols, W_gru + (size_t)l * G * H, tr->preb[l],
                            l == 0 ? tr->dhX : tr->dhG, l == 0, chain))
                return 1;
            if (overlap) {
                CFP_HIP_TRY(hipEventRecord(tr->ev_dh[l], chain));
                if (gemm_dw_x9(G, cols, tr->x[l], tr->preb[l], G,
                               g + CFP_OFF_W_GRU + (size_t)l * G * H, terms, chain, 0, nullptr,
                               tr->dw_work2 + (size_t)l * tr->dw_work2_floats, tr->dw_work2_floats))
                    return 1;
                CFP_HIP_TRY(hipStreamWaitEvent(other, tr->ev_dh[l], 0));
                hipStream_t t = chain; chain = other; other = t;
            }
            dh_gemm = tr->dhG;
            dh_extra = tr->dhX;
        }
        // ---- encoder: db_enc; dW_enc += xobs^T dh_enc (dh_enc sits in dhX)
        if (colsum_into(tr, tr->dhX, H, g + CFP_OFF_B_ENC, H, cols, chain)) return 1;
        if (dw_enc_records_ok(mb)) {
            // map bytes straight from the records; xobs is free by now and takes the
            // 76-float rows of the fp32 remainder
            if (dw_enc_records(tr->r_obs, tr->dhX, g + CFP_OFF_W_ENC, tr->xobs, t0, cols, mb, n,
                               env_start, chain))
                return 1;
        } else if (gemm_dw_ld(CFP_OBS, cols, tr->dhX, tr->xobs, kObsPad, g + CFP_OFF_W_ENC, chain)) {
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
    const int pc = (int)tr->p->param_count;
    hipLaunchKernelGGL(k_adam, dim3(grid1(pc)), dim3(256), 0, st, tr->p->params, tr->grads,
                       tr->adam_m, tr->adam_v, tr->adam_ctr, tr->d_lr, 0.9f, 0.999f, 1e-8f,
                       pc);
    hipLaunchKernelGGL(k_bump_ctr, dim3(1), dim3(1), 0, st, tr->adam_ctr);
    CFP_HIP_TRY(hipGetLastError());
    return cfp_policy_refresh_weights(tr->p, stream);
}

// cu_train_body without its collect (craftax_full.cu:13348-13366): per epoch the loss
// sums start at zero, then every minibatch's backward is followed by its Adam step.
static int train_body(cfp_trainer* tr, void* stream) {
    for (int e = 0; e < tr->cfg.epochs; e++) {
        int rc = cfp_train_zero_loss(tr, stream);
        for (int m = 0; m < tr->cfg.minibatches && rc == 0; m++) {
            rc = cfp_train_backward(tr, m * tr->mb, tr->mb, stream);
            if (rc == 0) rc = cfp_train_adam(tr, stream);
        }
        if (rc != 0) return rc;
    }
    return 0;
}

int cfp_train_update(cfp_trainer* tr, int use_graph, void* stream) {
    CFP_REQUIRE(tr, "cfp_train_update: NULL trainer");
    hipStream_t st = (hipStream_t)stream;
    if (!use_graph) {
        const int rc = train_body(tr, st);
        if (rc != 0) return rc;
        CFP_HIP_TRY(hipStreamSynchronize(st));
        return 0;
    }
    if (!st) {   // the null stream cannot be captured
        if (!tr->st_own) CFP_HIP_TRY(hipStreamCreate(&tr->st_own));
        st = tr->st_own;
    }
    const int split = cfp_get_gemm_split(), bf = cfp_get_gemm_bf16(),
              pbf = cfp_policy_gemm_bf16(tr->p);
    if (tr->texec && (split != tr->graph_split || bf != tr->graph_bf16 ||
                      pbf != tr->graph_pol_bf16)) {
        (void)hipGraphExecDestroy(tr->texec);
        (void)hipGraphDestroy(tr->tgraph);
        tr->texec = nullptr;
        tr->tgraph = nullptr;
    }
    if (!tr->texec) {
        // Warm-up as in the reference (:13379-13386): one bare backward, no Adam, so that
        // the lazily allocated GEMM workspaces exist before the capture (an allocation
        // inside a capture is illegal); parameters stay untouched, the gradients it
        // left are cleared again.
        int rc = cfp_train_backward(tr, 0, tr->mb, st);
        if (rc != 0) return rc;
        hipLaunchKernelGGL(k_fill, dim3(grid1(tr->p->param_count)), dim3(256), 0, st, tr->grads,
                           tr->p->param_count, 0.0f);
        CFP_HIP_TRY(hipGetLastError());
        CFP_HIP_TRY(hipStreamSynchronize(st));
        CFP_HIP_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        rc = train_body(tr, st);
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
    }
    CFP_HIP_TRY(hipGraphLaunch(tr->texec, st));
    CFP_HIP_TRY(hipStreamSynchronize(st));
    return 0;
}

int cfp_train_loss(cfp_trainer* tr, double* host_loss4, void* stream) {
    CFP_REQUIRE(tr && host_loss4, "cfp_train_loss: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    const int T = tr->T, n = tr->n, L = tr->L;
    const int seg = T / tr->cfg.bptt_split;
    const size_t hn = (size_t)H * n;
    if (cfp_train_zero_loss(tr, stream)) return 1;
    const int hb = (n + 127) / 128;
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
        hipLaunchKernelGGL(k_loss_accum, dim3(hb), dim3(128), 0, st, tr->av_tmp, tr->r_act,
                           tr->r_logprob, tr->adv, tr->ret, tr->stats, tr->block_loss, t, n,
                           T, tr->cfg.clip);
        hipLaunchKernelGGL(k_loss_fold, dim3(1), dim3(256), 0, st, tr->block_loss, hb,
                           tr->loss_acc);
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
