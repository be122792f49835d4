/*
 * CPU restatement (fp64) of the PPO update's loss and gradients.
 * TEST INFRASTRUCTURE ONLY (see cfo.h).
 *
 * Follows craftax_full.cu:
 *   cu_train_backward (window recompute + reverse)   :13168-13335
 *   k_mingru_epi_replay_win (stored state every step) :9460-9503
 *   k_head_bwd_win                                     :9603-9706
 *   k_mingru_window_bwd                                :9510-9597
 *   k_add_dv_wv / colsums / dW, dh GEMM roles          :10224, :13256-13326
 *   cu_train_loss + k_loss_accum (live recurrence)     :13414-13480, :10508
 *   k_gae / k_adv_stats / k_adam                       :10617-10686
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "cfo.h"
#include "cfo_train.h"

enum { H = CFP_HIDDEN, G = CFP_GRU, F = CFP_OBS, A = CFP_ACTIONS };

/* bf16-operand mode: every operand of a matrix product (encoder, gate and actor GEMMs of
 * the forward; dW, dh and dW_enc GEMMs of the backward) is rounded to bf16 -- an
 * activation or gradient from its fp32 value, a weight from its fp32 value -- while
 * products and sums stay fp64.  This is the arithmetic of the library's bf16-input /
 * fp32-accumulate update with the accumulation made exact: what remains between it and
 * the device result is fp32 accumulation order and the fp32 elementwise work.  The value
 * row rides with the 43 actor rows in one 44-row head GEMM in the forward and in both
 * backward GEMMs of the head, so W_v, dv and h3 are rounded there as well. */
static int g_q = 0, g_map_exact = 0;
#pragma omp threadprivate(g_q, g_map_exact)
static double qb(double v) {
    float f = (float)v;
    uint32_t u;
    memcpy(&u, &f, 4);
    u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    memcpy(&f, &u, 4);
    return (double)f;
}
static double qa(double v) { return g_q ? qb(v) : v; }   /* activation / gradient operand */
/* g_q == 2: the window workspace of the backward is stored as bf16 as well
 * (cfp_train_set_bf16_storage): gate pre-activations and layer inputs as the sweep reads
 * them, gate gradients and the highway term as it writes them, and the outputs of the
 * dh GEMMs (the layer-0 one adds the stored highway term and rounds the sum). */
static double qs(double v) { return g_q == 2 ? qb(v) : v; }

static double sig(double x) { return 1.0 / (1.0 + exp(-x)); }
static double gfun(double x) { return x >= 0.0 ? x + 0.5 : sig(x); }
static double dgfun(double x) {
    if (x >= 0.0) return 1.0;
    double s = sig(x);
    return s * (1.0 - s);
}

typedef struct {
    const float *W_enc, *b_enc, *W_gru, *W_a, *b_a, *W_v, *b_v;
} Weights;

static Weights split(const float* p, int L) {
    Weights w = {p + CFP_OFF_W_ENC, p + CFP_OFF_B_ENC, p + CFP_OFF_W_GRU,
                 p + CFP_OFF_W_A(L), p + CFP_OFF_B_A(L), p + CFP_OFF_W_V(L),
                 p + CFP_OFF_B_V(L)};
    return w;
}

/* per-(t) saved forward quantities for one env */
typedef struct {
    double x[CFP_MAX_LAYERS + 1][H]; /* layer inputs; x[L] = h3 */
    double zh[CFP_MAX_LAYERS][H], zg[CFP_MAX_LAYERS][H], zp[CFP_MAX_LAYERS][H];
    double s_in[CFP_MAX_LAYERS][H];
    double out[CFP_MAX_LAYERS][H];
    float feat[F];
} Step;

static void adv_norm(const cfo_ppo_batch* b, double* mean, double* inv_std) {
    /* k_head_bwd_win :9628-9632: mean and inv_std are rounded to fp32 there;
     * the fp64 oracle keeps the same formula in double. */
    const double inv_count = 1.0 / ((double)b->n * (double)b->T);
    const double m = b->adv_sum * inv_count;
    double var = b->adv_sumsq * inv_count - m * m;
    if (var < 0.0) var = 0.0;
    *mean = m;
    *inv_std = 1.0 / (sqrt(var) + 1e-8);
}

/* forward of one step for one env; state input given in s_in (already
 * post-zero), fills Step. */
static void step_forward(const Weights* w, int L, const uint8_t* rec, Step* s) {
    cfo_expand_record(rec, s->feat);
    for (int k = 0; k < H; k++) s->x[0][k] = (double)w->b_enc[k];
    for (int f = 0; f < F; f++) {
        const double xf = qa((double)s->feat[f]);
        if (xf == 0.0) continue;
        const float* wr = w->W_enc + (size_t)f * H;   /* W_enc / W_gru / W_a: pre-rounded in bf16 mode */
        for (int k = 0; k < H; k++) s->x[0][k] += xf * (double)wr[k];
    }
    for (int l = 0; l < L; l++) {
        const float* Wl = w->W_gru + (size_t)l * G * H;
        double xq[H];
        for (int j = 0; j < H; j++) xq[j] = qa(s->x[l][j]);
        for (int k = 0; k < H; k++) {
            double zh = 0, zg = 0, zp = 0;
            const float* a = Wl + (size_t)k * H;
            const float* bq = Wl + (size_t)(H + k) * H;
            const float* c = Wl + (size_t)(2 * H + k) * H;
            for (int j = 0; j < H; j++) {
                zh += (double)a[j] * xq[j];
                zg += (double)bq[j] * xq[j];
                zp += (double)c[j] * xq[j];
            }
            s->zh[l][k] = zh; s->zg[l][k] = zg; s->zp[l][k] = zp;
            const double st = s->s_in[l][k];
            const double out = st + sig(zg) * (gfun(zh) - st);
            const double p = sig(zp);
            s->out[l][k] = out;
            s->x[l + 1][k] = p * out + (1.0 - p) * s->x[l][k];
        }
    }
}

/* head terms for one sample; returns the three raw loss terms and (optionally)
 * dlogits[43], dv.  k_head_bwd_win :9635-9689. */
static void head_terms(const Weights* w, const cfo_ppo_batch* b, const double* h3,
                       size_t o, double amean, double ainv, double inv_batch,
                       double* l_pg, double* l_v, double* l_ent, double* dlogits,
                       double* dv) {
    double lg[A], pi[A];
    double mx = -1e300;
    double h3q[H];
    for (int j = 0; j < H; j++) h3q[j] = qa(h3[j]);
    for (int a = 0; a < A; a++) {
        double z = (double)w->b_a[a];
        for (int j = 0; j < H; j++) z += (double)w->W_a[a * H + j] * h3q[j];
        lg[a] = z;
        if (z > mx) mx = z;
    }
    double total = 0.0;
    for (int a = 0; a < A; a++) { pi[a] = exp(lg[a] - mx); total += pi[a]; }
    for (int a = 0; a < A; a++) pi[a] /= total;
    const double lse = mx + log(total);
    const int act = b->r_act[o];
    const double ratio = exp((lg[act] - lse) - (double)b->r_logprob[o]);
    const double Ad = ((double)b->adv[o] - amean) * ainv;
    const double u1 = ratio * Ad;
    double rc = ratio;
    if (rc < 1.0 - (double)b->clip) rc = 1.0 - (double)b->clip;
    if (rc > 1.0 + (double)b->clip) rc = 1.0 + (double)b->clip;
    const double u2 = rc * Ad;
    const double dlogp = (u1 <= u2) ? -Ad * ratio : 0.0;
    double Hent = 0.0;
    for (int a = 0; a < A; a++) Hent -= pi[a] * (lg[a] - lse);
    double v = (double)w->b_v[0];
    for (int j = 0; j < H; j++) v += (double)w->W_v[j] * h3q[j];
    const double dret = v - (double)b->ret[o];
    *l_pg = -(u1 < u2 ? u1 : u2);
    *l_v = 0.5 * dret * dret;
    *l_ent = Hent;
    if (dlogits) {
        *dv = inv_batch * (double)b->vf * dret;
        for (int a = 0; a < A; a++) {
            double d = dlogp * ((a == act ? 1.0 : 0.0) - pi[a]);
            d += (double)b->ent * pi[a] * ((lg[a] - lse) + Hent);
            dlogits[a] = d * inv_batch;
        }
    }
}

static size_t rstate_off(const cfo_ppo_batch* b, int t, int l, int env) {
    return (((size_t)t * b->layers + l) * (size_t)b->n + (size_t)env) * H;
}

/* Loss of the minibatch [env_start, env_start+mb) with LIVE recurrence inside
 * BPTT segments and the stored state only at segment starts (cu_train_loss),
 * normalised by T*mb; loss3 receives the raw sums (pg, v, ent). */
double cfo_ppo_loss_f64(const float* params, const cfo_ppo_batch* b, double* loss3) {
    const int L = b->layers, T = b->T;
    const Weights w = split(params, L);
    double amean, ainv;
    adv_norm(b, &amean, &ainv);
    double s_pg = 0, s_v = 0, s_e = 0;
#pragma omp parallel for schedule(static) reduction(+ : s_pg, s_v, s_e)
    for (int el = 0; el < b->mb; el++) {
        const int env = b->env_start + el;
        Step* s = (Step*)malloc(sizeof(Step));
        double live[CFP_MAX_LAYERS][H];
        for (int t = 0; t < T; t++) {
            const int segstart = (t % b->seg_len) == 0;
            for (int l = 0; l < L; l++)
                for (int k = 0; k < H; k++) {
                    if (segstart) {
                        s->s_in[l][k] = (double)b->r_state[rstate_off(b, t, l, env) + k];
                    } else {
                        const int dprev = b->r_done[(size_t)(t - 1) * b->n + env] != 0;
                        s->s_in[l][k] = dprev ? 0.0 : live[l][k];
                    }
                }
            step_forward(&w, L, b->r_obs + ((size_t)t * b->n + env) * CFP_REC_BYTES, s);
            for (int l = 0; l < L; l++) memcpy(live[l], s->out[l], sizeof(live[l]));
            double lp, lv, le;
            head_terms(&w, b, s->x[L], (size_t)t * b->n + env, amean, ainv, 0.0, &lp,
                       &lv, &le, NULL, NULL);
            s_pg += lp; s_v += lv; s_e += le;
        }
        free(s);
    }
    if (loss3) { loss3[0] = s_pg; loss3[1] = s_v; loss3[2] = s_e; }
    return (s_pg + (double)b->vf * s_v - (double)b->ent * s_e) / ((double)T * b->mb);
}

/* Gradients of the minibatch as cu_train_backward forms them: forward
 * recompute from the STORED state at every step, reverse sweep with a live
 * dcarry that is cut at t == T-1 and at BPTT segment ends and blocked by
 * done_t.  grads (param layout, fp64) is overwritten. */
static void ppo_backward(const float* params, const cfo_ppo_batch* b, double* grads,
                         double* loss3, int bf16_ops);

void cfo_ppo_backward_f64(const float* params, const cfo_ppo_batch* b, double* grads,
                          double* loss3) {
    ppo_backward(params, b, grads, loss3, 0);
}

/* A copy of the parameters with the four weight matrices rounded to bf16 (biases as they are). */
static float* bf16_weights(const float* params, int L) {
    const size_t pc = (size_t)CFP_PARAM_COUNT(L);
    float* pq = (float*)malloc(pc * sizeof(float));
    memcpy(pq, params, pc * sizeof(float));
    for (size_t i = CFP_OFF_W_ENC; i < (size_t)CFP_OFF_B_ENC; i++) pq[i] = (float)qb(pq[i]);
    for (size_t i = CFP_OFF_W_GRU; i < (size_t)CFP_OFF_B_A(L); i++) pq[i] = (float)qb(pq[i]);   /* W_gru, W_a */
    for (size_t i = CFP_OFF_W_V(L); i < (size_t)CFP_OFF_W_V(L) + CFP_HIDDEN; i++) pq[i] = (float)qb(pq[i]);
    return pq;
}

/* The same update with every matrix-product operand rounded to bf16 (see qb above). */
void cfo_ppo_backward_bf16ops_f64(const float* params, const cfo_ppo_batch* b, double* grads,
                                  double* loss3, int flags) {
    float* pq = bf16_weights(params, b->layers);
    ppo_backward(pq, b, grads, loss3, (flags & 1 ? 2 : 1) | (flags & 2 ? 4 : 0));
    free(pq);
}

static void ppo_backward(const float* params, const cfo_ppo_batch* b, double* grads,
                         double* loss3, int bf16_ops) {
    const int L = b->layers, T = b->T;
    const Weights w = split(params, L);
    const size_t pc = (size_t)CFP_PARAM_COUNT(L);
    double amean, ainv;
    adv_norm(b, &amean, &ainv);
    const double inv_batch = 1.0 / ((double)T * (double)b->mb);
    memset(grads, 0, pc * sizeof(double));
    double s_pg = 0, s_v = 0, s_e = 0;
    int nth = 1;
#ifdef _OPENMP
    nth = omp_get_max_threads();
    if (nth > b->mb) nth = b->mb;
#endif
    double* gbuf = (double*)calloc(pc * (size_t)nth, sizeof(double));
#pragma omp parallel num_threads(nth) reduction(+ : s_pg, s_v, s_e)
    {
        int tid = 0;
#ifdef _OPENMP
        tid = omp_get_thread_num();
#endif
        g_q = bf16_ops & 3;
        g_map_exact = (bf16_ops & 4) != 0;
        double* g = gbuf + pc * (size_t)tid;
        double* gW_enc = g + CFP_OFF_W_ENC;
        double* gb_enc = g + CFP_OFF_B_ENC;
        double* gW_gru = g + CFP_OFF_W_GRU;
        double* gW_a = g + CFP_OFF_W_A(L);
        double* gb_a = g + CFP_OFF_B_A(L);
        double* gW_v = g + CFP_OFF_W_V(L);
        double* gb_v = g + CFP_OFF_B_V(L);
        Step* steps = (Step*)malloc(sizeof(Step) * (size_t)T);
#pragma omp for schedule(static)
        for (int el = 0; el < b->mb; el++) {
            const int env = b->env_start + el;
            for (int t = 0; t < T; t++) {
                Step* s = &steps[t];
                for (int l = 0; l < L; l++)
                    for (int k = 0; k < H; k++)
                        s->s_in[l][k] = (double)b->r_state[rstate_off(b, t, l, env) + k];
                step_forward(&w, L, b->r_obs + ((size_t)t * b->n + env) * CFP_REC_BYTES, s);
            }
            double dc[CFP_MAX_LAYERS][H];
            memset(dc, 0, sizeof(dc));
            for (int t = T - 1; t >= 0; t--) {
                Step* s = &steps[t];
                const size_t o = (size_t)t * b->n + env;
                double dlog[A], dv, lp, lv, le;
                head_terms(&w, b, s->x[L], o, amean, ainv, inv_batch, &lp, &lv, &le,
                           dlog, &dv);
                s_pg += lp; s_v += lv; s_e += le;
                double dh[H], dhx[H], dhn[H], h3q[H];
                for (int k = 0; k < H; k++) dh[k] = qa(dv) * (double)w.W_v[k];
                for (int k = 0; k < H; k++) h3q[k] = qa(s->x[L][k]);
                for (int a = 0; a < A; a++) {
                    gb_a[a] += dlog[a];
                    const double dq = qa(dlog[a]);
                    for (int k = 0; k < H; k++) {
                        dh[k] += (double)w.W_a[a * H + k] * dq;
                        gW_a[a * H + k] += dq * h3q[k];
                    }
                }
                for (int k = 0; k < H; k++) dh[k] = qs(dh[k]);
                gb_v[0] += dv;
                for (int k = 0; k < H; k++) gW_v[k] += qa(dv) * h3q[k];
                memset(dhx, 0, sizeof(dhx));
                const int cut = (t == T - 1) || ((t + 1) % b->seg_len) == 0;
                const int done_t = b->r_done[o] != 0;
                for (int l = L - 1; l >= 0; l--) {
                    const float* Wl = w.W_gru + (size_t)l * G * H;
                    double* gWl = gW_gru + (size_t)l * G * H;
                    double dpre[G];
                    for (int k = 0; k < H; k++) {
                        if (cut) dc[l][k] = 0.0;
                        const double dhout = dh[k] + dhx[k];
                        const double zh = qs(s->zh[l][k]);
                        const double sgv = sig(qs(s->zg[l][k]));
                        const double gh = gfun(zh);
                        const double p = sig(qs(s->zp[l][k]));
                        const double s_in = s->s_in[l][k];
                        const double out = s_in + sgv * (gh - s_in);
                        const double dout = dhout * p + (done_t ? 0.0 : dc[l][k]);
                        dpre[2 * H + k] = qs(dhout * (out - qs(s->x[l][k])) * p * (1.0 - p));
                        dhx[k] = qs(dhout * (1.0 - p));
                        dc[l][k] = dout * (1.0 - sgv);
                        dpre[H + k] = qs(dout * (gh - s_in) * sgv * (1.0 - sgv));
                        dpre[k] = qs(dout * sgv * dgfun(zh));
                    }
                    memset(dhn, 0, sizeof(dhn));
                    double xq[H];
                    for (int j = 0; j < H; j++) xq[j] = qa(s->x[l][j]);
                    for (int r = 0; r < G; r++) {
                        const double d = qa(dpre[r]);
                        if (d == 0.0) continue;
                        const float* wr = Wl + (size_t)r * H;
                        double* gr = gWl + (size_t)r * H;
                        for (int j = 0; j < H; j++) {
                            gr[j] += d * xq[j];
                            dhn[j] += (double)wr[j] * d;
                        }
                    }
                    if (l > 0)
                        for (int k = 0; k < H; k++) dh[k] = qs(dhn[k]);
                    else
                        memcpy(dh, dhn, sizeof(dh));
                }
                for (int k = 0; k < H; k++) {
                    dh[k] = qs(dh[k] + dhx[k]);
                    gb_enc[k] += dh[k];
                }
                /* dW_enc straight from the records: the 768 leading map bytes are exact in
                 * bf16 and multiply either dh_enc rounded like every other operand of the
                 * mode (split kernels on) or an exact three-term bf16 split of it (split
                 * kernels off: g_map_exact); the other 75 features go through the mode's
                 * GEMM either way. */
                double dhq[H];
                for (int k = 0; k < H; k++) dhq[k] = qa(dh[k]);
                for (int f = 0; f < F; f++) {
                    const double xf = qa((double)s->feat[f]);
                    if (xf == 0.0) continue;
                    double* gr = gW_enc + (size_t)f * H;
                    const double* d = (f < 768 && g_map_exact) ? dh : dhq;
                    for (int k = 0; k < H; k++) gr[k] += xf * d[k];
                }
            }
        }
        free(steps);
        g_q = 0;
        g_map_exact = 0;
    }
    for (int t = 0; t < nth; t++) {
        const double* g = gbuf + pc * (size_t)t;
        for (size_t i = 0; i < pc; i++) grads[i] += g[i];
    }
    free(gbuf);
    if (loss3) { loss3[0] = s_pg; loss3[1] = s_v; loss3[2] = s_e; }
}

/* Smallest |zh| over every (step, env of the minibatch, layer, unit) of the recompute.  The
 * candidate g(zh) = zh + 0.5 (zh >= 0) / sigmoid(zh) (craftax_full.cu:9357) is continuous at
 * zero but its derivative jumps from 1/4 to 1 there, so the update's gradient is
 * discontinuous in the parameters wherever a zh is zero: a batch with a zh inside fp32
 * rounding of zero has two equally valid gradients, and a test that compares an fp32
 * evaluation with this oracle has to know.  bf16_ops: the zh of the bf16-operand update. */
double cfo_ppo_min_abs_zh(const float* params, const cfo_ppo_batch* b, int bf16_ops) {
    const int L = b->layers, T = b->T;
    float* pq = bf16_ops ? bf16_weights(params, L) : NULL;
    const Weights w = split(pq ? pq : params, L);
    double best = 1e300;
    g_q = bf16_ops ? 1 : 0;
    Step* s = (Step*)malloc(sizeof(Step));
    for (int el = 0; el < b->mb; el++) {
        const int env = b->env_start + el;
        for (int t = 0; t < T; t++) {
            for (int l = 0; l < L; l++)
                for (int k = 0; k < H; k++)
                    s->s_in[l][k] = (double)b->r_state[rstate_off(b, t, l, env) + k];
            step_forward(&w, L, b->r_obs + ((size_t)t * b->n + env) * CFP_REC_BYTES, s);
            for (int l = 0; l < L; l++)
                for (int k = 0; k < H; k++)
                    if (fabs(s->zh[l][k]) < best) best = fabs(s->zh[l][k]);
        }
    }
    free(s);
    free(pq);
    g_q = 0;
    return best;
}

/* k_gae :10617-10634, in fp64 on fp32 inputs. */
void cfo_gae_f64(const float* values, const float* rewards, const uint8_t* dones,
                 const float* v_boot, double* adv, double* ret, int n, int T,
                 double gamma, double lam) {
    for (int e = 0; e < n; e++) {
        double Aacc = 0.0;
        for (int t = T - 1; t >= 0; t--) {
            const size_t o = (size_t)t * n + e;
            const double vnext = (t == T - 1) ? (double)v_boot[e] : (double)values[o + n];
            const double nonterm = dones[o] ? 0.0 : 1.0;
            const double delta = (double)rewards[o] + gamma * vnext * nonterm - (double)values[o];
            Aacc = delta + gamma * lam * nonterm * Aacc;
            adv[o] = Aacc;
            ret[o] = Aacc + (double)values[o];
        }
    }
}

/* k_adam :10668-10686 in fp64; step is the 1-based step number. */
void cfo_adam_f64(double* params, const double* grads, double* m, double* v,
                  size_t count, int step, double lr, double beta1, double beta2,
                  double eps) {
    const double c1 = 1.0 - pow(beta1, (double)step);
    const double c2 = 1.0 - pow(beta2, (double)step);
    for (size_t i = 0; i < count; i++) {
        const double g = grads[i];
        m[i] = beta1 * m[i] + (1.0 - beta1) * g;
        v[i] = beta2 * v[i] + (1.0 - beta2) * g * g;
        params[i] -= lr * (m[i] / c1) / (sqrt(v[i] / c2) + eps);
    }
}
