/*
 * CPU restatement of the policy forward.  TEST INFRASTRUCTURE ONLY (see cfo.h).
 *
 * Follows craftax_full.cu:
 *   k_policy_ref_l3                         :9778-9854  (the scalar spec)
 *   cf_nn_sigmoid / cf_nn_mingru_g          :9133-9138
 *   k_mingru_epi_fwd (state zeroing, order) :9350-9395
 *   parameter arena layout                  :9094-9102
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "cfo.h"

enum { H = CFP_HIDDEN, G = CFP_GRU, FM = CFP_OBS_MAP };

int cfo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static double sigmoid64(double x) { return 1.0 / (1.0 + exp(-x)); }
static double mingru_g64(double x) { return x >= 0.0 ? x + 0.5 : sigmoid64(x); }

/* Shared by the full-game (F = 843, A = 43) and classic-game (F = 1345, A = 17)
 * policies: the arena has the same segment order for both
 * (craftax_full.cu:9094-9102, craftax_classic.cu:1526-1533). */
static void forward_f64_impl(const float* params, int layers, int n, int F, int A,
                             const float* x, const double* state_in,
                             const float* prev_terminals, double* h_enc,
                             double* r_state, double* state_out, double* h3,
                             double* logits, double* values) {
    const float* W_enc = params;
    const float* b_enc = W_enc + (size_t)F * H;
    const float* W_gru = b_enc + H;
    const float* W_a = W_gru + (size_t)layers * G * H;
    const float* b_a = W_a + (size_t)A * H;
    const float* W_v = b_a + A;
    const float* b_v = W_v + H;
    const size_t hn = (size_t)H * n;

#pragma omp parallel for schedule(static)
    for (int e = 0; e < n; e++) {
        double h[H], h2[H];
        const float* xe = x + (size_t)e * F;
        for (int k = 0; k < H; k++) h[k] = (double)b_enc[k];
        for (int f = 0; f < F; f++) {
            const double xf = (double)xe[f];
            if (xf == 0.0) continue;
            const float* w = W_enc + (size_t)f * H;
            for (int k = 0; k < H; k++) h[k] += xf * (double)w[k];
        }
        if (h_enc) memcpy(h_enc + (size_t)e * H, h, sizeof(h));
        const int dz = prev_terminals && prev_terminals[e] != 0.0f;
        for (int l = 0; l < layers; l++) {
            const float* Wl = W_gru + (size_t)l * G * H;
            const size_t so = (size_t)l * hn + (size_t)e * H;
            for (int k = 0; k < H; k++) {
                const double st = dz ? 0.0 : state_in[so + k];
                if (r_state) r_state[so + k] = st;
                double zh = 0.0, zg = 0.0, zp = 0.0;
                const float* wh = Wl + (size_t)k * H;
                const float* wg = Wl + (size_t)(H + k) * H;
                const float* wp = Wl + (size_t)(2 * H + k) * H;
                for (int j = 0; j < H; j++) {
                    zh += (double)wh[j] * h[j];
                    zg += (double)wg[j] * h[j];
                    zp += (double)wp[j] * h[j];
                }
                const double out = st + sigmoid64(zg) * (mingru_g64(zh) - st);
                const double p = sigmoid64(zp);
                h2[k] = p * out + (1.0 - p) * h[k];
                if (state_out) state_out[so + k] = out;
            }
            memcpy(h, h2, sizeof(h));
        }
        if (h3) memcpy(h3 + (size_t)e * H, h, sizeof(h));
        if (logits)
            for (int a = 0; a < A; a++) {
                double z = (double)b_a[a];
                for (int j = 0; j < H; j++) z += (double)W_a[a * H + j] * h[j];
                logits[(size_t)e * A + a] = z;
            }
        if (values) {
            double v = (double)b_v[0];
            for (int j = 0; j < H; j++) v += (double)W_v[j] * h[j];
            values[e] = v;
        }
    }
}

void cfo_forward_f64(const float* params, int layers, int n, const float* x,
                     const double* state_in, const float* prev_terminals,
                     double* h_enc, double* r_state, double* state_out,
                     double* h3, double* logits, double* values) {
    forward_f64_impl(params, layers, n, CFP_OBS, CFP_ACTIONS, x, state_in, prev_terminals,
                     h_enc, r_state, state_out, h3, logits, values);
}

/* Classic game.  Record -> 1345 features as encode_obs_kernel reads them
 * (craftax_classic.cu:1714-1751; layout :50-59): per view cell a block one-hot
 * (21 channels: 17 block types + 4 mob bits), 12 inventory + 4 intrinsics as
 * (float)v / 10, direction one-hot, light, sleeping. */
void cfo_classic_expand(const uint8_t* rec, float* x) {
    memset(x, 0, sizeof(float) * CFP_CLASSIC_OBS);
    for (int cell = 0; cell < 63; cell++) {
        x[cell * 21 + (int8_t)rec[cell]] = 1.0f;
        const uint8_t m = rec[63 + cell];
        for (int j = 0; j < 4; j++)
            if (m & (1 << j)) x[cell * 21 + 17 + j] = 1.0f;
    }
    int f = 63 * 21;
    for (int j = 0; j < 16; j++) x[f++] = (float)(int8_t)rec[126 + j] / 10.0f;
    const int dir = (int8_t)rec[142];
    for (int d = 1; d <= 4; d++) x[f++] = dir == d ? 1.0f : 0.0f;
    float light;
    memcpy(&light, rec + 144, sizeof(float));
    x[f++] = light;
    x[f++] = rec[143] ? 1.0f : 0.0f;
}

void cfo_classic_forward_f64(const float* params, int layers, int n, const float* x,
                             const double* state_in, const float* prev_terminals,
                             double* h_enc, double* r_state, double* state_out,
                             double* h3, double* logits, double* values) {
    forward_f64_impl(params, layers, n, CFP_CLASSIC_OBS, CFP_CLASSIC_ACTIONS, x, state_in,
                     prev_terminals, h_enc, r_state, state_out, h3, logits, values);
}

static float sigmoid32(float x) { return 1.0f / (1.0f + expf(-x)); }
static float mingru_g32(float x) { return x >= 0.0f ? x + 0.5f : sigmoid32(x); }

void cfo_forward_f32(const float* params, int layers, int n, const uint8_t* rec,
                     float* state, const float* prev_terminals, float* av,
                     int threads) {
    enum { F = CFP_OBS, A = CFP_ACTIONS };
    const float* W_enc = params + CFP_OFF_W_ENC;
    const float* b_enc = params + CFP_OFF_B_ENC;
    const float* W_gru = params + CFP_OFF_W_GRU;
    const float* W_a = params + CFP_OFF_W_A(layers);
    const float* b_a = params + CFP_OFF_B_A(layers);
    const float* W_v = params + CFP_OFF_W_V(layers);
    const float* b_v = params + CFP_OFF_B_V(layers);
    const size_t hn = (size_t)H * n;
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#else
    threads = 1;
#endif

#pragma omp parallel for schedule(static) num_threads(threads)
    for (int e = 0; e < n; e++) {
        float h[H], h2[H];
        const uint8_t* r = rec + (size_t)e * CFP_REC_BYTES;
        for (int k = 0; k < H; k++) h[k] = b_enc[k];
        for (int f = 0; f < F; f++) {
            float xf;
            if (f < FM) xf = (float)r[f];
            else memcpy(&xf, r + FM + 4 * (f - FM), sizeof(float));
            if (xf == 0.0f) continue;
            const float* w = W_enc + (size_t)f * H;
            for (int k = 0; k < H; k++) h[k] = fmaf(xf, w[k], h[k]);
        }
        const int dz = prev_terminals && prev_terminals[e] != 0.0f;
        for (int l = 0; l < layers; l++) {
            const float* Wl = W_gru + (size_t)l * G * H;
            float* st_l = state + (size_t)l * hn + (size_t)e * H;
            for (int k = 0; k < H; k++) {
                const float st = dz ? 0.0f : st_l[k];
                float zh = 0.0f, zg = 0.0f, zp = 0.0f;
                const float* wh = Wl + (size_t)k * H;
                const float* wg = Wl + (size_t)(H + k) * H;
                const float* wp = Wl + (size_t)(2 * H + k) * H;
                for (int j = 0; j < H; j++) {
                    zh = fmaf(wh[j], h[j], zh);
                    zg = fmaf(wg[j], h[j], zg);
                    zp = fmaf(wp[j], h[j], zp);
                }
                const float out = st + sigmoid32(zg) * (mingru_g32(zh) - st);
                const float p = sigmoid32(zp);
                h2[k] = p * out + (1.0f - p) * h[k];
                st_l[k] = out;
            }
            memcpy(h, h2, sizeof(h));
        }
        float* ave = av + (size_t)e * CFP_AV;
        for (int a = 0; a < A; a++) {
            float z = b_a[a];
            for (int j = 0; j < H; j++) z = fmaf(W_a[a * H + j], h[j], z);
            ave[a] = z;
        }
        float v = b_v[0];
        for (int j = 0; j < H; j++) v = fmaf(W_v[j], h[j], v);
        ave[A] = v;
    }
}

/* cf_nn_sample_action (craftax_full.cu:9147-9165): max-shifted expf, ascending
 * cumulative sum, first action with u*total <= cum, last action as the
 * fall-through; logprob = log softmax at the action.  fp32 like the reference. */
int cfo_sample_action(const float* logits, int actions, float u, float* logprob) {
    float m = logits[0];
    for (int a = 1; a < actions; a++) m = fmaxf(m, logits[a]);
    float p[64], total = 0.0f;
    for (int a = 0; a < actions; a++) {
        p[a] = expf(logits[a] - m);
        total += p[a];
    }
    const float target = u * total;
    float cum = 0.0f;
    int action = actions - 1;
    for (int a = 0; a < actions; a++) {
        cum += p[a];
        if (target <= cum) { action = a; break; }
    }
    if (logprob) *logprob = logits[action] - m - logf(total);
    return action;
}

/* Philox4x32-10 block function (Salmon et al., SC'11; the generator of the
 * reference's curandStatePhilox4_32_10_t, craftax_full.cu:9123-9131, :9732-9736). */
void cfo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; r++) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c1 = (uint32_t)p1; c3 = (uint32_t)p0; c0 = n0; c2 = n2;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* First 32-bit draw after curand_init(seed, subsequence, offset) of a Philox state:
 * key = seed, counter = subsequence * 2^64 + offset / 4, output word offset % 4.
 * Pinned against rocRAND's rocrand_init + rocrand (tests/test_oracle_policy.py). */
uint32_t cfo_philox_draw(uint64_t seed, uint64_t subsequence, uint64_t offset) {
    const uint64_t blk = offset >> 2;
    const uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subsequence,
                             (uint32_t)(subsequence >> 32)};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t out[4];
    cfo_philox4x32_10(ctr, key, out);
    return out[offset & 3];
}

/* curand_uniform of that draw: x * 2^-32 + 2^-33, in (0, 1] (cuRAND's _curand_uniform;
 * the product is exact, so fused or not gives the same float).  rocRAND adds 2^-32
 * instead, which is why the float is not what the rocRAND check compares. */
float cfo_philox_uniform(uint64_t seed, uint64_t subsequence, uint64_t offset) {
    return fmaf((float)cfo_philox_draw(seed, subsequence, offset), 2.3283064365386963e-10f,
                1.1641532182693481e-10f);
}

/* Distance of u*total from the nearest cumulative-sum boundary, relative to
 * total: draws this close to a boundary may legitimately land on either side
 * when expf differs by an ulp between implementations. */
float cfo_sample_margin(const float* logits, int actions, float u) {
    float m = logits[0];
    for (int a = 1; a < actions; a++) m = fmaxf(m, logits[a]);
    float p[64], total = 0.0f;
    for (int a = 0; a < actions; a++) {
        p[a] = expf(logits[a] - m);
        total += p[a];
    }
    const float target = u * total;
    float cum = 0.0f, best = 1e30f;
    for (int a = 0; a < actions; a++) {
        cum += p[a];
        const float d = fabsf(target - cum);
        if (d < best) best = d;
    }
    return best / total;
}
