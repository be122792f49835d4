// C ABI: policy object lifetime, parameter upload, and the forward entry
// points.  Host-side mirror of the reference's CuPolicy layer
// (craftax_full.cu:11758-12092): every device buffer is allocated here at
// create time and owned by the object; step entry points only enqueue work.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <vector>

#include "cfp_common.h"
#include "cfp_internal.h"

namespace cfp {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

}  // namespace cfp


using namespace cfp;

extern "C" {

const char* cfp_last_error(void) { return g_err; }
int cfp_abi_version(void) { return 1; }

static void policy_release(cfp_policy* p) {
    if (!p) return;
    if (p->stream) (void)hipStreamDestroy(p->stream);
    (void)hipFree(p->params);
    (void)hipFree(p->we_pk);
    (void)hipFree(p->we_s3);
    (void)hipFree(p->wg_pk);
    (void)hipFree(p->wav_pk);
    (void)hipFree(p->we_bf);
    (void)hipFree(p->wg_bf);
    (void)hipFree(p->wav_bf);
    (void)hipFree(p->t16);
    (void)hipFree(p->enc_x9);
    (void)hipFree(p->h_state);
    (void)hipFree(p->rec);
    (void)hipFree(p->h_enc);
    (void)hipFree(p->h3);
    (void)hipFree(p->logits);
    delete p;
}

// Xavier-uniform weights, U(+-1/sqrt(fan_in)) biases; segment order is the
// arena order (craftax_full.cu:11832-11840).
static void init_params_host(std::vector<float>& w, int layers, int variant,
                             uint64_t seed) {
    struct Seg { size_t off, count; float bound; };
    const Arena ar = arena_of(variant, layers);
    const float xe = sqrtf(6.0f / (float)(ar.obs + CFP_HIDDEN));
    const float xg = sqrtf(6.0f / (float)(CFP_HIDDEN + CFP_GRU));
    const float xa = sqrtf(6.0f / (float)(CFP_HIDDEN + ar.actions));
    const float xv = sqrtf(6.0f / (float)(CFP_HIDDEN + 1));
    const float be = 1.0f / sqrtf((float)ar.obs);
    const float bh = 1.0f / sqrtf((float)CFP_HIDDEN);
    const Seg segs[7] = {
        {ar.w_enc, (size_t)ar.obs * CFP_HIDDEN, xe},
        {ar.b_enc, CFP_HIDDEN, be},
        {ar.w_gru, (size_t)layers * CFP_GRU * CFP_HIDDEN, xg},
        {ar.w_a, (size_t)ar.actions * CFP_HIDDEN, xa},
        {ar.b_a, (size_t)ar.actions, bh},
        {ar.w_v, CFP_HIDDEN, xv},
        {ar.b_v, 1, bh},
    };
    for (int s = 0; s < 7; s++)
        for (size_t i = 0; i < segs[s].count; i++) {
            float u = unit24(mix64(seed, (uint64_t)s, i));
            w[segs[s].off + i] = (2.0f * u - 1.0f) * segs[s].bound;
        }
}

static int policy_create(cfp_policy** out, int num_envs, int layers, uint64_t seed,
                         int variant);

int cfp_policy_create(cfp_policy** out, int num_envs, int layers, uint64_t seed) {
    return policy_create(out, num_envs, layers, seed, 0);
}
int cfp_policy_create_classic(cfp_policy** out, int num_envs, int layers,
                              uint64_t seed) {
    return policy_create(out, num_envs, layers, seed, 1);
}
int cfp_policy_variant(const cfp_policy* p) { return p ? p->variant : -1; }

static int policy_create(cfp_policy** out, int num_envs, int layers, uint64_t seed,
                         int variant) {
    CFP_REQUIRE(out != nullptr, "cfp_policy_create: out is NULL");
    *out = nullptr;
    CFP_REQUIRE(num_envs > 0 && num_envs % 32 == 0,
                "policy modes need the env count to be a positive multiple of "
                "32 (got %d)", num_envs);
    CFP_REQUIRE(layers >= 1 && layers <= CFP_MAX_LAYERS,
                "layers must be in 1..%d (got %d)", CFP_MAX_LAYERS, layers);
    cfp_policy* p = new cfp_policy();
    p->n = num_envs;
    p->layers = layers;
    p->variant = variant;
    p->param_count = arena_of(variant, layers).count;
    const size_t rec_bytes = variant ? CFP_CLASSIC_REC_BYTES : CFP_REC_BYTES;
    const size_t hn = (size_t)CFP_HIDDEN * num_envs;
#define CFP_ALLOC(ptr, bytes)                                                 \
    do {                                                                      \
        hipError_t e_ = hipMalloc((void**)&(ptr), (bytes));                   \
        if (e_ != hipSuccess) {                                               \
            set_error("hipMalloc(%zu bytes) for %s failed: %s",               \
                      (size_t)(bytes), #ptr, hipGetErrorString(e_));          \
            policy_release(p);                                                \
            return 1;                                                         \
        }                                                                     \
    } while (0)
    CFP_ALLOC(p->params, p->param_count * sizeof(float));
    CFP_ALLOC(p->we_pk, (size_t)(kKbEnc + kEncPadBlocks) * 2048 * sizeof(float));
    CFP_ALLOC(p->we_s3, kEncSplitBf16 * sizeof(uint16_t));
    CFP_ALLOC(p->wg_pk,
              ((size_t)layers * kGruPackFloats + 4 * 6 * 64 * 4) * sizeof(float));
    CFP_ALLOC(p->wav_pk, kAvPackFloats * sizeof(float));
    CFP_ALLOC(p->we_bf, kEncPackFloats * sizeof(uint16_t));
    CFP_ALLOC(p->wg_bf, (size_t)layers * kGruPackFloats * sizeof(uint16_t));
    CFP_ALLOC(p->wav_bf, kAvPackFloats * sizeof(uint16_t));
    if (variant == 0) CFP_ALLOC(p->t16, t16_mirror_bytes(layers));
    if (variant == 0) CFP_ALLOC(p->enc_x9, enc_mirror_bytes());
    CFP_ALLOC(p->h_state, (size_t)layers * hn * sizeof(float));
    CFP_ALLOC(p->rec, (size_t)num_envs * rec_bytes);
    CFP_ALLOC(p->h_enc, hn * sizeof(float));
    CFP_ALLOC(p->h3, hn * sizeof(float));
    CFP_ALLOC(p->logits, (size_t)CFP_AV * num_envs * sizeof(float));
#undef CFP_ALLOC
    hipError_t e = hipStreamCreateWithFlags(&p->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        set_error("hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
        policy_release(p);
        return 1;
    }
    e = hipMemset(p->h_state, 0, (size_t)layers * hn * sizeof(float));
    if (e == hipSuccess) e = hipMemset(p->rec, 0, (size_t)num_envs * rec_bytes);
    if (e != hipSuccess) {
        set_error("hipMemset failed: %s", hipGetErrorString(e));
        policy_release(p);
        return 1;
    }
    std::vector<float> w(p->param_count);
    init_params_host(w, layers, variant, seed);
    if (cfp_policy_set_params(p, w.data(), w.size()) != 0) {
        policy_release(p);
        return 1;
    }
    *out = p;
    return 0;
}

void cfp_policy_destroy(cfp_policy* p) { policy_release(p); }

int cfp_policy_num_envs(const cfp_policy* p) { return p ? p->n : 0; }
int cfp_policy_layers(const cfp_policy* p) { return p ? p->layers : 0; }
size_t cfp_policy_param_count(const cfp_policy* p) {
    return p ? p->param_count : 0;
}

int cfp_policy_set_params(cfp_policy* p, const float* host_params,
                          size_t count) {
    CFP_REQUIRE(p && host_params, "cfp_policy_set_params: NULL argument");
    CFP_REQUIRE(count == p->param_count,
                "param count mismatch: got %zu, policy has %zu", count,
                p->param_count);
    CFP_HIP_TRY(hipMemcpy(p->params, host_params, count * sizeof(float),
                          hipMemcpyHostToDevice));
    if (cfp_policy_refresh_weights(p, nullptr) != 0) return 1;
    CFP_HIP_TRY(hipDeviceSynchronize());
    return 0;
}

int cfp_policy_init_reference(cfp_policy* p, uint64_t seed) {
    CFP_REQUIRE(p, "cfp_policy_init_reference: NULL policy");
    const Arena ar = arena_of(p->variant, p->layers);
    const float be = 1.0f / sqrtf((float)ar.obs);
    const float bh = 1.0f / sqrtf((float)CFP_HIDDEN);
    struct Seg { size_t off, count; float bound; };
    const Seg segs[7] = {
        {ar.w_enc, (size_t)ar.obs * CFP_HIDDEN, be},
        {ar.b_enc, CFP_HIDDEN, be},
        {ar.w_gru, (size_t)p->layers * CFP_GRU * CFP_HIDDEN, bh},
        {ar.w_a, (size_t)ar.actions * CFP_HIDDEN, bh},
        {ar.b_a, (size_t)ar.actions, bh},
        {ar.w_v, CFP_HIDDEN, bh},
        {ar.b_v, 1, bh},
    };
    std::vector<float> w(p->param_count);
    for (int s = 0; s < 7; s++)
        for (size_t i = 0; i < segs[s].count; i++)
            w[segs[s].off + i] =
                (2.0f * philox_uniform(seed, (uint64_t)s, (uint64_t)i) - 1.0f) * segs[s].bound;
    return cfp_policy_set_params(p, w.data(), w.size());
}

int cfp_policy_get_params(const cfp_policy* p, float* host_params,
                          size_t count) {
    CFP_REQUIRE(p && host_params, "cfp_policy_get_params: NULL argument");
    CFP_REQUIRE(count == p->param_count,
                "param count mismatch: got %zu, policy has %zu", count,
                p->param_count);
    CFP_HIP_TRY(hipMemcpy(host_params, p->params, count * sizeof(float),
                          hipMemcpyDeviceToHost));
    return 0;
}

// CFW1 files (craftax_full.cu:12244-12293): uint32 {magic "CFW1", hidden, layers,
// param count} followed by the fp32 params arena.
static constexpr uint32_t kCkptMagic = 0x31574643u;

int cfp_save_weights(const cfp_policy* p, const char* path) {
    CFP_REQUIRE(p && path, "cfp_save_weights: NULL argument");
    std::vector<float> h(p->param_count);
    CFP_HIP_TRY(hipMemcpy(h.data(), p->params, h.size() * sizeof(float), hipMemcpyDeviceToHost));
    FILE* f = fopen(path, "wb");
    CFP_REQUIRE(f, "cannot write %s", path);
    const uint32_t hdr[4] = {kCkptMagic, CFP_HIDDEN, (uint32_t)p->layers,
                             (uint32_t)p->param_count};
    const bool ok = fwrite(hdr, sizeof(hdr), 1, f) == 1 &&
                    fwrite(h.data(), sizeof(float), h.size(), f) == h.size();
    const bool closed = fclose(f) == 0;
    CFP_REQUIRE(ok && closed, "short write to %s", path);
    return 0;
}

int cfp_load_weights(cfp_policy* p, const char* path) {
    CFP_REQUIRE(p && path, "cfp_load_weights: NULL argument");
    FILE* f = fopen(path, "rb");
    CFP_REQUIRE(f, "cannot read %s", path);
    uint32_t hdr[4];
    if (fread(hdr, sizeof(hdr), 1, f) != 1 || hdr[0] != kCkptMagic || hdr[1] != CFP_HIDDEN ||
        hdr[2] != (uint32_t)p->layers || hdr[3] != (uint32_t)p->param_count) {
        fclose(f);
        set_error("%s: bad header (want h%dx%d, %zu params)", path, CFP_HIDDEN, p->layers,
                  p->param_count);
        return 1;
    }
    std::vector<float> h(p->param_count);
    const size_t got = fread(h.data(), sizeof(float), h.size(), f);
    fclose(f);
    CFP_REQUIRE(got == h.size(), "%s: truncated", path);
    return cfp_policy_set_params(p, h.data(), h.size());   // also refreshes the mirrors
}

int cfp_policy_refresh_weights(cfp_policy* p, void* stream) {
    CFP_REQUIRE(p, "cfp_policy_refresh_weights: NULL policy");
    if (launch_pack_weights(p->params, p->layers, p->variant, p->we_pk, p->wg_pk, p->wav_pk,
                            (hipStream_t)stream) != 0)
        return 1;
    if (launch_pack_enc_split(p->params, p->layers, p->variant, p->we_s3, (hipStream_t)stream) != 0)
        return 1;
    if (launch_pack_weights_bf16(p->params, p->layers, p->variant, p->we_bf, p->wg_bf, p->wav_bf,
                                 (hipStream_t)stream) != 0)
        return 1;
    if (p->t16) return launch_pack_weights_t16(p->params, p->layers, p->t16, (hipStream_t)stream);
    return 0;
}

int cfp_policy_set_small_tiles(cfp_policy* p, int on) {
    CFP_REQUIRE(p, "cfp_policy_set_small_tiles: NULL policy");
    CFP_REQUIRE(!on || p->t16, "16-env tiles exist for the full-game policy only");
    p->small_tiles = on ? 1 : 0;
    return 0;
}
int cfp_policy_small_tiles(const cfp_policy* p) { return p ? p->small_tiles : -1; }

int cfp_policy_set_gemm_bf16(cfp_policy* p, int on) {
    CFP_REQUIRE(p, "cfp_policy_set_gemm_bf16: NULL policy");
    p->gemm_bf16 = on ? 1 : 0;
    return 0;
}
int cfp_policy_gemm_bf16(const cfp_policy* p) { return p ? p->gemm_bf16 : -1; }

float* cfp_policy_params(cfp_policy* p) { return p->params; }
float* cfp_policy_state(cfp_policy* p) { return p->h_state; }
uint8_t* cfp_policy_rec(cfp_policy* p) { return p->rec; }
float* cfp_policy_h_enc(cfp_policy* p) { return p->h_enc; }
float* cfp_policy_h3(cfp_policy* p) { return p->h3; }
float* cfp_policy_logits(cfp_policy* p) { return p->logits; }
void* cfp_policy_stream(cfp_policy* p) { return (void*)p->stream; }

static void fill_weights(const cfp_policy* p, FwdArgs& a) { cfp::fill_forward_weights(p, a); }

}  // extern "C"

void cfp::fill_forward_weights(const cfp_policy* p, FwdArgs& a) {
    const Arena ar = arena_of(p->variant, p->layers);
    a.we_pk = reinterpret_cast<const f4*>(p->we_pk);
    a.we_s3 = reinterpret_cast<const u4*>(p->we_s3);
    a.w_enc = p->params + ar.w_enc;
    a.b_enc = p->params + ar.b_enc;
    a.wg_pk = reinterpret_cast<const f4*>(p->wg_pk);
    a.wav_pk = reinterpret_cast<const f4*>(p->wav_pk);
    a.b_a = p->params + ar.b_a;
    a.b_v = p->params + ar.b_v;
    a.variant = p->variant;
    a.actions = ar.actions;
    a.we_bf = reinterpret_cast<const u4*>(p->we_bf);
    a.wg_bf = reinterpret_cast<const u4*>(p->wg_bf);
    a.wav_bf = reinterpret_cast<const u4*>(p->wav_bf);
    a.bf16 = p->gemm_bf16;
    a.rs_bf16 = p->rs_bf16;   // (the window recompute sets its own)
    if (p->small_tiles && p->t16)
        t16_mirror_layout(p->t16, p->layers, &a.t16_enc_s, &a.t16_enc_t, &a.t16_wg, &a.t16_wav);
}

extern "C" {

// Launch over [0, n) in chunks; every per-env pointer is advanced by the
// chunk start, the layer stride of state / r_state stays that of the full n.
static int run_chunked(FwdArgs a, int n, int chunk, hipStream_t st) {
    CFP_REQUIRE(n > 0 && n % 32 == 0,
                "env count must be a positive multiple of 32 (got %d)", n);
    if (chunk <= 0 || chunk > n) chunk = n;
    CFP_REQUIRE(chunk % 32 == 0, "chunk must be a multiple of 32 (got %d)",
                chunk);
    for (int e0 = 0; e0 < n; e0 += chunk) {
        FwdArgs c = a;
        c.n = n - e0 < chunk ? n - e0 : chunk;
        const size_t off = (size_t)e0;
        if (a.rec)
            c.rec = a.rec + off * (a.variant ? CFP_CLASSIC_REC_BYTES : CFP_REC_BYTES);
        if (a.x0) c.x0 = a.x0 + off * CFP_HIDDEN;
        if (a.state) c.state = a.state + off * CFP_HIDDEN;
        if (a.terminals) c.terminals = a.terminals + off;
        if (a.r_state) c.r_state = a.r_state + off * CFP_HIDDEN;
        if (a.h_enc_out) c.h_enc_out = a.h_enc_out + off * CFP_HIDDEN;
        if (a.h3_out) c.h3_out = a.h3_out + off * CFP_HIDDEN;
        if (a.av_out) c.av_out = a.av_out + off * (a.actions + 1);
        if (launch_forward(c, st) != 0) return 1;
    }
    return 0;
}

int cfp_encode_step(cfp_policy* p, const uint8_t* d_rec_row, int n,
                    void* stream) {
    CFP_REQUIRE(p, "cfp_encode_step: NULL policy");
    CFP_REQUIRE(n <= p->n, "cfp_encode_step: n=%d exceeds the policy's %d envs",
                n, p->n);
    FwdArgs a{};
    fill_weights(p, a);
    a.rec = d_rec_row ? d_rec_row : p->rec;
    a.h_enc_out = p->h_enc;
    a.layers = 0;
    a.do_head = 0;
    return run_chunked(a, n, 0, (hipStream_t)stream);
}

int cfp_gru_chain(cfp_policy* p, const float* d_x0, float* d_state,
                  const float* d_terminals, float* d_r_state_t, float* d_h3,
                  int n, int chunk, void* stream) {
    CFP_REQUIRE(p && d_x0 && d_state && d_h3, "cfp_gru_chain: NULL argument");
    FwdArgs a{};
    fill_weights(p, a);
    a.x0 = d_x0;
    a.state = d_state;
    a.terminals = d_terminals;
    a.r_state = d_r_state_t;
    a.h3_out = d_h3;
    a.layer_stride = (size_t)n * CFP_HIDDEN;
    a.layers = p->layers;
    a.do_head = 0;
    return run_chunked(a, n, chunk, (hipStream_t)stream);
}

int cfp_head(cfp_policy* p, const float* d_h3, float* d_av, int n,
             void* stream) {
    CFP_REQUIRE(p && d_h3 && d_av, "cfp_head: NULL argument");
    FwdArgs a{};
    fill_weights(p, a);
    a.x0 = d_h3;
    a.av_out = d_av;
    a.layers = 0;
    a.do_head = 1;
    return run_chunked(a, n, 0, (hipStream_t)stream);
}

int cfp_policy_forward(cfp_policy* p, const uint8_t* d_rec_row,
                       const float* d_terminals, float* d_state,
                       float* d_r_state_t, float* d_h_enc, float* d_h3,
                       float* d_av, int n, int chunk, void* stream) {
    CFP_REQUIRE(p, "cfp_policy_forward: NULL policy");
    CFP_REQUIRE(d_state != nullptr || n == p->n,
                "cfp_policy_forward: the object's live state covers %d envs, "
                "n=%d needs an explicit state buffer", p->n, n);
    CFP_REQUIRE(d_rec_row != nullptr || n <= p->n,
                "cfp_policy_forward: n=%d exceeds the record scratch (%d envs)",
                n, p->n);
    CFP_REQUIRE(d_av != nullptr || n <= p->n,
                "cfp_policy_forward: n=%d exceeds the logits buffer (%d envs)",
                n, p->n);
    FwdArgs a{};
    fill_weights(p, a);
    a.rec = d_rec_row ? d_rec_row : p->rec;
    a.terminals = d_terminals;
    a.state = d_state ? d_state : p->h_state;
    a.r_state = d_r_state_t;
    a.h_enc_out = d_h_enc;
    a.h3_out = d_h3;
    a.av_out = d_av ? d_av : p->logits;
    a.layer_stride = (size_t)n * CFP_HIDDEN;
    a.layers = p->layers;
    a.do_head = 1;
    return run_chunked(a, n, chunk, (hipStream_t)stream);
}

// The same step fed by the fp32 feature matrix instead of records: the reference's
// cu_gemm_enc_fwd on xobs (craftax_full.cu:11616) + k_add_bias (:10056), then the fused
// layers and heads from the encoder output.  fp32 features are not exact in bf16, so the
// encoder cannot run on the record path's three-term byte products; it goes through the
// seam's encoder GEMM (and follows the seam's process-wide GEMM switches).
int cfp_policy_forward_features(cfp_policy* p, const float* d_xobs, const float* d_terminals,
                                float* d_state, float* d_r_state_t, float* d_h_enc, float* d_h3,
                                float* d_av, int n, int chunk, void* stream) {
    CFP_REQUIRE(p && d_xobs, "cfp_policy_forward_features: NULL argument");
    CFP_REQUIRE(p->variant == 0, "cfp_policy_forward_features covers the full-game policy");
    CFP_REQUIRE(d_state != nullptr || n == p->n,
                "cfp_policy_forward_features: the object's live state covers %d envs, n=%d needs "
                "an explicit state buffer", p->n, n);
    CFP_REQUIRE((d_h_enc != nullptr && d_av != nullptr) || n <= p->n,
                "cfp_policy_forward_features: n=%d exceeds the object's buffers (%d envs)", n, p->n);
    float* h_enc = d_h_enc ? d_h_enc : p->h_enc;
    const Arena ar = arena_of(0, p->layers);
    // The encoder product on the split kernels where they are on (every fp32 operand as three
    // bf16 parts, nine / six exact products, or one with bf16 inputs); its bias is added where
    // the fused kernel stages h_enc.  Otherwise the fp32 MFMA GEMM and the bias pass.
    const int terms = gemm_split_terms();
    const bool split = terms != 0 && gemm_enc_fwd_x9_ok(n, d_xobs) && p->enc_x9;
    bool bias_at_staging = false;
    if (split) {
        if (gemm_enc_fwd_x9(n, p->params + ar.w_enc, d_xobs, CFP_OBS, h_enc, terms,
                            static_cast<u4*>(p->enc_x9), (hipStream_t)stream))
            return 1;
        // a caller who asked for h_enc gets it with the bias (the same fp32 addition, so the
        // rest of the step sees the same bits either way)
        if (d_h_enc) {
            if (cfp_add_bias(h_enc, p->params + ar.b_enc, n, stream)) return 1;
        } else {
            bias_at_staging = true;
        }
    } else {
        if (gemm_enc_fwd_ld(n, p->params + ar.w_enc, d_xobs, CFP_OBS, h_enc, (hipStream_t)stream)) return 1;
        if (cfp_add_bias(h_enc, p->params + ar.b_enc, n, stream)) return 1;
    }
    FwdArgs a{};
    fill_weights(p, a);
    a.x0 = h_enc;
    a.x0_add_bias = bias_at_staging ? 1 : 0;
    a.terminals = d_terminals;
    a.state = d_state ? d_state : p->h_state;
    a.r_state = d_r_state_t;
    a.h3_out = d_h3;
    a.av_out = d_av ? d_av : p->logits;
    a.layer_stride = (size_t)n * CFP_HIDDEN;
    a.layers = p->layers;
    a.do_head = 1;
    return run_chunked(a, n, chunk, (hipStream_t)stream);
}

}  // extern "C"

namespace cfp {
namespace {
__global__ void k_add_one_u64(uint64_t* ctr) { *ctr += 1; }
}  // namespace

int forward_and_sample(cfp_policy* p, const uint8_t* d_rec_row, const float* d_terminals,
                       float* d_r_state_t, int n, const SampleOut& s, hipStream_t st) {
    CFP_REQUIRE(p && d_rec_row && s.act && s.logp && s.step_ctr && s.ticket,
                "forward_and_sample: NULL argument");
    CFP_REQUIRE(n == p->n, "forward_and_sample: the policy's live state covers %d envs, not %d",
                p->n, n);
    FwdArgs a{};
    fill_weights(p, a);
    a.rec = d_rec_row;
    a.terminals = d_terminals;
    a.state = p->h_state;
    a.r_state = d_r_state_t;
    a.av_out = p->logits;
    a.layer_stride = (size_t)n * CFP_HIDDEN;
    a.layers = p->layers;
    a.do_head = 1;
    a.n = n;
    FwdArgs f = a;
    f.s_act = s.act;
    f.s_logp = s.logp;
    f.s_value = s.value;
    f.s_env_actions = s.env_actions;
    f.s_seed = s.seed;
    f.s_step = s.step_ctr;
    f.s_ticket = s.ticket;
    if (forward_t16_ok(f)) return launch_forward_t16(f, st);
    if (forward_draws(f)) return launch_forward(f, st);
    if (run_chunked(a, n, 0, st) != 0) return 1;
    const bool ride = n < kSampleRowsFrom;   // the sampler's launch bumps the counter itself
    if (value_sample(p->logits, n, a.actions, s.env_actions, s.act, s.logp, s.value, s.seed,
                     s.step_ctr, ride ? s.ticket : nullptr, st) != 0)
        return 1;
    if (!ride) {
        hipLaunchKernelGGL(k_add_one_u64, dim3(1), dim3(1), 0, st, s.step_ctr);
        CFP_HIP_TRY(hipGetLastError());
    }
    return 0;
}
}  // namespace cfp

// ---- synthetic records -------------------------------------------------------
namespace cfp {
// One thread per (env, dword): dwords 0..197 are four map bytes U{0..40},
// dwords 198..248 one tail float U[0,1) on a 24-bit grid.
__global__ void k_synth_records(uint32_t* __restrict__ rec, size_t total_dw,
                                int n, uint64_t seed, uint64_t step) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total_dw) return;
    size_t env = i / 249;
    int d = (int)(i - env * 249);
    uint64_t z = mix64(seed, step, env * 249 + (uint64_t)d);
    uint32_t w;
    if (d < CFP_OBS_MAP / 4) {
        w = (uint32_t)(z & 0xffff) % 41u;
        w |= ((uint32_t)((z >> 16) & 0xffff) % 41u) << 8;
        w |= ((uint32_t)((z >> 32) & 0xffff) % 41u) << 16;
        w |= ((uint32_t)((z >> 48) & 0xffff) % 41u) << 24;
    } else {
        w = __float_as_uint(unit24(z));
    }
    rec[i] = w;
}
}  // namespace cfp

namespace cfp {
// One thread per classic record (148 bytes), 8 draws of 64 bits cover the 63
// mob nibbles; every byte is a pure function of (seed, step, env, position).
__global__ void k_synth_classic(uint8_t* __restrict__ rec, int n, uint64_t seed,
                                uint64_t step) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    uint8_t* o = rec + (size_t)e * CFP_CLASSIC_REC_BYTES;
    for (int c = 0; c < 63; c++) {
        const uint64_t z = mix64(seed, step, (uint64_t)e * 160 + c);
        o[c] = (uint8_t)((z & 0xffff) % 17u);
        const uint32_t r = (uint32_t)(z >> 32);
        o[63 + c] = (r % 50u) == 0 ? (uint8_t)(1u + ((r >> 8) % 15u)) : 0;   // ~2 % of cells
    }
    for (int j = 0; j < 16; j++)
        o[126 + j] = (uint8_t)((mix64(seed, step, (uint64_t)e * 160 + 64 + j) & 0xffff) % 10u);
    const uint64_t z = mix64(seed, step, (uint64_t)e * 160 + 80);
    o[142] = (uint8_t)(1u + (uint32_t)(z & 0xffff) % 4u);
    o[143] = (uint8_t)((z >> 16) & 1u);
    const uint32_t lb = __float_as_uint(unit24(mix64(seed, step, (uint64_t)e * 160 + 81)));
    o[144] = (uint8_t)lb; o[145] = (uint8_t)(lb >> 8);
    o[146] = (uint8_t)(lb >> 16); o[147] = (uint8_t)(lb >> 24);
}
}  // namespace cfp

extern "C" int cfp_synth_classic_records(uint8_t* d_rec, int n, uint64_t seed,
                                         uint64_t step, void* stream) {
    CFP_REQUIRE(d_rec && n > 0, "cfp_synth_classic_records: bad argument");
    hipLaunchKernelGGL(cfp::k_synth_classic, dim3((n + 255) / 256), dim3(256), 0,
                       (hipStream_t)stream, d_rec, n, seed, step);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

extern "C" int cfp_synth_records(uint8_t* d_rec, int n, uint64_t seed,
                                 uint64_t step, void* stream) {
    CFP_REQUIRE(d_rec && n > 0, "cfp_synth_records: bad argument");
    CFP_REQUIRE((reinterpret_cast<uintptr_t>(d_rec) & 3u) == 0,
                "records must be 4-byte aligned");
    size_t total = (size_t)n * 249;
    hipLaunchKernelGGL(cfp::k_synth_records, dim3((unsigned)((total + 255) / 256)),
                       dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<uint32_t*>(d_rec), total, n, seed, step);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}
