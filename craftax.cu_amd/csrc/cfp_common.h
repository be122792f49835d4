// Shared host/device definitions for the gfx950 policy-path library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/cfp.h"

namespace cfp {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

// Workgroup tile of the fused forward: 32 envs x all 256 hidden units,
// 4 wavefronts, wave w owns units [64w, 64w+64).
constexpr int kTileEnvs = 32;
constexpr int kFwdThreads = 256;
// K is consumed in blocks of 8: one 16-byte operand fragment per lane feeds
// four 32x32x2 MFMA steps (lanes 0-31 carry k = 8b+j, lanes 32-63 k = 8b+4+j).
constexpr int kKBlock = 8;
constexpr int kObsPad = 848;                       // 843 rounded up to 8
constexpr int kKbEnc = kObsPad / kKBlock;          // 106
constexpr int kKbMap = CFP_OBS_MAP / kKBlock;      // 99: map bytes end on a block edge
constexpr int kKbHid = CFP_HIDDEN / kKBlock;       // 32
constexpr int kAvPad = 64;                         // head rows padded 44 -> 64
constexpr int kEncPadBlocks = 4;                   // encoder mirror: prefetch overrun

// MFMA-ordered weight mirror sizes, in floats.
constexpr size_t kEncPackFloats = (size_t)kObsPad * CFP_HIDDEN;
constexpr int kKb16Split = (CFP_OBS_MAP + 15) / 16;                   // 50 K blocks of 16 map bytes
// bf16 elements of the split mirror: 50 blocks (full game) or 83 (classic, 1323 cell features)
constexpr size_t kEncSplitBf16 = (size_t)83 * 4 * 6 * 64 * 8;
constexpr size_t kGruPackFloats = (size_t)CFP_GRU * CFP_HIDDEN;   // per layer
constexpr size_t kAvPackFloats = (size_t)kAvPad * CFP_HIDDEN;

void set_error(const char* fmt, ...);

// Counter-based generator shared with the host-side test utilities:
// value(seed, stream, index) is a splitmix64 finalizer of a linear counter.
__host__ __device__ inline uint64_t mix64(uint64_t seed, uint64_t stream, uint64_t index) {
    uint64_t z = seed + stream * 0xD1B54A32D192ED03ULL + (index + 1) * 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}
// uniform on the 24-bit grid [0, 1)
__host__ __device__ inline float unit24(uint64_t z) {
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2,
// 3", SC'11; the generator behind curandStatePhilox4_32_10_t): ten rounds of
//   (c0, c1, c2, c3) <- (hi(M1*c2) ^ c1 ^ k0, lo(M1*c2), hi(M0*c0) ^ c3 ^ k1, lo(M0*c0)),
// the key bumped by the Weyl constants between rounds.
__host__ __device__ inline void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
    for (int r = 0; r < 10; r++) {
        const uint64_t p0 = 0xD2511F53ull * c[0], p1 = 0xCD9E8D57ull * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        c[1] = (uint32_t)p1;
        c[3] = (uint32_t)p0;
        c[0] = n0;
        c[2] = n2;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}
// The first curand_uniform() after curand_init(seed, subsequence, offset, &state) of a
// Philox4_32_10 state, by cuRAND's documented state layout: key = seed, the 128-bit
// counter = subsequence * 2^64 + offset / 4, of whose four output words the draw is word
// offset % 4; uniform = x * 2^-32 + 2^-33, in (0, 1].
__host__ __device__ inline float philox_uniform(uint64_t seed, uint64_t subsequence,
                                                uint64_t offset) {
    const uint64_t blk = offset >> 2;
    uint32_t c[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subsequence,
                     (uint32_t)(subsequence >> 32)};
    philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
    return __builtin_fmaf((float)c[offset & 3], 2.3283064365386963e-10f, 1.1641532182693481e-10f);
}

#define CFP_HIP_TRY(expr)                                                     \
    do {                                                                      \
        hipError_t e_ = (expr);                                               \
        if (e_ != hipSuccess) {                                               \
            cfp::set_error("%s:%d: %s -> %s", __FILE__, __LINE__, #expr,      \
                           hipGetErrorString(e_));                            \
            return 1;                                                         \
        }                                                                     \
    } while (0)

#define CFP_REQUIRE(cond, ...)                                                \
    do {                                                                      \
        if (!(cond)) {                                                        \
            cfp::set_error(__VA_ARGS__);                                      \
            return 1;                                                         \
        }                                                                     \
    } while (0)

// ---- launchers implemented in the .hip files -------------------------------
struct FwdArgs {
    const uint8_t* rec;      // [n][996] or null (then x0 is the layer-0 input)
    const float* x0;         // [n][256] or null
    int x0_add_bias;         // x0 is the encoder product without its bias: staging adds b_enc
    const f4* we_pk;         // packed encoder weights
    const u4* we_s3;         // map rows of W_enc as three bf16 terms (hi, mid, lo) per weight
    const float* b_enc;
    const f4* wg_pk;         // packed gate weights, layers back to back
    const f4* wav_pk;        // packed head weights
    const float* b_a;
    const float* b_v;
    float* state;            // [layers][state_envs][256] in/out, or null
    const float* terminals;  // [n] or null (= no terminal)
    float* r_state;          // like state, or null
    int rs_bf16;             // bf16-input kernel only: r_state (written) and, in the window
                             // recompute, the stored state (read) are bf16 arrays of the same shape
    float* h_enc_out;        // [n][256] or null
    float* h3_out;           // [n][256] or null
    float* av_out;           // [n][44] or null
    size_t layer_stride;     // floats between layers in state / r_state
    int n;                   // envs in this launch (multiple of 32)
    int layers;              // MinGRU layers to run (0 = encoder only)
    int do_head;
    int variant;             // 0 full game (996-byte records), 1 classic (148-byte)
    int actions;             // 43 or 17; av rows = actions + 1
    const float* w_enc;      // classic: unpacked W_enc [1345][256] for the gather
    const u4* we_bf;         // bf16 mirrors, used when bf16 != 0
    const u4* wg_bf;
    const u4* wav_bf;
    int bf16;                // bf16-input / fp32-accumulate kernel
    // mirrors of the 16-env-tile kernel (policy_forward_t16.hip); null = not in use
    const u4* t16_enc_s;
    const f4* t16_enc_t;
    const f4* t16_wg;
    const f4* t16_wav;
    // 16-env-tile kernel only: the draw behind the heads (s_act null = no sampling).
    // Offset *s_step, bumped by the last workgroup through the tickets at *s_ticket.
    int32_t* s_act;
    float* s_logp;
    float* s_value;
    float* s_env_actions;    // or null
    uint64_t s_seed;
    uint64_t* s_step;
    unsigned* s_ticket;
    // Window recompute of the PPO update (fp32 full game only): "env" c of this
    // launch is window column c = (t0 + c / mb, env_start + c % mb); `rec` is the
    // r_obs slab, `state` the r_state slab [T][layers][n_all][256] whose stored
    // post-zero state is the layer's state input (nothing is written back);
    // every layer's gate pre-activations and output are written out for the
    // reverse pass.  tr_x[0] is filled through h_enc_out.
    int train;
    int tr_bf16;             // bf16-input kernel only: tr_pre / tr_x (tr_x[0] included) are bf16 arrays
    int tr_t0, tr_mb, tr_n_all, tr_env_start;
    float* tr_pre[CFP_MAX_LAYERS];   // [cols][768]: zh | zg | zp
    float* tr_x[CFP_MAX_LAYERS + 1]; // [cols][256]: tr_x[l+1] = output of layer l
};
int launch_forward(const FwdArgs& a, hipStream_t st);
int launch_forward_bf16(const FwdArgs& a, hipStream_t st);   // called by launch_forward
// 16-env tiles for small batches (opt-in per policy); called by launch_forward
bool forward_t16_ok(const FwdArgs& a);
int launch_forward_t16(const FwdArgs& a, hipStream_t st);
size_t t16_mirror_bytes(int layers);
void t16_mirror_layout(void* base, int layers, const u4** enc_s, const f4** enc_t, const f4** gru,
                       const f4** av);
int launch_pack_weights_t16(const float* params, int layers, void* mirrors, hipStream_t st);
int launch_pack_weights_bf16(const float* params, int layers, int variant, uint16_t* we_bf,
                             uint16_t* wg_bf, uint16_t* wav_bf, hipStream_t st);

int launch_pack_enc_split(const float* params, int layers, int variant, uint16_t* we_s3,
                          hipStream_t st);
int launch_pack_weights(const float* params, int layers, int variant, float* we_pk,
                        float* wg_pk, float* wav_pk, hipStream_t st);

// Library-internal forms of the dense-math seam with explicit leading dimensions
// (the trainer keeps its feature matrix 848 floats wide so that rows stay
// 16-byte aligned); the C ABI entry points call these with the tight widths.
int launch_expand_obs(const uint8_t* r_obs, float* xobs, int t0, int count, int mb, int n,
                      int env_start, int ld, hipStream_t st);
int gemm_enc_fwd_ld(int cols, const float* W_enc, const float* xobs, int ldx, float* h,
                    hipStream_t st);
// Scratch memory of the seam's kernels: the split mirror of W that k_dh_x9 reads, the
// split-K partial sums of a dW GEMM, the slice sums of the value-head gemv.  One user
// at a time: calls that share a SeamWork must be ordered (one stream, or events).
// A trainer owns its own; the raw C entry points share the process-wide one.
struct SeamWork {
    u4* w_mirror = nullptr;
    float* dw_part = nullptr;
    size_t dw_part_floats = 0;
    float* gemv_part = nullptr;
};
int seam_work_create(SeamWork* w);
void seam_work_destroy(SeamWork* w);
// process-wide workspace of the raw C entry points: made by cfp_seam_reserve() or by the
// first call that needs it; null (error set) when the allocation fails
const SeamWork* seam_default();

int gemm_dh_acc(int m3, int cols, const float* W, const float* dpre, float* dh, bool accumulate,
                const SeamWork& sw, hipStream_t st);
int gemm_dw_ld(int rows, int cols, const float* x, const float* dpre, int ld_dpre, float* dW,
               const SeamWork& sw, hipStream_t st);

// the fixed-order fold dst[i] += sum_z part[z*stride + i] of split-K partial sums
int launch_splitk_reduce(float* dst, const float* part, long count, long stride, int splits,
                         hipStream_t st);
// dW_enc[843][256] += features^T dh over the window columns, read from the records
// (bf16 MFMA on the map bytes); needs envs per minibatch % 8 == 0.  tail_scratch:
// cols * 76 floats.  dh_bf16: dh holds bf16 (one-product mode only).  sw_tail / st_tail:
// workspace and stream for the GEMM of the last 75 features (both must be ordered behind
// dh; default: the same as the first 768).
bool dw_enc_records_ok(int mb);
int dw_enc_records(const uint8_t* r_obs, const float* dh, float* dW, float* tail_scratch, int t0,
                   int cols, int mb, int n_all, int env_start, const SeamWork& sw, hipStream_t st,
                   bool dh_bf16 = false, const SeamWork* sw_tail = nullptr,
                   hipStream_t st_tail = nullptr);

// dW[rows][256] += dpre^T x with both fp32 operands split into bf16 triples
// (cols % 8 == 0)
bool gemm_dw_x9_ok(int rows, int cols);
int gemm_dw_x9(int rows, int cols, const float* x, const float* dpre, int ld_dpre, float* dW,
               int terms, const SeamWork& sw, hipStream_t st, int rows_first = 0,
               float* dW_rest = nullptr, bool dpre_bf16 = false, bool x_bf16 = false);
// partial products per product the split kernels run with now (9, 6, or 1 with bf16
// inputs); 0 when they are switched off
int gemm_split_terms();
// h[cols][256] = xobs[cols][843] . W_enc on the split kernels (no bias); the mirror is
// enc_mirror_bytes() of device memory owned by the caller
size_t enc_mirror_bytes();
bool gemm_enc_fwd_x9_ok(int cols, const float* xobs);
int gemm_enc_fwd_x9(int cols, const float* W_enc, const float* xobs, int ldx, float* h, int terms,
                    u4* enc_mirror, hipStream_t st);
// The GEMM mode in effect for the calling thread: the process-wide switches
// (cfp_set_gemm_bf16 / cfp_set_gemm_split) unless a GemmModeScope overrides them.
int gemm_mode_bf16();
int gemm_mode_split();
// Overrides the mode for the calls the current thread issues while the object lives;
// a negative value leaves that switch as it is.
struct GemmModeScope {
    GemmModeScope(int bf16, int split);
    ~GemmModeScope();
    GemmModeScope(const GemmModeScope&) = delete;
    GemmModeScope& operator=(const GemmModeScope&) = delete;
    int old_bf16, old_split;
};
// dW_a[rows_a][256] += and dW_b[rows_b][256] += from adjacent columns of one dpre matrix
// (one pass over x on the split kernels, two passes otherwise)
int gemm_dw_two(int rows_a, int rows_b, int cols, const float* x, const float* dpre, int ld_dpre,
                float* dW_a, float* dW_b, const SeamWork& sw, hipStream_t st);

// dh[cols][256] (+)= dpre[cols][m3] . W[m3][256], same splitting (m3 % 16 == 0,
// cols % 32 == 0, dpre 16-byte aligned); dpre_bf16 / dh_bf16: that array holds bf16
// (one-product mode only)
bool gemm_dh_x9_ok(int m3, int cols, const float* dpre);
int gemm_dh_x9(int m3, int cols, const float* W, const float* dpre, float* dh, bool accumulate,
               int terms, u4* w_mirror, hipStream_t st, bool dpre_bf16 = false,
               bool dh_bf16 = false);
size_t dh_mirror_bytes();   // size of the split mirror of W (K up to 768)

// y[cols][m] = x[cols][k] . W[m][k]^T on the same kernel (m % 256 == 0, k % 16 == 0,
// cols % 32 == 0, x 16-byte aligned)
bool gemm_fwd_x9_ok(int m, int cols, int k, const float* x);
int gemm_fwd_x9(int m, int cols, int k, const float* W, const float* x, float* y, int terms,
                u4* w_mirror, hipStream_t st);

// per-variant arena geometry
struct Arena {
    int obs, actions;
    size_t w_enc, b_enc, w_gru, w_a, b_a, w_v, b_v, count;
};
inline Arena arena_of(int variant, int layers) {
    Arena a;
    a.obs = variant ? CFP_CLASSIC_OBS : CFP_OBS;
    a.actions = variant ? CFP_CLASSIC_ACTIONS : CFP_ACTIONS;
    a.w_enc = 0;
    a.b_enc = (size_t)a.obs * CFP_HIDDEN;
    a.w_gru = a.b_enc + CFP_HIDDEN;
    a.w_a = a.w_gru + (size_t)layers * CFP_GRU * CFP_HIDDEN;
    a.b_a = a.w_a + (size_t)a.actions * CFP_HIDDEN;
    a.w_v = a.b_a + a.actions;
    a.b_v = a.w_v + CFP_HIDDEN;
    a.count = a.b_v + 1;
    return a;
}

}  // namespace cfp
