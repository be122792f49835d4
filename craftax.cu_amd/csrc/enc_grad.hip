// Encoder weight gradient of the PPO update, taken straight from the recorded
// observation records:  dW_enc[f][u] += sum_c feature_f(c) * dh_enc[c][u]  over the
// window columns c.  The reference expands the records into a dense fp32 feature
// matrix (k_expand_obs, craftax_full.cu:10022-10031) and calls
// cu_gemm_dw(CF_NN_OBS, cols, dh, xobs) on it (craftax_full.cu:13324).
//
// Here the 768 leading map bytes never become floats in memory.  A byte is exact in
// bf16, and an fp32 gradient is exactly the sum of three bf16 numbers (8 + 8 + 8
// significand bits), so byte * gradient is three bf16 MFMA products accumulated in
// fp32: the same sum of exact fp32 products that the fp32 MFMA adds up, at 3/16 of its
// cost, and the operand read per column is 768 bytes instead of 3 KiB.
//   grid      : 3 feature groups (256 map bytes each) x S splits of the columns; the
//               three groups of a split run on one XCD so that dh is fetched from HBM
//               once and shared through that L2
//   workgroup : 8 waves; wave w owns units 32w..32w+31 and all 8 row blocks of the
//               group: 8 accumulators of v_mfma_f32_32x32x16_bf16
//   K loop    : 64 columns per iteration (4 MFMA K steps of 16).  The record side is
//               shared through LDS: each wave fetches the dwords of one (K step,
//               128-byte span) -- 4 features x 8 columns per lane -- turns them into
//               four ready MFMA fragments (feature 4i+c of the span is row i of
//               fragment c) and all waves read them back, one 16-byte read per
//               fragment.  The gradient side is private to the wave: 8 loads of 4
//               bytes per lane and K step (each a coalesced 128-byte row piece),
//               split into hi/mid/lo by masking.
//   output    : partial sums per split, folded in ascending split order by
//               k_splitk_reduce (run-to-run bitwise stable).
// The last map bytes (768..791) and the 51 fp32 features go through the fp32 GEMM as
// a 75-row operand (k_expand_obs_tail + gemm_dw_ld).
#include "policy_tile.h"
#include "ppo_kernels.h"

namespace cfp {
namespace {

constexpr int kEgThreads = 512;
constexpr int kEgGroups = 3;               // feature groups of 256 map bytes
constexpr int kEgBlocks = 8;               // 32-row MFMA blocks per group
constexpr int kEgIterCols = 64;            // columns per iteration
constexpr int kEgFeat = kEgGroups * 256;   // 768 features on the bf16 path
constexpr int kEgTail = CFP_OBS - kEgFeat; // 75 features on the fp32 path
constexpr int kEgTailLd = 76;
constexpr int kEgXcds = 8;
constexpr int kRecDw = CFP_REC_BYTES / 4;  // 249

// bf16 pair {byte c of a (low half), byte c of b (high half)}
template <int C>
__device__ __forceinline__ uint32_t byte_pair_bf16(uint32_t a, uint32_t b) {
    const float lo = (float)((a >> (8 * C)) & 0xffu);
    const float hi = (float)((b >> (8 * C)) & 0xffu);
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}
template <int C>
__device__ __forceinline__ u4 byte_frag(const uint32_t (&d)[8]) {
    u4 f;
    f.x = byte_pair_bf16<C>(d[0], d[1]);
    f.y = byte_pair_bf16<C>(d[2], d[3]);
    f.z = byte_pair_bf16<C>(d[4], d[5]);
    f.w = byte_pair_bf16<C>(d[6], d[7]);
    return f;
}

// ONE: the bf16-input mode of the seam: the gradient is rounded to bf16 (nearest even), one
// product per byte.  D16: dh is a bf16 array (the update's bf16 storage), which implies ONE.
template <bool D16, bool ONE>
__global__ __launch_bounds__(kEgThreads) void k_dw_enc_bytes(
    const uint8_t* __restrict__ r_obs, const float* __restrict__ dh, float* __restrict__ part,
    int t0, int cols, int mb, int n_all, int env_start, int iters_per_split, int n_wg) {
    __shared__ u4 stage[2][4][kEgBlocks][64];   // 64 KiB: [buffer][K step][fragment][lane]
    const int xcd = (int)(blockIdx.x % kEgXcds), q = (int)(blockIdx.x / kEgXcds);
    const int lin = xcd * (int)(gridDim.x / kEgXcds) + q;
    if (lin >= n_wg) return;
    const int split = lin / kEgGroups, gi = lin - split * kEgGroups;
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int total_iters = (cols + kEgIterCols - 1) / kEgIterCols;
    const int it0 = split * iters_per_split;
    const int it1 = min(total_iters, it0 + iters_per_split);
    const int pks = w >> 1, psb = w & 1;   // the (K step, 128-byte span) this wave stages

    // columns cg..cg+7 of a lane share their time step: minibatches are multiples of 8
    // envs.  The loop body is branch free: loads past the last column are redirected
    // to the last 8 columns, and the record side of such columns is zeroed, which
    // makes their products zero whatever the gradient side holds.
    auto rec_load = [&](int it, uint32_t (&d)[8]) {
        const int cg = it * kEgIterCols + pks * 16 + 8 * g;
        const int cc = min(cg, cols - 8);
        const unsigned trw = (unsigned)cc / (unsigned)mb;
        const unsigned el = (unsigned)cc - trw * (unsigned)mb;
        const uint32_t* p = reinterpret_cast<const uint32_t*>(
            r_obs + (((size_t)t0 + trw) * (size_t)n_all + env_start + el) * CFP_REC_BYTES +
            gi * 256 + psb * 128 + 4 * n);
#pragma unroll
        for (int j = 0; j < 8; j++) d[j] = __builtin_nontemporal_load(p + j * kRecDw);
    };
    auto rec_store = [&](int it, int buf, const uint32_t (&d)[8]) {
        const bool in = it * kEgIterCols + pks * 16 + 8 * g < cols;
        uint32_t e[8];
#pragma unroll
        for (int j = 0; j < 8; j++) e[j] = in ? d[j] : 0u;
        stage[buf][pks][psb * 4 + 0][lane] = byte_frag<0>(e);
        stage[buf][pks][psb * 4 + 1][lane] = byte_frag<1>(e);
        stage[buf][pks][psb * 4 + 2][lane] = byte_frag<2>(e);
        stage[buf][pks][psb * 4 + 3][lane] = byte_frag<3>(e);
    };
    const float* dh_lane = dh + 32 * w + n;
    const uint16_t* dh16_lane = reinterpret_cast<const uint16_t*>(dh) + 32 * w + n;
    auto dh_load = [&](int it, int ks, float (&v)[8]) {
        const int cc = min(it * kEgIterCols + ks * 16 + 8 * g, cols - 8);
        if (D16) {
            const uint16_t* p = dh16_lane + (size_t)cc * CFP_HIDDEN;
#pragma unroll
            for (int j = 0; j < 8; j++)
                v[j] = __uint_as_float((uint32_t)p[j * CFP_HIDDEN] << 16);
            return;
        }
        const float* p = dh_lane + (size_t)cc * CFP_HIDDEN;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = p[j * CFP_HIDDEN];
    };
    // hi / mid / lo parts of eight gradients; bf16 values are their own hi part
    auto dh_parts = [&](const float (&v)[8], u4& h, u4& m, u4& l) {
        if (ONE) {
            h = round_bf16x8(v);
            m = h;
            l = h;
        } else {
            split3(v, h, m, l);
        }
    };

    f16v acc[kEgBlocks];
#pragma unroll
    for (int b = 0; b < kEgBlocks; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = 0.0f;

    if (it0 < it1) {
        // Software pipeline.  Gradient rows are requested three K steps ahead of their
        // MFMAs and split one K step ahead; record fragments come out of LDS one pair
        // ahead; the next iteration's records are requested at the top of the
        // iteration and staged into the other buffer during its last K step.  The
        // barrier sits after this wave's last read of the current buffer has
        // returned, so a buffer is never written while another wave still reads it.
        uint32_t d[8];
        float raw[4][8];
        rec_load(it0, d);
        rec_store(it0, 0, d);
        dh_load(it0, 0, raw[0]);
        dh_load(it0, 1, raw[1]);
        dh_load(it0, 2, raw[2]);
        __syncthreads();
        u4 a[2][2];
        a[0][0] = stage[0][0][0][lane];
        a[0][1] = stage[0][0][1][lane];
        u4 bh, bm, bl;
        dh_parts(raw[0], bh, bm, bl);
        for (int it = it0; it < it1; it++) {
            const int buf = (it - it0) & 1;
            const int itn = min(it + 1, it1 - 1);
            rec_load(itn, d);
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                if (ks < 1) dh_load(it, ks + 3, raw[ks + 3]);
                else dh_load(itn, ks - 1, raw[ks - 1]);
                u4 nh, nm, nl;
                dh_parts(raw[(ks + 1) & 3], nh, nm, nl);
#pragma unroll
                for (int pr = 0; pr < 4; pr++) {
                    const int cur = pr & 1, nxt = cur ^ 1;
                    if (pr < 3) {
                        a[nxt][0] = stage[buf][ks][2 * pr + 2][lane];
                        a[nxt][1] = stage[buf][ks][2 * pr + 3][lane];
                    } else if (ks < 3) {
                        a[nxt][0] = stage[buf][ks + 1][0][lane];
                        a[nxt][1] = stage[buf][ks + 1][1][lane];
                    } else {
                        rec_store(itn, buf ^ 1, d);
                        __syncthreads();
                        a[nxt][0] = stage[buf ^ 1][0][0][lane];
                        a[nxt][1] = stage[buf ^ 1][0][1][lane];
                    }
                    const int b = 2 * pr;
                    acc[b] = mfma16(a[cur][0], bh, acc[b]);
                    acc[b + 1] = mfma16(a[cur][1], bh, acc[b + 1]);
                    if (!ONE) {
                        acc[b] = mfma16(a[cur][0], bm, acc[b]);
                        acc[b + 1] = mfma16(a[cur][1], bm, acc[b + 1]);
                        acc[b] = mfma16(a[cur][0], bl, acc[b]);
                        acc[b + 1] = mfma16(a[cur][1], bl, acc[b + 1]);
                    }
                }
                bh = nh; bm = nm; bl = nl;
            }
        }
    }
    // accumulator register r of fragment c of span sb: feature sb*128 + 4*row + c
    float* o = part + ((size_t)split * kEgFeat + gi * 256) * CFP_HIDDEN + 32 * w + n;
#pragma unroll
    for (int b = 0; b < kEgBlocks; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = acc_row(r) + 4 * g;
            o[(size_t)((b >> 2) * 128 + 4 * row + (b & 3)) * CFP_HIDDEN] = acc[b][r];
        }
}

// Features 768..842 of the window columns as an fp32 matrix [cols][76]: 24 map bytes,
// then the record's 51 floats; thread = one 16-byte piece.
__global__ void k_expand_obs_tail(const uint8_t* __restrict__ r_obs, f4* __restrict__ out,
                                  int t0, size_t total4, int mb, int n_all, int env_start) {
    static_assert((CFP_OBS_MAP - kEgFeat) % 4 == 0 && kEgTailLd % 4 == 0, "whole dwords");
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total4) return;
    constexpr int LD4 = kEgTailLd / 4, MAP4 = (CFP_OBS_MAP - kEgFeat) / 4;   // 19, 6
    const unsigned c = (unsigned)(idx / LD4);
    const int q = (int)(idx - (size_t)c * LD4);
    const unsigned trw = c / (unsigned)mb, el = c - trw * (unsigned)mb;
    const uint32_t* rec = reinterpret_cast<const uint32_t*>(
        r_obs + (((size_t)t0 + trw) * (size_t)n_all + env_start + el) * CFP_REC_BYTES);
    f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (q < MAP4) {
        const uint32_t b = rec[kEgFeat / 4 + q];
        v[0] = (float)(b & 0xffu);
        v[1] = (float)((b >> 8) & 0xffu);
        v[2] = (float)((b >> 16) & 0xffu);
        v[3] = (float)(b >> 24);
    } else {
        const int f = 4 * (q - MAP4);
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (f + j < CFP_OBS - CFP_OBS_MAP) v[j] = __uint_as_float(rec[CFP_OBS_MAP / 4 + f + j]);
    }
    out[idx] = v;
}

}  // namespace

bool dw_enc_records_ok(int mb) { return mb > 0 && mb % 8 == 0; }

int dw_enc_tail_expand(const uint8_t* r_obs, float* tail_scratch, int t0, int cols, int mb, int n_all,
                       int env_start, hipStream_t st) {
    CFP_REQUIRE(r_obs && tail_scratch && cols > 0 && dw_enc_records_ok(mb), "dw_enc_tail_expand: bad argument");
    const size_t total4 = (size_t)cols * (kEgTailLd / 4);
    hipLaunchKernelGGL(k_expand_obs_tail, dim3((unsigned)((total4 + 255) / 256)), dim3(256), 0, st, r_obs,
                       reinterpret_cast<f4*>(tail_scratch), t0, total4, mb, n_all, env_start);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

static int dw_enc_records_impl(const uint8_t* r_obs, const float* dh, float* dW, float* tail_scratch, int t0,
                               int cols, int mb, int n_all, int env_start, const SeamWork& sw, hipStream_t st,
                               bool dh_bf16, const SeamWork* sw_tail, hipStream_t st_tail, bool tail_ready) {
    CFP_REQUIRE(r_obs && dh && dW && tail_scratch && cols > 0 && dw_enc_records_ok(mb) &&
                    cols % 8 == 0,
                "dw_enc_records: columns and envs per minibatch must be multiples of 8");
    float* work = sw.dw_part;
    const size_t work_floats = sw.dw_part_floats;
    CFP_REQUIRE(work, "dw_enc_records: no split workspace");
    const int total_iters = (cols + kEgIterCols - 1) / kEgIterCols;
    // one workgroup per CU: 85 splits x 3 groups
    int splits = 256 / kEgGroups;
    const int cap = (int)(work_floats / ((size_t)kEgFeat * CFP_HIDDEN));
    if (splits > cap) splits = cap;
    if (splits > total_iters) splits = total_iters;
    const int ips = (total_iters + splits - 1) / splits;
    splits = (total_iters + ips - 1) / ips;
    const int n_wg = splits * kEgGroups;
    const int grid = (n_wg + kEgXcds - 1) / kEgXcds * kEgXcds;
    if (dh_bf16)
        hipLaunchKernelGGL((k_dw_enc_bytes<true, true>), dim3(grid), dim3(kEgThreads), 0, st, r_obs, dh,
                           work, t0, cols, mb, n_all, env_start, ips, n_wg);
    else if (gemm_split_terms() == 1)   // bf16 GEMM inputs: like every other GEMM of that mode
        hipLaunchKernelGGL((k_dw_enc_bytes<false, true>), dim3(grid), dim3(kEgThreads), 0, st, r_obs,
                           dh, work, t0, cols, mb, n_all, env_start, ips, n_wg);
    else
        hipLaunchKernelGGL((k_dw_enc_bytes<false, false>), dim3(grid), dim3(kEgThreads), 0, st, r_obs,
                           dh, work, t0, cols, mb, n_all, env_start, ips, n_wg);
    const long count = (long)kEgFeat * CFP_HIDDEN;
    if (launch_splitk_reduce(dW, work, count, count, splits, st)) return 1;
    // rows 768..842: a GEMM of its own on other rows of dW, on the second stream and
    // workspace when the caller has one to spare
    const SeamWork& swt = sw_tail ? *sw_tail : sw;
    hipStream_t stt = sw_tail ? st_tail : st;
    if (!tail_ready && dw_enc_tail_expand(r_obs, tail_scratch, t0, cols, mb, n_all, env_start, stt)) return 1;
    if (dh_bf16)   // dh is the 256-wide operand of this GEMM, the 75 tail features its rows
        return gemm_dw_x9(kEgTail, cols, dh, tail_scratch, kEgTailLd, dW + count, 1, swt, stt, 0,
                          nullptr, false, true);
    return gemm_dw_ld(kEgTail, cols, dh, tail_scratch, kEgTailLd, dW + count, swt, stt);
}

int dw_enc_records(const uint8_t* r_obs, const float* dh, float* dW, float* tail_scratch, int t0,
                   int cols, int mb, int n_all, int env_start, const SeamWork& sw, hipStream_t st,
                   bool dh_bf16, const SeamWork* sw_tail, hipStream_t st_tail) {
    return dw_enc_records_impl(r_obs, dh, dW, tail_scratch, t0, cols, mb, n_all, env_start, sw, st, dh_bf16,
                               sw_tail, st_tail, false);
}
int dw_enc_records_tail_ready(const uint8_t* r_obs, const float* dh, float* dW, float* tail_scratch, int t0,
                              int cols, int mb, int n_all, int env_start, const SeamWork& sw, hipStream_t st,
                              bool dh_bf16, const SeamWork* sw_tail, hipStream_t st_tail) {
    return dw_enc_records_impl(r_obs, dh, dW, tail_scratch, t0, cols, mb, n_all, env_start, sw, st, dh_bf16,
                               sw_tail, st_tail, true);
}

}  // namespace cfp
