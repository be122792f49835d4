// Fused policy forward for gfx950: 996-byte records -> Linear(843->256)
// -> MinGRU x L -> actor(43)/value(1), one workgroup per tile of 32 envs.
//
// Replaces, in one launch, the reference's per-step chain
//   k_expand_obs + cublasSgemm + k_add_bias       (craftax_full.cu:11954-11962)
//   L x { cublasSgemm(768 x cn x 256) + k_mingru_epi_fwd }   (:11988-12008)
//   cublasSgemm(44 x n x 256) + bias adds of k_value_sample  (:12044, :9726)
// so neither the fp32 feature matrix nor the [768][chunk] gate
// pre-activations ever exist in HBM: the activations of a tile stay in LDS
// from the record bytes to the logits.
//
// Data flow of one workgroup (256 threads = 4 waves, wave w owns hidden units
// [64w, 64w+64)):
//   records (31 872 contiguous bytes) -> LDS, rows re-strided to 255 dwords
//   encoder: C[env][unit] += x[env][f] * W_enc[f][unit] on 32x32x2 fp32 MFMA,
//            x taken from the LDS bytes (v_cvt_f32_ubyteN) / tail floats,
//            W_enc fragments streamed from the MFMA-ordered mirror in L2
//   h = C + b_enc -> LDS x tile [32][260] fp32 (aliases the record bytes)
//   per layer: 6 accumulators (zh, zg, zp for 2 unit tiles) over K = 256,
//            gate/blend epilogue in registers, state streamed from/to HBM
//            with non-temporal accesses, h' written back into the x tile
//   heads:   2 row tiles x 2 K halves over the 4 waves, reduced through LDS.
//
// MFMA operand convention (v_mfma_f32_32x32x2_f32): A = activations
// (row = env), B = weights (column = unit), so accumulator register r of lane
// l holds env 8*(r/4) + 4*(l/32) + r%4, unit l%32: a half-wave touches 32
// consecutive units of one env, i.e. one full 128-byte line of state.
#include "cfp_common.h"

namespace cfp {

namespace {

constexpr int XS = 260;   // floats per env row of the LDS x tile (256 + 4 pad)
constexpr int XS4 = XS / 4;
constexpr int RS = 255;   // dwords per record row in LDS: 249 data + 6 zero
constexpr int REC_DW = CFP_REC_BYTES / 4;             // 249
constexpr int TILE_REC_V4 = kTileEnvs * REC_DW / 4;   // 1992 16-byte chunks
constexpr int LDS_FLOATS = kTileEnvs * XS;            // 8320 >= 32*255

__device__ __forceinline__ float sigmoid_fast(float z) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-z));
}

__device__ __forceinline__ f16v mfma(float a, float b, f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ f16v zero16() {
    f16v z;
#pragma unroll
    for (int i = 0; i < 16; i++) z[i] = 0.0f;
    return z;
}

// Accumulator register r of a lane in half-wave h holds env row
// acc_row(r) + 4*h of the 32-env tile.
__device__ __forceinline__ constexpr int acc_row(int r) {
    return 8 * (r >> 2) + (r & 3);
}

// LDS x tile [32][XS] -> dense [32][256] in HBM, 16 bytes per thread per step.
__device__ __forceinline__ void copy_tile_out(const float* lds, float* dst,
                                              int tid) {
    const f4* xs4 = reinterpret_cast<const f4*>(lds);
    f4* d4 = reinterpret_cast<f4*>(dst);
#pragma unroll
    for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads)
        d4[i] = xs4[(i >> 6) * XS4 + (i & 63)];
}

// Classic-game encoder (encode_obs_kernel, craftax_classic.cu:1714-1751): the
// observation is one-hot per view cell, so h0 is b_enc plus a sum of W_enc
// rows selected by the record bytes, in feature order.  Thread k owns hidden
// unit k and walks the tile's 32 envs; the record bytes are LDS broadcasts and
// every W_enc row read is one coalesced 1 KiB line set from L2.
__device__ __forceinline__ void classic_encode_tile(const FwdArgs& a, uint8_t* crec,
                                                    float* lds, size_t e0, int tid) {
    constexpr int CELLS = 63, CH = 21, NBLK = 17;
    constexpr int TILE_V4 = kTileEnvs * CFP_CLASSIC_REC_BYTES / 16;   // 296
    const u4* src = reinterpret_cast<const u4*>(a.rec + e0 * CFP_CLASSIC_REC_BYTES);
    u4* dst = reinterpret_cast<u4*>(crec);
    for (int i = tid; i < TILE_V4; i += kFwdThreads) dst[i] = src[i];
    __syncthreads();
    const float* W = a.w_enc + tid;
    const float bias = a.b_enc[tid];
    for (int e = 0; e < kTileEnvs; e++) {
        const uint8_t* o = crec + e * CFP_CLASSIC_REC_BYTES;
        float hv = bias;
        for (int cell = 0; cell < CELLS; cell++) {
            hv += W[(size_t)(cell * CH + (int8_t)o[cell]) * CFP_HIDDEN];
            const uint32_t m = o[CELLS + cell];
            if (m) {
                const float* wm = W + (size_t)(cell * CH + NBLK) * CFP_HIDDEN;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (m & (1u << j)) hv += wm[(size_t)j * CFP_HIDDEN];
            }
        }
        int f = CELLS * CH;
#pragma unroll
        for (int j = 0; j < 16; j++, f++)
            hv = fmaf((float)(int8_t)o[2 * CELLS + j] / 10.0f, W[(size_t)f * CFP_HIDDEN], hv);
        const int dir = (int8_t)o[2 * CELLS + 16];
#pragma unroll
        for (int d = 1; d <= 4; d++, f++)
            hv = fmaf(dir == d ? 1.0f : 0.0f, W[(size_t)f * CFP_HIDDEN], hv);
        const float sleeping = o[2 * CELLS + 17] ? 1.0f : 0.0f;
        const float light = *reinterpret_cast<const float*>(o + 2 * CELLS + 18);
        hv = fmaf(light, W[(size_t)f * CFP_HIDDEN], hv); f++;
        hv = fmaf(sleeping, W[(size_t)f * CFP_HIDDEN], hv);
        lds[e * XS + tid] = hv;
    }
}

}  // namespace

__global__ __launch_bounds__(kFwdThreads, 2) void k_policy_forward(FwdArgs a) {
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    __shared__ float term_s[kTileEnvs];
    __shared__ __attribute__((aligned(16))) uint8_t crec[kTileEnvs * CFP_CLASSIC_REC_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const size_t e0 = (size_t)blockIdx.x * kTileEnvs;

    if (tid < kTileEnvs)
        term_s[tid] = a.terminals ? a.terminals[e0 + tid] : 0.0f;

    if (a.rec && a.variant == 1) {
        classic_encode_tile(a, crec, lds, e0, tid);
        __syncthreads();
        if (a.h_enc_out) copy_tile_out(lds, a.h_enc_out + e0 * CFP_HIDDEN, tid);
    } else if (a.rec) {
        // ---- stage the tile's records: contiguous 16-byte loads, rows
        // re-strided to an odd dword count so that 32 envs reading the same
        // feature hit 32 different LDS banks.
        uint32_t* rs = reinterpret_cast<uint32_t*>(lds);
        const u4* src =
            reinterpret_cast<const u4*>(a.rec + e0 * CFP_REC_BYTES);
        for (int i = tid; i < TILE_REC_V4; i += kFwdThreads) {
            u4 v = __builtin_nontemporal_load(src + i);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                int d = 4 * i + c;
                int row = d / REC_DW;
                int col = d - row * REC_DW;
                rs[row * RS + col] = w[c];
            }
        }
        if (tid < kTileEnvs * (RS - REC_DW)) {
            int row = tid / (RS - REC_DW);
            int c = tid - row * (RS - REC_DW);
            rs[row * RS + REC_DW + c] = 0u;   // features 843..847 read as 0.0f
        }
        __syncthreads();

        // ---- encoder GEMM: K = 848 in 106 blocks of 8; 3 rotating weight
        // buffers, prefetch distance 2 blocks (the mirror is padded by 2).
        f16v acc0 = zero16(), acc1 = zero16();
        const f4* wp = a.we_pk + (size_t)(wave * 2) * 64 + lane;
        constexpr int KB_STRIDE = 4 * 2 * 64;   // f4 per K block
        const uint32_t* rrow = rs + l32 * RS;
        f4 bq[3][2];
        uint32_t wq[3];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            bq[s][0] = wp[(size_t)s * KB_STRIDE];
            bq[s][1] = wp[(size_t)s * KB_STRIDE + 64];
        }
        wq[0] = rrow[half];
        // The scheduling barriers pin the prefetches ahead of the MFMA block
        // that hides them; without them the compiler sinks each load to just
        // before its use and the L2 latency lands on the matrix pipe.
#pragma unroll 1
        for (int kb0 = 0; kb0 < kKbMap; kb0 += 3) {
#pragma unroll
            for (int s = 0; s < 3; s++) {
                const int kb = kb0 + s;
                const int sp = (s + 2) % 3;
                bq[sp][0] = wp[(size_t)(kb + 2) * KB_STRIDE];
                bq[sp][1] = wp[(size_t)(kb + 2) * KB_STRIDE + 64];
                wq[(s + 1) % 3] = rrow[2 * (kb + 1) + half];
                __builtin_amdgcn_sched_barrier(0);
                const uint32_t w = wq[s];
                const float x0 = (float)(w & 0xffu);
                const float x1 = (float)((w >> 8) & 0xffu);
                const float x2 = (float)((w >> 16) & 0xffu);
                const float x3 = (float)(w >> 24);
                acc0 = mfma(x0, bq[s][0].x, acc0);
                acc1 = mfma(x0, bq[s][1].x, acc1);
                acc0 = mfma(x1, bq[s][0].y, acc0);
                acc1 = mfma(x1, bq[s][1].y, acc1);
                acc0 = mfma(x2, bq[s][0].z, acc0);
                acc1 = mfma(x2, bq[s][1].z, acc1);
                acc0 = mfma(x3, bq[s][0].w, acc0);
                acc1 = mfma(x3, bq[s][1].w, acc1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // tail floats: blocks 99..105 (buffer index stays kb % 3; 99 % 3 == 0)
        const float* frow = reinterpret_cast<const float*>(rrow) +
                            (CFP_OBS_MAP / 4) + 4 * half;
#pragma unroll
        for (int kt = 0; kt < kKbEnc - kKbMap; kt++) {
            const int kb = kKbMap + kt;
            const int s = kt % 3;
            const int sp = (kt + 2) % 3;
            bq[sp][0] = wp[(size_t)(kb + 2) * KB_STRIDE];
            bq[sp][1] = wp[(size_t)(kb + 2) * KB_STRIDE + 64];
            const float x0 = frow[8 * kt + 0];
            const float x1 = frow[8 * kt + 1];
            const float x2 = frow[8 * kt + 2];
            const float x3 = frow[8 * kt + 3];
            acc0 = mfma(x0, bq[s][0].x, acc0);
            acc1 = mfma(x0, bq[s][1].x, acc1);
            acc0 = mfma(x1, bq[s][0].y, acc0);
            acc1 = mfma(x1, bq[s][1].y, acc1);
            acc0 = mfma(x2, bq[s][0].z, acc0);
            acc1 = mfma(x2, bq[s][1].z, acc1);
            acc0 = mfma(x3, bq[s][0].w, acc0);
            acc1 = mfma(x3, bq[s][1].w, acc1);
        }
        __syncthreads();   // every wave is done with the record bytes

        // ---- bias epilogue -> x tile (aliases the record bytes)
#pragma unroll
        for (int ut = 0; ut < 2; ut++) {
            const float bias = a.b_enc[wave * 64 + ut * 32 + l32];
            float* xrow = lds + (4 * half) * XS + wave * 64 + ut * 32 + l32;
            const f16v& acc = ut ? acc1 : acc0;
#pragma unroll
            for (int r = 0; r < 16; r++)
                xrow[acc_row(r) * XS] = acc[r] + bias;
        }
        __syncthreads();
        if (a.h_enc_out) copy_tile_out(lds, a.h_enc_out + e0 * CFP_HIDDEN, tid);
    } else {
        // layer-0 input given in HBM: stage [32][256] fp32 into the x tile
        const f4* src = reinterpret_cast<const f4*>(a.x0 + e0 * CFP_HIDDEN);
        f4* xs4 = reinterpret_cast<f4*>(lds);
        for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads) {
            int row = i >> 6, c4 = i & 63;
            xs4[row * XS4 + c4] = src[i];
        }
        __syncthreads();
    }

    const f4* xs4 = reinterpret_cast<const f4*>(lds);
    const int arow4 = l32 * XS4 + half;   // + 2*kb

    // ---- MinGRU layers --------------------------------------------------
    for (int l = 0; l < a.layers; l++) {
        constexpr int KB_STRIDE = 4 * 6 * 64;   // f4 per K block
        const f4* wp = a.wg_pk + (size_t)l * (kGruPackFloats / 4) +
                       (size_t)(wave * 6) * 64 + lane;
        f16v acc[6];
#pragma unroll
        for (int t = 0; t < 6; t++) acc[t] = zero16();
        f4 bA[6], bB[6], aA, aB;
#pragma unroll
        for (int t = 0; t < 6; t++) bA[t] = wp[t * 64];
        aA = xs4[arow4];
#pragma unroll 1
        for (int kb = 0; kb < kKbHid; kb += 2) {
#pragma unroll
            for (int t = 0; t < 6; t++)
                bB[t] = wp[(size_t)(kb + 1) * KB_STRIDE + t * 64];
            aB = xs4[arow4 + 2 * (kb + 1)];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int t = 0; t < 6; t++)
                    acc[t] = mfma(aA[j], bA[t][j], acc[t]);
            __builtin_amdgcn_sched_barrier(0);
            // kb + 2 == 32 prefetches the next layer's first weight block (or
            // the zero pad behind the last layer); the x index is clamped.
#pragma unroll
            for (int t = 0; t < 6; t++)
                bA[t] = wp[(size_t)(kb + 2) * KB_STRIDE + t * 64];
            aA = xs4[arow4 + 2 * (kb + 2 < kKbHid ? kb + 2 : kKbHid - 1)];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int t = 0; t < 6; t++)
                    acc[t] = mfma(aB[j], bB[t][j], acc[t]);
            __builtin_amdgcn_sched_barrier(0);
        }

        // State for this wave's 2 x 16 elements per lane, issued before the
        // barrier so the HBM latency overlaps the other waves' K loops.
        // Addresses are (uniform base + compile-time row offset)[lane offset]
        // so they live in SGPRs plus one VGPR.
        const int loff = (4 * half) * CFP_HIDDEN + wave * 64 + l32;
        float* st_base =
            a.state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN;
        float st[2][16];
#pragma unroll
        for (int ut = 0; ut < 2; ut++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                st[ut][r] = __builtin_nontemporal_load(
                    st_base + (acc_row(r) * CFP_HIDDEN + ut * 32) + loff);

        __syncthreads();   // all waves finished reading the x tile

#pragma unroll
        for (int ut = 0; ut < 2; ut++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (term_s[acc_row(r) + 4 * half] != 0.0f) st[ut][r] = 0.0f;
        if (a.r_state) {
            float* rs_base =
                a.r_state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN;
#pragma unroll
            for (int ut = 0; ut < 2; ut++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    __builtin_nontemporal_store(
                        st[ut][r],
                        rs_base + (acc_row(r) * CFP_HIDDEN + ut * 32) + loff);
        }
#pragma unroll
        for (int ut = 0; ut < 2; ut++) {
            float* xrow = lds + (4 * half) * XS + wave * 64 + ut * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float s = st[ut][r];
                const float zh = acc[0 + ut][r];
                const float zg = acc[2 + ut][r];
                const float zp = acc[4 + ut][r];
                const float sg = sigmoid_fast(zg);
                const float gh = zh >= 0.0f ? zh + 0.5f : sigmoid_fast(zh);
                const float out = s + sg * (gh - s);
                const float p = sigmoid_fast(zp);
                const float xv = xrow[acc_row(r) * XS];
                xrow[acc_row(r) * XS] = p * out + (1.0f - p) * xv;
                __builtin_nontemporal_store(
                    out, st_base + (acc_row(r) * CFP_HIDDEN + ut * 32) + loff);
            }
        }
        __syncthreads();
    }
    if (a.layers > 0 && a.h3_out)
        copy_tile_out(lds, a.h3_out + e0 * CFP_HIDDEN, tid);

    // ---- heads: wave = (row tile nt, K half kh) ---------------------------
    if (a.do_head) {
        const int nt = wave & 1;
        const int kh = wave >> 1;
        f16v acc = zero16();
        const f4* wp = a.wav_pk + (size_t)nt * 64 + lane;
#pragma unroll
        for (int i = 0; i < kKbHid / 2; i++) {
            const int kb = kh * (kKbHid / 2) + i;
            const f4 b = wp[(size_t)kb * 128];
            const f4 av = xs4[arow4 + 2 * kb];
#pragma unroll
            for (int j = 0; j < 4; j++) acc = mfma(av[j], b[j], acc);
        }
        __syncthreads();   // x tile dead; reuse LDS for the K-half reduction
        float* red = lds + (nt * 16) * 64 + lane;
        if (kh == 1) {
#pragma unroll
            for (int r = 0; r < 16; r++) red[r * 64] = acc[r];
        }
        __syncthreads();
        if (kh == 0) {
            const int arow = nt * 32 + l32;
            const int avs = a.actions + 1;     // 44, or 18 for the classic game
            if (arow < avs) {
                const float bias = arow < a.actions ? a.b_a[arow] : a.b_v[0];
                float* av_base = a.av_out + e0 * avs;
                const int aoff = (4 * half) * avs + arow;
#pragma unroll
                for (int r = 0; r < 16; r++)
                    (av_base + acc_row(r) * avs)[aoff] =
                        acc[r] + red[r * 64] + bias;
            }
        }
    }
}

int launch_forward(const FwdArgs& a, hipStream_t st) {
    CFP_REQUIRE(a.n > 0 && a.n % kTileEnvs == 0,
                "policy forward needs a positive env count that is a multiple "
                "of 32 (got %d)", a.n);
    CFP_REQUIRE((a.rec != nullptr) != (a.x0 != nullptr),
                "policy forward takes either records or a layer-0 input");
    CFP_REQUIRE(a.rec == nullptr ||
                    (reinterpret_cast<uintptr_t>(a.rec) & 15u) == 0,
                "record rows must start on a 16-byte boundary");
    CFP_REQUIRE(a.x0 == nullptr ||
                    (reinterpret_cast<uintptr_t>(a.x0) & 15u) == 0,
                "layer-0 input must be 16-byte aligned");
    CFP_REQUIRE(a.variant == 0 || a.rec == nullptr || a.w_enc != nullptr,
                "classic forward needs the unpacked W_enc");
    CFP_REQUIRE(a.actions > 0 && a.actions < kAvPad, "bad action count %d", a.actions);
    CFP_REQUIRE(a.layers >= 0 && a.layers <= CFP_MAX_LAYERS,
                "layers must be in 0..%d", CFP_MAX_LAYERS);
    CFP_REQUIRE(a.layers == 0 || a.state != nullptr,
                "MinGRU layers need a state buffer");
    CFP_REQUIRE(!a.do_head || a.av_out != nullptr,
                "head requested without an output buffer");
    hipLaunchKernelGGL(k_policy_forward, dim3(a.n / kTileEnvs),
                       dim3(kFwdThreads), 0, st, a);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

// ---- MFMA-ordered weight mirrors --------------------------------------------
// Each 16-byte element feeds one lane for one K block: lane l carries
// k = 8*kb + 4*(l/32) + j, column l%32 of its 32-wide tile, so a wave's
// fragment load is one contiguous 1 KiB read.
__global__ void k_pack_enc(const float* __restrict__ W_enc,
                           float* __restrict__ out, int total) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int j = idx & 3, lane = (idx >> 2) & 63, ut = (idx >> 8) & 1,
        wave = (idx >> 9) & 3, kb = idx >> 11;
    int unit = wave * 64 + ut * 32 + (lane & 31);
    int f = kKBlock * kb + 4 * (lane >> 5) + j;
    out[idx] = f < CFP_OBS ? W_enc[(size_t)f * CFP_HIDDEN + unit] : 0.0f;
}

__global__ void k_pack_gru(const float* __restrict__ W_gru,
                           float* __restrict__ out, int layers, int total) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int layer = idx / (int)kGruPackFloats;
    if (layer >= layers) { out[idx] = 0.0f; return; }   // prefetch pad
    int i = idx - layer * (int)kGruPackFloats;
    int j = i & 3, lane = (i >> 2) & 63, q = i >> 8;
    int t = q % 6, wave = (q / 6) & 3, kb = q / 24;
    int gate = t >> 1, ut = t & 1;
    int row = gate * CFP_HIDDEN + wave * 64 + ut * 32 + (lane & 31);
    int k = kKBlock * kb + 4 * (lane >> 5) + j;
    out[idx] = W_gru[(size_t)layer * kGruPackFloats + (size_t)row * CFP_HIDDEN + k];
}

__global__ void k_pack_av(const float* __restrict__ W_a,
                          const float* __restrict__ W_v,
                          float* __restrict__ out, int actions) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int)kAvPackFloats) return;
    int j = idx & 3, lane = (idx >> 2) & 63, nt = (idx >> 8) & 1, kb = idx >> 9;
    int arow = nt * 32 + (lane & 31);
    int k = kKBlock * kb + 4 * (lane >> 5) + j;
    float v = 0.0f;
    if (arow < actions) v = W_a[arow * CFP_HIDDEN + k];
    else if (arow == actions) v = W_v[k];
    out[idx] = v;
}

int launch_pack_weights(const float* params, int layers, int variant, float* we_pk,
                        float* wg_pk, float* wav_pk, hipStream_t st) {
    const Arena ar = arena_of(variant, layers);
    if (variant == 0) {   // the classic encoder gathers from the unpacked W_enc
        const int enc_total = (kKbEnc + 2) * 2048;
        hipLaunchKernelGGL(k_pack_enc, dim3((enc_total + 255) / 256), dim3(256), 0,
                           st, params + ar.w_enc, we_pk, enc_total);
    }
    const int gru_total = layers * (int)kGruPackFloats + 4 * 6 * 64 * 4;
    hipLaunchKernelGGL(k_pack_gru, dim3((gru_total + 255) / 256), dim3(256), 0,
                       st, params + ar.w_gru, wg_pk, layers, gru_total);
    hipLaunchKernelGGL(k_pack_av, dim3(((int)kAvPackFloats + 255) / 256),
                       dim3(256), 0, st, params + ar.w_a, params + ar.w_v, wav_pk,
                       ar.actions);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace cfp
