// bf16-input / fp32-accumulate variant of the fused policy forward for gfx950.
//
// Same interface and data flow as the fp32 kernel (records -> encoder -> MinGRU
// x L -> heads, one 32-env tile per workgroup, activations resident in LDS);
// the three GEMMs run on v_mfma_f32_32x32x16_bf16 with weights read from bf16
// mirrors and activations rounded to bf16 (round-to-nearest-even) as they are
// loaded into the A operand.  Everything else stays fp32: accumulators, biases,
// the gate/blend epilogue, the recurrent state and every output.  This is the
// counterpart of the reference's CF_GEMM_BF16 mode (craftax_full.cu:11306-11316,
// bf16 GEMM wrappers :11688-11756).  Its bf16 storage of activations exists for the
// window recompute of the update only (TR16: gate pre-activations and layer outputs
// leave as bf16, half the bytes of a kernel that is bound by its HBM writes there).
//
// At bf16 MFMA rates the matrix pipe is no longer the bound (a layer's gate GEMM
// is 96 MFMAs of 32 cycles per wave); the kernel is bound by the epilogue's
// vector instructions and the weight loads, so it runs two workgroups per CU
// (one tile each, no cross-tile software pipeline) and lets the hardware
// overlap one workgroup's epilogue with the other's GEMM.
//
// Operand layout of v_mfma_f32_32x32x16_bf16: lane l supplies row (A) / column
// (B) l%32 and the eight consecutive k = 8*(l/32) .. 8*(l/32)+7 of the 16-wide K
// block; the accumulator layout is that of the fp32 32x32 MFMA.
#include "policy_tile.h"

namespace cfp {

namespace {

typedef float f8 __attribute__((ext_vector_type(8)));

constexpr int kKb16Enc = kObsPad / 16;        // 53 K blocks of 16
constexpr int kKb16Map = CFP_OBS_MAP / 16;    // 49 all-map blocks; block 49 is half map, half tail
constexpr int kKb16Hid = CFP_HIDDEN / 16;     // 16

// eight fp32 -> eight bf16, round to nearest even
__device__ __forceinline__ u4 to_bf16x8(const f4& lo, const f4& hi) {
    f8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(u4, __builtin_convertvector(v, bf16x8));
}

__device__ __forceinline__ u4 floats_to_bf16x8(const float* p) {
    f4 lo = {p[0], p[1], p[2], p[3]}, hi = {p[4], p[5], p[6], p[7]};
    return to_bf16x8(lo, hi);
}

// A fragment of K block kb from an fp32 x tile: x[row][16kb + 8g .. +7]
__device__ __forceinline__ u4 a_frag(const f4* xs4, int l32, int g, int kb) {
    const f4* p = xs4 + l32 * XS4 + 4 * kb + 2 * g;
    return to_bf16x8(p[0], p[1]);
}

}  // namespace

// TRAIN: window recompute of the PPO update, as in the fp32 kernel: tile = 32 columns of
// one step of the slabs (records in r_obs, the stored post-zero state of every layer
// as the state input), every layer's gate pre-activations and output written out,
// nothing written back to the state.
// LDS x tile [32][XS] -> dense bf16 [32][256] in HBM, 8 bytes per thread per step.
__device__ __forceinline__ void copy_tile_out_bf16(const float* lds, uint16_t* dst, int tid) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
    const f4* xs4 = reinterpret_cast<const f4*>(lds);
    u2_t* d2 = reinterpret_cast<u2_t*>(dst);
    for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads)
        d2[i] = __builtin_bit_cast(u2_t, __builtin_convertvector(xs4[(i >> 6) * XS4 + (i & 63)], bf16x4_t));
}

// RS16: the recorded state is a bf16 slab -- written as bf16 by the rollout (HAS_RS), read as
// bf16 by the window recompute (TRAIN).
template <int VARIANT, bool HAS_RS, bool TRAIN, bool TR16 = false, bool RS16 = false>
__global__ __launch_bounds__(kFwdThreads, 2) void k_policy_forward_bf16(FwdArgs a) {
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    __shared__ float term_s[kTileEnvs];
    // classic game: the records and the encoder's tables sit in the x tile until the
    // encoder's result replaces them
    static_assert(ClsLayout<kTileEnvs>::end <= LDS_FLOATS * 4, "classic tables fit the x tile");
    uint8_t* const crec = reinterpret_cast<uint8_t*>(lds);

    const int tid = threadIdx.x;
    const unsigned lane_u = (unsigned)(tid & 63);
    const int g = (tid & 63) >> 5;       // k group of the A/B operand, env-row group of the accumulator
    const int l32 = tid & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned loff = (unsigned)((4 * g) * CFP_HIDDEN + l32);
    const unsigned loff3 = (unsigned)((4 * g) * CFP_GRU + l32);
    const size_t e0 = (size_t)blockIdx.x * kTileEnvs;
    const f4* xs4 = reinterpret_cast<const f4*>(lds);
    // first env of the tile as an index into the [T][n_all] slabs
    size_t se = e0;
    if (TRAIN) {
        const size_t tr = e0 / (size_t)a.tr_mb;
        se = ((size_t)a.tr_t0 + tr) * a.tr_n_all + a.tr_env_start + (e0 - tr * a.tr_mb);
    }

    stage_tile<VARIANT>(a, se, lds, crec, term_s, tid);
    __syncthreads();

    unsigned tmask = 0u;
#pragma unroll
    for (int r = 0; r < 16; r++)
        if (term_s[acc_row(r) + 4 * g] != 0.0f) tmask |= 1u << r;

    float st[32], stn[32];
    constexpr int kGateAhead = 2;   // K blocks of gate weights in flight
    u4 bq[kGateAhead + 1][6];
    auto state_fetch = [&](const float* base, float (&v)[32]) {
#pragma unroll
        for (int e = 0; e < 32; e++) {
            const int off = acc_row(e % 16) * CFP_HIDDEN + (e / 16) * 32;
            if (TRAIN && RS16)
                v[e] = (float)__builtin_nontemporal_load((reinterpret_cast<const __bf16*>(base) + off) + loff);
            else
                v[e] = __builtin_nontemporal_load((base + off) + loff);
        }
    };
    auto state_base = [&](int l) -> float* {
        if (TRAIN) {
            const size_t tt = se / a.tr_n_all, ee = se - tt * a.tr_n_all;
            const size_t el = ((tt * a.layers + l) * a.tr_n_all + ee) * CFP_HIDDEN + wave * 64;
            // a bf16 slab: the same element index in 2-byte elements (state_fetch casts back)
            if (RS16) return reinterpret_cast<float*>(reinterpret_cast<__bf16*>(a.state) + el);
            return a.state + el;
        }
        return a.state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN + wave * 64;
    };
    // layer 0's state is requested before the encoder and lands under it
    if (a.layers > 0) state_fetch(state_base(0), st);

    // ---- encoder ---------------------------------------------------------------
    if (VARIANT == 1 && a.rec) {
        // encode_obs_kernel (craftax_classic.cu:1714-1751).  Cell features: bits -> bf16
        // 0/1 through the table, against the hi and mid parts of the three-term split
        // of W_enc (16 significant bits of every weight: at least what rounding the
        // weight to bf16 keeps); the 22 scalar features on the fp32 MFMA.
        using LY = ClsLayout<kTileEnvs>;
        classic_prepare<kTileEnvs>(crec, tid);
        f16v acc[2] = {zero16(), zero16()};
        const uint8_t* brow = crec + LY::offBits + l32 * (kClsBitRow * 4) + g;
        const u4* lut = reinterpret_cast<const u4*>(crec + LY::offLut);
        const u4* wp = a.we_s3 + (size_t)(wave * 6) * 64;
        constexpr int KB_STRIDE = 4 * 6 * 64;   // u4 per K block: [wave][unit tile][part][lane]
        u4 b[2][4];
#pragma unroll
        for (int i = 0; i < 4; i++) b[0][i] = (wp + ((i >> 1) * 3 + (i & 1)) * 64)[lane_u];
        u4 av = lut[brow[0]];
#pragma unroll 2
        for (int kb = 0; kb < kClsKb16; kb++) {
            const int cb = kb & 1, nb = cb ^ 1;
            u4 an = av;
            if (kb + 1 < kClsKb16) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    b[nb][i] = (wp + (size_t)(kb + 1) * KB_STRIDE + ((i >> 1) * 3 + (i & 1)) * 64)[lane_u];
                an = lut[brow[2 * (kb + 1)]];
            }
            acc[0] = mfma16(av, b[cb][0], acc[0]);
            acc[1] = mfma16(av, b[cb][2], acc[1]);
            acc[0] = mfma16(av, b[cb][1], acc[0]);
            acc[1] = mfma16(av, b[cb][3], acc[1]);
            av = an;
        }
        const f4* wq = a.we_pk + (size_t)(wave * 2) * 64;
        constexpr int KB8_STRIDE = 4 * 2 * 64;
        const float* fx = reinterpret_cast<const float*>(crec + LY::offSv) + l32 * kClsSv + 4 * g;
#pragma unroll
        for (int t = 0; t < kClsTailKb; t++) {
            const f4 w0 = (wq + (size_t)t * KB8_STRIDE)[lane_u];
            const f4 w1 = (wq + (size_t)t * KB8_STRIDE + 64)[lane_u];
            const f4 x = *reinterpret_cast<const f4*>(fx + 8 * t);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc[0] = mfma(x[j], w0[j], acc[0]);
                acc[1] = mfma(x[j], w1[j], acc[1]);
            }
        }
        __syncthreads();   // every wave is done with the records and tables
#pragma unroll
        for (int ut = 0; ut < 2; ut++) {
            const float bias = a.b_enc[wave * 64 + ut * 32 + l32];
            float* xrow = lds + (4 * g) * XS + wave * 64 + ut * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) xrow[acc_row(r) * XS] = acc[ut][r] + bias;
        }
    } else if (VARIANT == 0 && a.rec) {
        f16v acc[2] = {zero16(), zero16()};
        const uint32_t* rrow = reinterpret_cast<const uint32_t*>(lds) + l32 * RS;
        const float* frow = reinterpret_cast<const float*>(rrow) + CFP_OBS_MAP / 4;
        const u4* wp = a.we_bf + (size_t)(wave * 2) * 64;
        constexpr int KB_STRIDE = 4 * 2 * 64;   // u4 per K block
        // weights of kEncAhead K blocks in flight: one block ahead the wave would sit out
        // an L2 round trip per block of two MFMAs
        constexpr int kEncAhead = 4;
        static_assert(kKb16Map - 1 == 12 * kEncAhead && kKb16Enc == kKb16Map + 4, "block schedule below");
        u4 bw[kEncAhead][2];
#pragma unroll
        for (int i = 0; i < kEncAhead; i++) {
            bw[i][0] = (wp + (size_t)i * KB_STRIDE)[lane_u];
            bw[i][1] = (wp + (size_t)i * KB_STRIDE + 64)[lane_u];
        }
        uint32_t w0 = rrow[2 * g], w1 = rrow[2 * g + 1];
#pragma unroll 1
        for (int kb0 = 0; kb0 < kKb16Map - 1; kb0 += kEncAhead) {
#pragma unroll
            for (int i = 0; i < kEncAhead; i++) {
                const int kb = kb0 + i;
                const uint32_t m0 = rrow[4 * (kb + 1) + 2 * g];
                const uint32_t m1 = rrow[4 * (kb + 1) + 2 * g + 1];
                const u4 av = bytes_to_bf16x8(w0, w1);
                acc[0] = mfma16(av, bw[i][0], acc[0]);
                acc[1] = mfma16(av, bw[i][1], acc[1]);
                bw[i][0] = (wp + (size_t)(kb + kEncAhead) * KB_STRIDE)[lane_u];     // <= block 51
                bw[i][1] = (wp + (size_t)(kb + kEncAhead) * KB_STRIDE + 64)[lane_u];
                w0 = m0; w1 = m1;
            }
        }
        // bw[0..3] now hold blocks 48..51.  Block 48: the last all-map block
        {
            const uint32_t m0 = rrow[4 * kKb16Map + 2 * g];       // g = 1 reads tail bits, which
            const uint32_t m1 = rrow[4 * kKb16Map + 2 * g + 1];   // block 49 replaces by floats
            const u4 av = bytes_to_bf16x8(w0, w1);
            acc[0] = mfma16(av, bw[0][0], acc[0]);
            acc[1] = mfma16(av, bw[0][1], acc[1]);
            bw[0][0] = (wp + (size_t)(kKb16Enc - 1) * KB_STRIDE)[lane_u];           // block 52
            bw[0][1] = (wp + (size_t)(kKb16Enc - 1) * KB_STRIDE + 64)[lane_u];
            w0 = m0; w1 = m1;
        }
        // block 49: features 784..791 are map bytes (g = 0), 792..799 tail floats (g = 1)
        {
            const u4 ab = bytes_to_bf16x8(w0, w1);
            const u4 af = floats_to_bf16x8(frow);
            const u4 av = g ? af : ab;
            acc[0] = mfma16(av, bw[1][0], acc[0]);
            acc[1] = mfma16(av, bw[1][1], acc[1]);
        }
        // blocks 50..52: tail floats 8 + 16(kb-50) + 8g .. ; features 843..847 read as 0
#pragma unroll
        for (int kb = kKb16Map + 1; kb < kKb16Enc; kb++) {
            const int slot = (kb - (kKb16Map - 1)) % kEncAhead;
            const u4 av = floats_to_bf16x8(frow + 16 * kb - CFP_OBS_MAP + 8 * g);
            acc[0] = mfma16(av, bw[slot][0], acc[0]);
            acc[1] = mfma16(av, bw[slot][1], acc[1]);
        }
        __syncthreads();   // every wave is done with the record bytes
#pragma unroll
        for (int ut = 0; ut < 2; ut++) {
            const float bias = a.b_enc[wave * 64 + ut * 32 + l32];
            float* xrow = lds + (4 * g) * XS + wave * 64 + ut * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) xrow[acc_row(r) * XS] = acc[ut][r] + bias;
        }
    }
    __syncthreads();
    if (a.rec && a.h_enc_out) {
        if (TR16)
            copy_tile_out_bf16(lds, reinterpret_cast<uint16_t*>(a.h_enc_out) + e0 * CFP_HIDDEN, tid);
        else
            copy_tile_out(lds, a.h_enc_out + e0 * CFP_HIDDEN, tid);
    }

    // ---- MinGRU layers ------------------------------------------------------------
    constexpr int KB_STRIDE = 4 * 6 * 64;   // u4 per K block of the gate mirror
#pragma unroll 1
    for (int l = 0; l < a.layers; l++) {
        float* st_base = a.state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN + wave * 64;
        if (TRAIN) {
            const size_t tt = se / a.tr_n_all, ee = se - tt * a.tr_n_all;
            st_base = a.state + ((tt * a.layers + l) * a.tr_n_all + ee) * CFP_HIDDEN + wave * 64;
        }
        // The state was requested one layer ahead (at the start of the previous layer's
        // epilogue): vector loads return in order, so a request made here would hold
        // the first weight fragments of the K loop behind its HBM latency.

        f16v acc[6];
#pragma unroll
        for (int t = 0; t < 6; t++) acc[t] = zero16();
        const u4* wp = a.wg_bf + ((size_t)l * kKb16Hid * 4 + wave) * 6 * 64;
        // The weights travel kGateAhead K blocks ahead: one block ahead, every block of six
        // MFMAs (192 cycles) sat out a whole L2 round trip (~1000 cycles under this load).
        // The first blocks of layers 1.. were requested before the previous epilogue, ahead
        // of its stores and of the state requests in the in-order return queue.
        if (l == 0) {
#pragma unroll
            for (int i = 0; i < kGateAhead; i++)
#pragma unroll
                for (int t = 0; t < 6; t++)
                    bq[i][t] = (wp + (size_t)i * KB_STRIDE + t * 64)[lane_u];
        }
#pragma unroll
        for (int kb = 0; kb < kKb16Hid; kb++) {
            if (kb + kGateAhead < kKb16Hid) {
#pragma unroll
                for (int t = 0; t < 6; t++)
                    bq[(kb + kGateAhead) % (kGateAhead + 1)][t] =
                        (wp + (size_t)(kb + kGateAhead) * KB_STRIDE + t * 64)[lane_u];
            }
            const u4 av = a_frag(xs4, l32, g, kb);
#pragma unroll
            for (int t = 0; t < 6; t++)
                acc[t] = mfma16(av, bq[kb % (kGateAhead + 1)][t], acc[t]);
        }
        if (l + 1 < a.layers) {
            const u4* wn = wp + (size_t)kKb16Hid * 4 * 6 * 64;   // next layer's mirror
#pragma unroll
            for (int i = 0; i < kGateAhead; i++)
#pragma unroll
                for (int t = 0; t < 6; t++)
                    bq[i][t] = (wn + (size_t)i * KB_STRIDE + t * 64)[lane_u];
        }
        __syncthreads();   // every wave has read the layer input

        if (l + 1 < a.layers) state_fetch(state_base(l + 1), stn);
        float* rs_base = HAS_RS ? a.r_state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN + wave * 64
                                : nullptr;
        __bf16* rs16 = (HAS_RS && RS16) ? reinterpret_cast<__bf16*>(a.r_state) + (size_t)l * a.layer_stride +
                                              e0 * CFP_HIDDEN + wave * 64
                                        : nullptr;
        float* out_base = TRAIN ? a.tr_x[l + 1] + e0 * CFP_HIDDEN + wave * 64 : nullptr;
        float* pre_base = TRAIN ? a.tr_pre[l] + e0 * CFP_GRU + wave * 64 : nullptr;
        __bf16* out16 = TR16 ? reinterpret_cast<__bf16*>(a.tr_x[l + 1]) + e0 * CFP_HIDDEN + wave * 64 : nullptr;
        __bf16* pre16 = TR16 ? reinterpret_cast<__bf16*>(a.tr_pre[l]) + e0 * CFP_GRU + wave * 64 : nullptr;
#pragma unroll
        for (int e = 0; e < 32; e++) {
            const int ut = e / 16, r = e % 16;
            const int soff = acc_row(r) * CFP_HIDDEN + ut * 32;
            float* xp = lds + (acc_row(r) + 4 * g) * XS + wave * 64 + ut * 32 + l32;
            const float s = (!TRAIN && ((tmask >> r) & 1u)) ? 0.0f : st[e];
            if (HAS_RS && RS16) __builtin_nontemporal_store((__bf16)s, (rs16 + soff) + loff);
            else if (HAS_RS) __builtin_nontemporal_store(s, (rs_base + soff) + loff);
            const float zh = acc[0 + ut][r];
            const float zg = acc[2 + ut][r];
            const float zp = acc[4 + ut][r];
            if (TR16) {
                __bf16* pp = pre16 + (acc_row(r) * CFP_GRU + ut * 32);
                __builtin_nontemporal_store((__bf16)zh, pp + loff3);
                __builtin_nontemporal_store((__bf16)zg, (pp + CFP_HIDDEN) + loff3);
                __builtin_nontemporal_store((__bf16)zp, (pp + 2 * CFP_HIDDEN) + loff3);
            } else if (TRAIN) {
                float* pp = pre_base + (acc_row(r) * CFP_GRU + ut * 32);
                __builtin_nontemporal_store(zh, pp + loff3);
                __builtin_nontemporal_store(zg, (pp + CFP_HIDDEN) + loff3);
                __builtin_nontemporal_store(zp, (pp + 2 * CFP_HIDDEN) + loff3);
            }
            const float sg = sigmoid_fast(zg);
            const float sh = sigmoid_fast(zh);
            const float gh = zh >= 0.0f ? zh + 0.5f : sh;
            // explicit fused multiply-adds: left to the compiler, which product of
            // p*out + (1-p)*x gets contracted depends on the surrounding code, and every
            // instantiation of this kernel must produce the same bits
            const float out = __builtin_fmaf(sg, gh - s, s);
            const float p = sigmoid_fast(zp);
            const float xv = *xp;
            const float hn = __builtin_fmaf(p, out - xv, xv);
            *xp = hn;
            if (TR16) __builtin_nontemporal_store((__bf16)hn, (out16 + soff) + loff);
            else if (TRAIN) __builtin_nontemporal_store(hn, (out_base + soff) + loff);
            else __builtin_nontemporal_store(out, (st_base + soff) + loff);
        }
#pragma unroll
        for (int e = 0; e < 32; e++) st[e] = stn[e];
        __syncthreads();
    }
    if (a.layers > 0 && a.h3_out) copy_tile_out(lds, a.h3_out + e0 * CFP_HIDDEN, tid);

    // ---- heads: waves 0 and 1 take one 32-row tile each over the full K -------
    if (a.do_head && wave < 2) {
        f16v hacc = zero16();
        const u4* wp = a.wav_bf + (size_t)wave * 64;
#pragma unroll
        for (int kb = 0; kb < kKb16Hid; kb++) {
            const u4 b = (wp + (size_t)kb * 128)[lane_u];
            const u4 av = a_frag(xs4, l32, g, kb);
            hacc = mfma16(av, b, hacc);
        }
        const int arow = wave * 32 + l32;
        const int avs = a.actions + 1;     // 44, or 18 for the classic game
        if (arow < avs) {
            const float bias = arow < a.actions ? a.b_a[arow] : a.b_v[0];
            float* av_base = a.av_out + e0 * avs;
            const int aoff = (4 * g) * avs + arow;
#pragma unroll
            for (int r = 0; r < 16; r++)
                (av_base + acc_row(r) * avs)[aoff] = hacc[r] + bias;
        }
    }
}

int launch_forward_bf16(const FwdArgs& a, hipStream_t st) {
    CFP_REQUIRE(a.we_bf && a.wg_bf && a.wav_bf, "bf16 forward without bf16 weight mirrors");
    CFP_REQUIRE(a.variant == 0 || !a.rec || (a.we_s3 && a.we_pk),
                "classic bf16 forward without the split encoder mirror");
    const dim3 g(a.n / kTileEnvs), b(kFwdThreads);
    if (a.train) {
        CFP_REQUIRE(a.variant == 0 && a.rec && a.state && a.layers > 0 && !a.r_state &&
                        !a.terminals && a.tr_mb > 0 && a.tr_mb % kTileEnvs == 0 &&
                        a.h_enc_out == a.tr_x[0],
                    "window recompute: bad arguments");
        CFP_REQUIRE(!a.rs_bf16 || a.tr_bf16, "a bf16 state slab goes with the bf16 storage of the window");
        if (a.tr_bf16 && a.rs_bf16)
            hipLaunchKernelGGL((k_policy_forward_bf16<0, false, true, true, true>), g, b, 0, st, a);
        else if (a.tr_bf16) hipLaunchKernelGGL((k_policy_forward_bf16<0, false, true, true>), g, b, 0, st, a);
        else hipLaunchKernelGGL((k_policy_forward_bf16<0, false, true>), g, b, 0, st, a);
    } else if (a.variant == 1) {
        CFP_REQUIRE(!(a.rs_bf16 && a.r_state), "the classic policy has no bf16 state slab");
        if (a.r_state) hipLaunchKernelGGL((k_policy_forward_bf16<1, true, false>), g, b, 0, st, a);
        else hipLaunchKernelGGL((k_policy_forward_bf16<1, false, false>), g, b, 0, st, a);
    } else {
        if (a.r_state && a.rs_bf16)
            hipLaunchKernelGGL((k_policy_forward_bf16<0, true, false, false, true>), g, b, 0, st, a);
        else if (a.r_state) hipLaunchKernelGGL((k_policy_forward_bf16<0, true, false>), g, b, 0, st, a);
        else hipLaunchKernelGGL((k_policy_forward_bf16<0, false, false>), g, b, 0, st, a);
    }
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

// ---- bf16 MFMA-ordered weight mirrors ---------------------------------------------
// One 16-byte element (eight bf16) per lane and K block: lane l carries
// k = 16*kb + 8*(l/32) + j of column l%32 of its 32-wide tile.
__global__ void k_pack_enc_bf16(const float* __restrict__ W_enc, __bf16* __restrict__ out,
                                int total) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int j = idx & 7, lane = (idx >> 3) & 63, ut = (idx >> 9) & 1, wave = (idx >> 10) & 3,
        kb = idx >> 12;
    int unit = wave * 64 + ut * 32 + (lane & 31);
    int f = 16 * kb + 8 * (lane >> 5) + j;
    out[idx] = (__bf16)(f < CFP_OBS ? W_enc[(size_t)f * CFP_HIDDEN + unit] : 0.0f);
}

__global__ void k_pack_gru_bf16(const float* __restrict__ W_gru, __bf16* __restrict__ out,
                                int total) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int layer = idx / (int)kGruPackFloats;
    int i = idx - layer * (int)kGruPackFloats;
    int j = i & 7, lane = (i >> 3) & 63, q = i >> 9;
    int t = q % 6, wave = (q / 6) & 3, kb = q / 24;
    int gate = t >> 1, ut = t & 1;
    int row = gate * CFP_HIDDEN + wave * 64 + ut * 32 + (lane & 31);
    int k = 16 * kb + 8 * (lane >> 5) + j;
    out[idx] = (__bf16)W_gru[(size_t)layer * kGruPackFloats + (size_t)row * CFP_HIDDEN + k];
}

__global__ void k_pack_av_bf16(const float* __restrict__ W_a, const float* __restrict__ W_v,
                               __bf16* __restrict__ out, int actions) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int)kAvPackFloats) return;
    int j = idx & 7, lane = (idx >> 3) & 63, nt = (idx >> 9) & 1, kb = idx >> 10;
    int arow = nt * 32 + (lane & 31);
    int k = 16 * kb + 8 * (lane >> 5) + j;
    float v = 0.0f;
    if (arow < actions) v = W_a[arow * CFP_HIDDEN + k];
    else if (arow == actions) v = W_v[k];
    out[idx] = (__bf16)v;
}

int launch_pack_weights_bf16(const float* params, int layers, int variant, uint16_t* we_bf,
                             uint16_t* wg_bf, uint16_t* wav_bf, hipStream_t st) {
    const Arena ar = arena_of(variant, layers);
    if (variant == 0) {   // the classic encoder gathers from the unpacked fp32 W_enc
        const int enc_total = (int)kEncPackFloats;
        hipLaunchKernelGGL(k_pack_enc_bf16, dim3((enc_total + 255) / 256), dim3(256), 0, st,
                           params + ar.w_enc, reinterpret_cast<__bf16*>(we_bf), enc_total);
    }
    const int gru_total = layers * (int)kGruPackFloats;
    hipLaunchKernelGGL(k_pack_gru_bf16, dim3((gru_total + 255) / 256), dim3(256), 0, st,
                       params + ar.w_gru, reinterpret_cast<__bf16*>(wg_bf), gru_total);
    hipLaunchKernelGGL(k_pack_av_bf16, dim3(((int)kAvPackFloats + 255) / 256), dim3(256), 0, st,
                       params + ar.w_a, params + ar.w_v, reinterpret_cast<__bf16*>(wav_bf),
                       ar.actions);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace cfp
