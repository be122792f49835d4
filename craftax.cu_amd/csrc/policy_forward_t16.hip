// Fused policy forward on 16-env tiles, for batches too small to give every CU a
// 32-env tile (the rollout of a PPO run: a few thousand envs).  Same path as
// policy_forward.hip -- records -> Linear(843->256) -> MinGRU x L -> actor/value heads,
// replacing the reference's per-step chain (craftax_full.cu:11954-11962, 11988-12008,
// 12044) in one launch -- on the 16 x 16 matrix instructions:
//   v_mfma_f32_16x16x4_f32   gates, heads, the encoder's 51 fp32 tail features
//   v_mfma_f32_16x16x32_bf16 the encoder's 792 byte-valued features against the exact
//                            three-term bf16 split of the fp32 weights
// A tile's matrix-pipe time is half that of a 32-env tile, and 4096 envs are 256 tiles:
// one per CU instead of one per two.  Opt-in (cfp_policy_set_small_tiles): another MFMA
// shape adds its products up in another order, so the last bits differ from the 32-env
// kernels', which every other entry point and batch size share.
//
// Workgroup: 512 threads = 8 waves, two per SIMD (one wave's weight requests and
// epilogue issue while the other's MFMAs run); wave w owns units [32w, 32w+32) as two
// 16-wide unit tiles.  Weights stream L2 -> per-wave LDS ring (LDS-direct loads, two K
// blocks ahead, no registers written) -> registers (one block ahead): a 16-byte global
// load into registers costs the issuing wave several times the matrix-pipe time of an
// LDS-direct request plus the LDS read, and a 16-env tile needs twice the weight bytes
// per MFMA cycle of a 32-env one.  Operand layout of the 16 x 16 instructions: lane l supplies row (A) /
// column (B) l%16 and k group l/16; accumulator register r of lane l holds env
// 4*(l/16) + r, unit l%16.  Weights come from mirrors in that order (k_pack_t16): one
// 16-byte element per lane feeds four k steps, a wave's fragment is a contiguous 1 KiB.
#include "policy_tile.h"
#include "sample_row.h"

namespace cfp {
namespace {

constexpr int kT16Envs = 16;
constexpr int kT16Threads = 512;
constexpr int kT16EncSteps = (CFP_OBS_MAP + 31) / 32;   // 25 K steps of 32 map bytes
constexpr int kT16TailBlocks = 4;                       // 64 >= 51 fp32 tail features
constexpr int kT16GateBlocks = CFP_HIDDEN / 16;         // 16 K blocks of 16
constexpr int kT16HeadTiles = 3;                        // 48 >= 44 head rows
constexpr int kT16RecV4 = kT16Envs * REC_DW / 4;        // 996 16-byte chunks of records
constexpr int kT16LdsFloats = kT16Envs * XS;            // x tile [16][260] >= records [16][255]
static_assert(kT16Envs * RS <= kT16LdsFloats, "records fit the x tile");
static_assert((kT16Envs * REC_DW) % 4 == 0, "a tile's records are whole 16-byte chunks");

// mirror sizes in 16-byte elements
constexpr size_t kT16EncS = (size_t)kT16EncSteps * 16 * 3 * 64;
constexpr size_t kT16EncT = (size_t)kT16TailBlocks * 16 * 64;
constexpr size_t kT16Gru = (size_t)kT16GateBlocks * 8 * 6 * 64;   // per layer
constexpr size_t kT16Av = (size_t)kT16GateBlocks * kT16HeadTiles * 64;

// ---- weight stream: global -> LDS ring -> registers ---------------------------------
// One K block of a wave = six 1 KiB fragments = one ring slot.  The LDS-direct loads are
// issued from inline assembly (lane l's 16 bytes land at M0 base + 16 l + offset); the
// compiler does not know of them, so the wait that makes a slot readable is an explicit
// s_waitcnt vmcnt(N), N = the number of vector-memory operations this lane's wave issued
// after the slot's six (they complete in issue order).  The compiler's own waits then
// only ever over-wait.  `after`: a register the slot's previous contents were last read
// into; as an operand it keeps the request behind the completion of those reads.
constexpr int kT16RingSlots = 2;
constexpr int kT16SlotF4 = 6 * 64;

__device__ __forceinline__ void t16_dma(const f4* src, f4* slot, unsigned lane, float after = 0.0f) {
    const unsigned lds_lo = (unsigned)(size_t)slot;
    const unsigned voff = lane * 16u;
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, %1\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:1024\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:2048\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:3072"
        :
        : "v"(voff), "s"(src), "s"(lds_lo), "v"(after)
        : "memory", "m0");
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, %1\n\t"
        "global_load_lds_dwordx4 %0, %1 offset:1024"
        :
        : "v"(voff), "s"(src + 4 * 64), "s"(lds_lo + 4096u)
        : "memory", "m0");
}

// s_waitcnt vmcnt(n); n folds to a constant or to one of a few values chosen at run time
__device__ __forceinline__ void t16_wait(int n) {
#define CFP_T16_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        CFP_T16_W(6) CFP_T16_W(8) CFP_T16_W(14) CFP_T16_W(16) CFP_T16_W(22) CFP_T16_W(24) CFP_T16_W(30)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef CFP_T16_W
}

__device__ __forceinline__ f4 mfma4(float a, float b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f4 mfma32b(const u4& a, const u4& b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// One 16-byte element of the mirrors per thread.
//   encoder, map bytes : [step s][unit tile T][term][lane]  eight bf16: feature 32 s + 8 (l/16) + j,
//                        unit 16 T + l%16, term = hi / mid / lo of the fp32 weight
//   encoder, fp32 tail : [block B][unit tile T][lane]       feature 792 + 16 B + 4 (l/16) + m
//   gates              : [layer][K][wave][gate*2 + ut][lane] row gate*256 + 32 wave + 16 ut + l%16,
//                        k = 16 K + 4 (l/16) + m
//   heads              : [K][row tile][lane]                 row 16 tile + l%16 (43 = value, then zeros)
__global__ void k_pack_t16(const float* __restrict__ W_enc, const float* __restrict__ W_gru,
                           const float* __restrict__ W_a, const float* __restrict__ W_v, int layers,
                           u4* __restrict__ enc_s, f4* __restrict__ enc_t, f4* __restrict__ gru,
                           f4* __restrict__ av) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = (int)(i & 63), q = lane >> 4, c = lane & 15;
    if (i < kT16EncS) {
        const int term = (int)((i >> 6) % 3), T = (int)((i / 192) % 16), s = (int)(i / (192 * 16));
        uint32_t d[4];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            uint32_t pair = 0;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int f = 32 * s + 8 * q + 2 * p + h;
                const float w = f < CFP_OBS_MAP ? W_enc[(size_t)f * CFP_HIDDEN + 16 * T + c] : 0.0f;
                const __bf16 hi = (__bf16)w;
                const float r1 = w - (float)hi;
                const __bf16 mid = (__bf16)r1;
                const __bf16 lo = (__bf16)(r1 - (float)mid);
                const __bf16 v = term == 0 ? hi : (term == 1 ? mid : lo);
                pair |= (uint32_t)__builtin_bit_cast(uint16_t, v) << (16 * h);
            }
            d[p] = pair;
        }
        enc_s[i] = u4{d[0], d[1], d[2], d[3]};
        return;
    }
    i -= kT16EncS;
    if (i < kT16EncT) {
        const int T = (int)((i >> 6) % 16), B = (int)(i / (64 * 16));
        f4 v;
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const int f = CFP_OBS_MAP + 16 * B + 4 * q + m;
            v[m] = f < CFP_OBS ? W_enc[(size_t)f * CFP_HIDDEN + 16 * T + c] : 0.0f;
        }
        enc_t[i] = v;
        return;
    }
    i -= kT16EncT;
    if (i < (size_t)layers * kT16Gru) {
        const int layer = (int)(i / kT16Gru);
        const size_t j = i - (size_t)layer * kT16Gru;
        const int t = (int)((j >> 6) % 6), wave = (int)((j / 384) % 8), K = (int)(j / (384 * 8));
        const int row = (t >> 1) * CFP_HIDDEN + 32 * wave + 16 * (t & 1) + c;
        const float* src = W_gru + ((size_t)layer * CFP_GRU + row) * CFP_HIDDEN + 16 * K + 4 * q;
        gru[i] = f4{src[0], src[1], src[2], src[3]};
        return;
    }
    i -= (size_t)layers * kT16Gru;
    if (i < kT16Av) {
        const int tile = (int)((i >> 6) % kT16HeadTiles), K = (int)(i / (64 * kT16HeadTiles));
        const int row = 16 * tile + c;
        const float* src = row < CFP_ACTIONS ? W_a + (size_t)row * CFP_HIDDEN
                                             : (row == CFP_ACTIONS ? W_v : nullptr);
        f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (src) {
            src += 16 * K + 4 * q;
            v = f4{src[0], src[1], src[2], src[3]};
        }
        av[i] = v;
    }
}

// MODE 0: inference; MODE 1: also records the post-zero state (r_state).
template <int MODE>
__global__ __launch_bounds__(kT16Threads, 1) void k_policy_forward_t16(FwdArgs a) {
    __shared__ __attribute__((aligned(16))) float lds[kT16LdsFloats];
    __shared__ __attribute__((aligned(16))) f4 ring_all[8 * kT16RingSlots * kT16SlotF4];   // 96 KiB
    __shared__ float term_s[kT16Envs];
    const int tid = threadIdx.x;
    const unsigned lane = (unsigned)(tid & 63);
    const int q = (tid & 63) >> 4;     // k group of the operands, env group of the accumulators
    const int c = tid & 15;            // row (A) / column (B) / unit within a 16-wide tile
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const size_t e0 = (size_t)blockIdx.x * kT16Envs;
    const f4* xs4 = reinterpret_cast<const f4*>(lds);
    f4* const ring = ring_all + wave * (kT16RingSlots * kT16SlotF4);   // this wave's ring

    // element e = 4 ut + r of a lane: env 4 q + r, unit 32 wave + 16 ut + c
    const unsigned soff = (unsigned)((4 * q) * CFP_HIDDEN + 32 * wave + c);
    auto state_fetch = [&](const float* base, float (&v)[8]) {
#pragma unroll
        for (int e = 0; e < 8; e++)
            v[e] = __builtin_nontemporal_load((base + ((e & 3) * CFP_HIDDEN + (e >> 2) * 16)) + soff);
    };
    // the draw's offset (rollout step in one launch), requested before anything else
    const uint64_t draw_step = a.s_act ? *a.s_step : 0;
    // Every layer's state first: it travels beside the records, is older than every weight
    // request (requests return in order: a state load issued later would hold the weight
    // stream up behind its HBM latency) and has long landed when its epilogue comes.
    float st[CFP_MAX_LAYERS][8];
#pragma unroll
    for (int l = 0; l < CFP_MAX_LAYERS; l++)
        if (l < a.layers) state_fetch(a.state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN, st[l]);
    // The encoder's first weights next, ahead of the records: the fp32 tail's rows (used
    // last) and the first two steps of the ring.  The record loads that follow are the
    // compiler's; its waits for them only over-wait for these older requests.
    const f4* ws = reinterpret_cast<const f4*>(a.t16_enc_s) + (size_t)(2 * wave) * 3 * 64;
    constexpr size_t kStep = 16 * 3 * 64;
    f4 tw[kT16TailBlocks][2];
#pragma unroll
    for (int B = 0; B < kT16TailBlocks; B++) {
        tw[B][0] = a.t16_enc_t[(size_t)(B * 16 + 2 * wave) * 64 + lane];
        tw[B][1] = a.t16_enc_t[(size_t)(B * 16 + 2 * wave + 1) * 64 + lane];
    }
    // ... and the heads' weights: a wave takes K blocks 2 wave and 2 wave + 1 of the three
    // row tiles
    f4 hw[2][kT16HeadTiles];
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int t = 0; t < kT16HeadTiles; t++)
            hw[kb][t] = a.t16_wav[((size_t)(2 * wave + kb) * kT16HeadTiles + t) * 64 + lane];
    // (waves 0..2 finish head row 16 wave + c: its bias)
    const int head_row = 16 * wave + c;
    float head_bias = 0.0f;
    if (head_row < CFP_AV) head_bias = head_row < CFP_ACTIONS ? a.b_a[head_row] : a.b_v[0];
    asm volatile("" ::: "memory");
    t16_dma(ws, ring, lane);
    t16_dma(ws + kStep, ring + kT16SlotF4, lane);

    // ---- stage the tile's records: contiguous 16-byte loads, rows re-strided to RS dwords
    {
        uint32_t* rs = reinterpret_cast<uint32_t*>(lds);
        const u4* src = reinterpret_cast<const u4*>(a.rec + e0 * CFP_REC_BYTES);
        for (int i = tid; i < kT16RecV4; i += kT16Threads) {
            const u4 v = __builtin_nontemporal_load(src + i);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int d = 4 * i + k, row = d / REC_DW;
                rs[row * RS + (d - row * REC_DW)] = w[k];
            }
        }
        if (tid < kT16Envs * (RS - REC_DW)) {
            const int row = tid / (RS - REC_DW);
            rs[row * RS + REC_DW + (tid - row * (RS - REC_DW))] = 0u;
        }
        if (tid < kT16Envs) term_s[tid] = a.terminals ? a.terminals[e0 + tid] : 0.0f;
    }
    __syncthreads();
    unsigned tmask = 0u;
#pragma unroll
    for (int r = 0; r < 4; r++)
        if (term_s[4 * q + r] != 0.0f) tmask |= 1u << r;

    constexpr size_t kBlock = 8 * 6 * 64;   // f4 per K block of the gate mirror
    auto gate_base = [&](int l) { return a.t16_wg + ((size_t)l * kT16GateBlocks * 8 + wave) * 6 * 64; };
    // the first two K blocks of a layer are requested before the phase in front of it ends
    // (after0 / after1: registers the slots' last contents were read into)
    auto gate_preload = [&](int l, float after0, float after1) {
        t16_dma(gate_base(l), ring, lane, after0);
        t16_dma(gate_base(l) + kBlock, ring + kT16SlotF4, lane, after1);
    };
    constexpr int kStores = MODE == 1 ? 16 : 8;   // an epilogue's stores per lane: state (+ r_state)

    // ---- encoder ----------------------------------------------------------------------
    {
        f4 eacc[2] = {f4{0, 0, 0, 0}, f4{0, 0, 0, 0}};
        const uint32_t* rrow = reinterpret_cast<const uint32_t*>(lds) + c * RS;
        // (this wave's six fragments of a step: unit tiles 2 wave, 2 wave + 1 x (hi, mid, lo);
        // steps 0 and 1 were requested before the records; every request of this lane
        // since then has been consumed)
        u4 b[2][6];
        t16_wait(6);   // step 0 landed; step 1 may be in flight
#pragma unroll
        for (int t = 0; t < 6; t++) b[0][t] = __builtin_bit_cast(u4, ring[t * 64 + lane]);
#pragma unroll
        for (int s = 0; s < kT16EncSteps; s++) {
            const int cb = s & 1, nb = cb ^ 1;
            if (s + 2 < kT16EncSteps)
                t16_dma(ws + (size_t)(s + 2) * kStep, ring + (s % kT16RingSlots) * kT16SlotF4, lane,
                        __uint_as_float(b[cb][5].w));
            if (s + 1 < kT16EncSteps) {
                t16_wait(s + 2 < kT16EncSteps ? 6 : 0);   // step s+1 landed; younger: step s+2
                const f4* slot = ring + ((s + 1) % kT16RingSlots) * kT16SlotF4 + lane;
#pragma unroll
                for (int t = 0; t < 6; t++) b[nb][t] = __builtin_bit_cast(u4, slot[t * 64]);
            }
            u4 av = bytes_to_bf16x8(rrow[8 * s + 2 * q], rrow[8 * s + 2 * q + 1]);
            if (s == kT16EncSteps - 1 && q == 3) av = u4{0u, 0u, 0u, 0u};   // 792..799: not map bytes
#pragma unroll
            for (int term = 0; term < 3; term++) {
                eacc[0] = mfma32b(av, b[cb][term], eacc[0]);
                eacc[1] = mfma32b(av, b[cb][3 + term], eacc[1]);
            }
        }
        const float* frow = reinterpret_cast<const float*>(rrow) + CFP_OBS_MAP / 4;
#pragma unroll
        for (int B = 0; B < kT16TailBlocks; B++) {
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const int k = 16 * B + 4 * q + m;
                const float x = k < CFP_OBS_TAIL ? frow[k] : 0.0f;   // past the record: not read as a float
                eacc[0] = mfma4(x, tw[B][0][m], eacc[0]);
                eacc[1] = mfma4(x, tw[B][1][m], eacc[1]);
            }
        }
        // biases before the preload: a load behind it would have to wait for it
        float bias[2];
#pragma unroll
        for (int ut = 0; ut < 2; ut++) bias[ut] = a.b_enc[32 * wave + 16 * ut + c];
        asm volatile("" ::: "memory");
        // the ring is idle: its last two slots were read into b[0] and b[1]
        if (a.layers > 0) gate_preload(0, __uint_as_float(b[0][5].w), __uint_as_float(b[1][5].w));
        __syncthreads();   // every wave is done with the record bytes
#pragma unroll
        for (int ut = 0; ut < 2; ut++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                lds[(4 * q + r) * XS + 32 * wave + 16 * ut + c] = eacc[ut][r] + bias[ut];
    }
    __syncthreads();
    auto tile_out = [&](float* dst) {   // two 16-byte stores per lane
        f4* d4 = reinterpret_cast<f4*>(dst + e0 * CFP_HIDDEN);
#pragma unroll
        for (int j = 0; j < kT16Envs * CFP_HIDDEN / 4 / kT16Threads; j++) {
            const int i = tid + j * kT16Threads;
            d4[i] = xs4[(i >> 6) * XS4 + (i & 63)];
        }
    };
    // vector-memory operations this lane issued after the pending preload of layer 0:
    // the stores of tile_out, if any
    int pending = 0;
    if (a.h_enc_out) {
        tile_out(a.h_enc_out);
        pending = 2;
    }

    // ---- MinGRU layers -------------------------------------------------------------------
#pragma unroll
    for (int l = 0; l < CFP_MAX_LAYERS; l++) {
        if (l >= a.layers) break;
        f4 acc[6];
#pragma unroll
        for (int t = 0; t < 6; t++) acc[t] = f4{0, 0, 0, 0};
        const f4* wp = gate_base(l);
        // On entry blocks 0 and 1 have been requested, followed by `pending` other
        // operations of this lane: block 0 has landed when at most 6 + pending are left.
        f4 bl[2][6];
        t16_wait(6 + pending);
#pragma unroll
        for (int t = 0; t < 6; t++) bl[0][t] = ring[t * 64 + lane];
        f4 av = xs4[c * XS4 + q];
#pragma unroll
        for (int K = 0; K < kT16GateBlocks; K++) {
            const int cb = K & 1, nb = cb ^ 1;
            if (K + 2 < kT16GateBlocks)
                t16_dma(wp + (size_t)(K + 2) * kBlock, ring + (K % kT16RingSlots) * kT16SlotF4, lane,
                        bl[cb][5][3]);
            f4 avn = av;
            if (K + 1 < kT16GateBlocks) {
                // block K+1 landed; younger: block K+2 and, at K = 0, what followed the preload
                if (K == 0) t16_wait(6 + pending);
                else t16_wait(K + 2 < kT16GateBlocks ? 6 : 0);
                const f4* slot = ring + ((K + 1) % kT16RingSlots) * kT16SlotF4 + lane;
#pragma unroll
                for (int t = 0; t < 6; t++) bl[nb][t] = slot[t * 64];
                avn = xs4[c * XS4 + 4 * (K + 1) + q];
            }
#pragma unroll
            for (int m = 0; m < 4; m++)
#pragma unroll
                for (int t = 0; t < 6; t++) acc[t] = mfma4(av[m], bl[cb][t][m], acc[t]);
            av = avn;
        }
        // next layer's first blocks, ahead of this epilogue's loads and stores
        if (l + 1 < a.layers) gate_preload(l + 1, bl[0][5][3], bl[1][5][3]);
        __syncthreads();   // every wave has read the layer input
        pending = kStores;
        float* st_base = a.state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN;
        float* rs_base = MODE == 1 ? a.r_state + (size_t)l * a.layer_stride + e0 * CFP_HIDDEN : nullptr;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int ut = e >> 2, r = e & 3;
            const unsigned off = (unsigned)(r * CFP_HIDDEN + ut * 16);
            const float s = ((tmask >> r) & 1u) ? 0.0f : st[l][e];
            if (MODE == 1) __builtin_nontemporal_store(s, (rs_base + off) + soff);
            const float zh = acc[0 + ut][r], zg = acc[2 + ut][r], zp = acc[4 + ut][r];
            const float sg = sigmoid_fast(zg);
            const float sh = sigmoid_fast(zh);
            const float gh = zh >= 0.0f ? zh + 0.5f : sh;
            const float out = __builtin_fmaf(sg, gh - s, s);
            const float p = sigmoid_fast(zp);
            float* xp = lds + (4 * q + r) * XS + 32 * wave + 16 * ut + c;
            const float xv = *xp;
            *xp = __builtin_fmaf(p, out - xv, xv);
            __builtin_nontemporal_store(out, (st_base + off) + soff);
        }
        __syncthreads();
    }
    if (a.h3_out) tile_out(a.h3_out);

    // ---- heads: every wave takes two of the sixteen K blocks of all three 16-row tiles;
    // the eight partial sums meet in LDS and are added in wave order
    __shared__ float s_logit[kT16Envs * CFP_AV];
    __shared__ float s_expo[kT16Envs * kMaxActions];
    __shared__ __attribute__((aligned(16))) f4 s_hpart[8][kT16HeadTiles][64];   // 24 KiB
    static_assert(kT16GateBlocks == 16, "two K blocks per wave");
    {
        f4 hacc[kT16HeadTiles];
#pragma unroll
        for (int t = 0; t < kT16HeadTiles; t++) hacc[t] = f4{0, 0, 0, 0};
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const f4 av = xs4[c * XS4 + 4 * (2 * wave + kb) + q];
#pragma unroll
            for (int m = 0; m < 4; m++)
#pragma unroll
                for (int t = 0; t < kT16HeadTiles; t++) hacc[t] = mfma4(av[m], hw[kb][t][m], hacc[t]);
        }
#pragma unroll
        for (int t = 0; t < kT16HeadTiles; t++) s_hpart[wave][t][lane] = hacc[t];
    }
    __syncthreads();
    if (wave < kT16HeadTiles) {
        f4 hacc = s_hpart[0][wave][lane];
#pragma unroll
        for (int w = 1; w < 8; w++) {
            const f4 part = s_hpart[w][wave][lane];
#pragma unroll
            for (int r = 0; r < 4; r++) hacc[r] += part[r];
        }
        const int row = head_row;
        if (row < CFP_AV) {
            float* o = a.av_out + (e0 + 4 * q) * CFP_AV + row;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float v = hacc[r] + head_bias;
                o[r * CFP_AV] = v;
                s_logit[(4 * q + r) * CFP_AV + row] = v;
            }
        }
    }
    // ---- the draw, sixteen lanes per env (sample_row.h), and the step counter's bump ---------
    if (a.s_act) {   // uniform over the launch
        __syncthreads();
        const int sub = tid % kSampleLanes, slot = tid / kSampleLanes;
        const bool live = slot < kT16Envs;
        const float* lp = s_logit + (live ? slot : 0) * CFP_AV;
        float* px = s_expo + (live ? slot : 0) * kMaxActions;
        const float mx = sample_spread(lp, px, CFP_ACTIONS, sub, live);
        __syncthreads();
        // The ticket behind the last barrier (a barrier waits for the atomic's return): its
        // round trip runs under the scan of the draw.  Every lane's read of the counter
        // (draw_step, the kernel's first load) has returned: loads return in order, and
        // younger ones fed the MFMAs in front of the barriers above.
        unsigned ticket_no = 0u;
        if (tid == 0) ticket_no = take_ticket(a.s_ticket);
        if (live && sub == 0)
            sample_draw<CFP_ACTIONS>(lp, px, mx, CFP_ACTIONS, (int)e0 + slot, a.s_seed, draw_step,
                        a.s_env_actions, a.s_act, a.s_logp, a.s_value);
        if (tid == 0) bump_if_last(ticket_no, gridDim.x, a.s_ticket, a.s_step, draw_step);
    }
}

}  // namespace

size_t t16_mirror_bytes(int layers) {
    return (kT16EncS + kT16EncT + (size_t)layers * kT16Gru + kT16Av) * 16;
}

void t16_mirror_layout(void* base, int layers, const u4** enc_s, const f4** enc_t, const f4** gru,
                       const f4** av) {
    char* p = static_cast<char*>(base);
    *enc_s = reinterpret_cast<const u4*>(p);
    p += kT16EncS * 16;
    *enc_t = reinterpret_cast<const f4*>(p);
    p += kT16EncT * 16;
    *gru = reinterpret_cast<const f4*>(p);
    p += (size_t)layers * kT16Gru * 16;
    *av = reinterpret_cast<const f4*>(p);
}

int launch_pack_weights_t16(const float* params, int layers, void* mirrors, hipStream_t st) {
    const u4* es; const f4 *et, *g, *av;
    t16_mirror_layout(mirrors, layers, &es, &et, &g, &av);
    const size_t total = kT16EncS + kT16EncT + (size_t)layers * kT16Gru + kT16Av;
    const Arena ar = arena_of(0, layers);
    hipLaunchKernelGGL(k_pack_t16, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                       params + ar.w_enc, params + ar.w_gru, params + ar.w_a, params + ar.w_v, layers,
                       const_cast<u4*>(es), const_cast<f4*>(et), const_cast<f4*>(g),
                       const_cast<f4*>(av));
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

bool forward_t16_ok(const FwdArgs& a) {
    if (a.s_act && !(a.s_logp && a.s_step && a.s_ticket)) return false;
    return a.t16_wg && a.variant == 0 && a.rec && !a.train && !a.bf16 && a.layers > 0 && a.do_head &&
           a.state && a.av_out && a.n % kT16Envs == 0 && a.n <= kT16Envs * 256;
}

int launch_forward_t16(const FwdArgs& a, hipStream_t st) {
    CFP_REQUIRE(forward_t16_ok(a), "16-env tiles: records -> heads of the full game, at most 4096 envs");
    const dim3 g(a.n / kT16Envs), b(kT16Threads);
    if (a.r_state) hipLaunchKernelGGL(k_policy_forward_t16<1>, g, b, 0, st, a);
    else hipLaunchKernelGGL(k_policy_forward_t16<0>, g, b, 0, st, a);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace cfp
