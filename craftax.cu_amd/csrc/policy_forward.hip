// Fused policy forward for gfx950: 996-byte records -> Linear(843->256)
// -> MinGRU x L -> actor(43)/value(1), tiles of 32 envs.
//
// Replaces, in one launch, the reference's per-step chain
//   k_expand_obs + cublasSgemm + k_add_bias       (craftax_full.cu:11954-11962)
//   L x { cublasSgemm(768 x cn x 256) + k_mingru_epi_fwd }   (:11988-12008)
//   cublasSgemm(44 x n x 256) + bias adds of k_value_sample  (:12044, :9726)
// so neither the fp32 feature matrix nor the [768][chunk] gate
// pre-activations ever exist in HBM: the activations of a tile stay in LDS
// from the record bytes to the logits.
//
// Schedule.  One persistent workgroup (4 waves, one per SIMD, up to 512
// registers each) per CU walks PAIRS of 32-env tiles X, Y.  The gate/blend
// epilogue of one tile is woven, element by element, between the MFMAs of the
// other tile's next gate GEMM, so no wave ever sits in a pure vector phase:
//   ENC(X+Y) | bias | K(X,0) | K(Y,0)+epi(X,0) | K(X,1)+epi(Y,0) | ...
//   ... | K(Y,L-1)+epi(X,L-1) | epi(Y,L-1) | HEAD(X) HEAD(Y) | reduce, store
// ("|" = workgroup barrier).  `sched_group_barrier` pins the issue order inside
// a K block (1 MFMA : 2 VALU).  Measured on MI355X with v_mfma_f32_32x32x2_f32
// (64 cycles in the matrix pipe), one wave per SIMD: every vector or LDS
// instruction the MFMA-issuing wave issues in between delays its next MFMA by
// about 8.5 cycles (12.5 for a transcendental), a 16-byte global load into
// registers by 40-60.  So the design minimises instructions per MFMA rather than
// latency: per 24 MFMAs, 6 LDS-direct weight requests (no registers written),
// 7 LDS reads and ~25 epilogue instructions.  (The same instructions issued by a
// second wave on the SIMD cost the MFMA wave about as much: a two-group variant of
// this schedule measured no faster.)  The shader clock under this load settles at
// 2.36-2.41 GHz once it has ramped up from idle (some tens of milliseconds of load).
//
// Within the workgroup, wave w owns hidden units [64w, 64w+64).  MFMA operand
// convention (v_mfma_f32_32x32x2_f32): A = activations (row = env), B = weights
// (column = unit), so accumulator register r of lane l holds env
// 8*(r/4) + 4*(l/32) + r%4, unit l%32: a half-wave touches 32 consecutive units
// of one env, i.e. one full 128-byte line of state.
//   encoder: the byte-valued features (full game: 792 map bytes; classic game:
//            1323 cell bits) are exact in bf16 and run as three bf16 MFMAs per
//            product against an exact three-term bf16 split of the fp32 weights,
//            fp32 accumulate (policy_tile.h); the remaining fp32 features follow
//            on the fp32 MFMA.  Weight fragments stream through the same ring as
//            the gate weights and feed both tiles (4 accumulators)
//   layer:   6 accumulators (zh, zg, zp for 2 unit tiles) over K = 256; weights
//            go L2 -> per-wave LDS ring (LDS-direct loads, three K blocks ahead)
//            -> registers (one block ahead); the first three blocks and the 32
//            state values of the NEXT phase are requested before the barrier
//            that ends the current one; state and r_state leave through
//            non-temporal stores next to each epilogue element; h' goes back
//            into the x tile
//   heads:   2 row tiles x 2 K halves over the 4 waves, each weight fragment used for
//            both tiles, partial sums reduced through LDS.
#include "policy_tile.h"
#include "cfp_internal.h"
#include "sample_row.h"

namespace cfp {

namespace {

constexpr int kRedFloats = 2 * 16 * 64;               // head K-half partials
// ---- MinGRU phases ---------------------------------------------------------------
// Written-to-nowhere tile: state / r_state addresses of a pair's missing second
// tile point here, so the hot loop needs no predication.
__device__ float g_void_tile[kTileEnvs * CFP_HIDDEN];
__device__ float g_void_pre[kTileEnvs * CFP_GRU];

// State addressing of one (tile, layer) for the epilogue: element e = 0..31 of a
// lane is unit tile e/16, accumulator register e%16.
struct StateIO {
    float* st_base;    // state tile + wave*64 (uniform)
    float* rs_base;    // MODE 1: r_state tile likewise; MODE 2: next layer's input tile
    float* pre_base;   // MODE 2: gate pre-activation tile [32][768] + wave*64
    unsigned tmask;    // bit r: env row of accumulator register r had a terminal
};

// Kernel modes: 0 = inference, 1 = inference that also records the post-zero state
// (r_state), 2 = window recompute of the PPO update (state read from the stored
// slab and not written back; pre-activations and layer outputs written out).
constexpr int kModePlain = 0, kModeRecord = 1, kModeTrain = 2;

__device__ __forceinline__ constexpr int st_off(int e) {
    return acc_row(e % 16) * CFP_HIDDEN + (e / 16) * 32;
}

// Request the 32 state values the next epilogue will consume, in element order
// (the compiler barriers pin the issue order).  The epilogue consumes element kb
// in K block kb, so the wait the compiler places there leaves at least the 31
// youngest operations it knows of in flight -- and with them the weight requests
// issued since, which it does not know of and must not be made to wait for.
__device__ __forceinline__ void state_load(const StateIO& io, float (&st)[32], const Lane& L) {
#pragma unroll
    for (int e = 0; e < 32; e++) {
        st[e] = __builtin_nontemporal_load((io.st_base + st_off(e)) + L.loff);
        asm volatile("" ::: "memory");
    }
}

// ---- weight stream: global -> LDS -> registers -----------------------------------
// A 16-byte global load into registers costs the MFMA-issuing wave 40-60 cycles
// of matrix-pipe time on this machine wherever it hits; an LDS-direct load
// (global_load_lds_dwordx4: lane l's 16 bytes land at M0 base + 16*l, no
// registers involved) plus the LDS read that fetches the fragment cost about
// half of that together (a gate GEMM phase: 54.6k -> 51.0k cycles, of 49.2k
// ideal).  So each wave streams its weight fragments into a private LDS ring,
// three K blocks ahead, and reads the next block's six fragments back with
// ds_read_b128 while the current block multiplies.
// The LDS-direct loads are issued from inline assembly: the compiler does not
// know of them, so the wait that makes a ring slot readable is explicit
// (s_waitcnt vmcnt with the exact number of younger vector-memory operations;
// loads and stores complete in issue order) and every wait the compiler places
// for its own loads only ever over-waits.
constexpr int kRingSlots = 3;
constexpr int kRingSlotF4 = 6 * 64;                       // one K block of one wave: 6 KiB
constexpr int kRingF4 = 4 * kRingSlots * kRingSlotF4;     // 72 KiB for the workgroup

// K block kb of a layer (wp = mirror + layer + wave*6*64 fragments) -> ring slot.
// `after` is a register the slot's previous contents were last read into: as an
// operand it keeps the request behind the completion of those reads.  M0 (the LDS
// base of an LDS-direct load) is written by each block and declared as clobbered,
// so the compiler keeps nothing of its own in it across a request.
__device__ __forceinline__ void ring_dma(const f4* wp, int kb, f4* slot, const Lane& L,
                                         float after = 0.0f) {
    constexpr int KB_STRIDE = 4 * 6 * 64;
    const f4* src = wp + (size_t)kb * KB_STRIDE;
    const unsigned lds_lo = (unsigned)(size_t)slot;       // LDS byte address of the slot
    const unsigned voff = L.lane_u * 16u;
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

// First three K blocks of a layer's weights into ring slots 0, 1, 2.
__device__ __forceinline__ void ring_preload(f4* ring, const f4* wp, const Lane& L) {
#pragma unroll
    for (int i = 0; i < kRingSlots; i++) ring_dma(wp, i, ring + i * kRingSlotF4, L);
}

// s_waitcnt vmcnt(n); n must fold to a constant after unrolling (the switch then
// leaves one instruction).
__device__ __forceinline__ void vm_wait(int n) {
#define CFP_VMW(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        CFP_VMW(0) CFP_VMW(2) CFP_VMW(4) CFP_VMW(6) CFP_VMW(8) CFP_VMW(10) CFP_VMW(12)
        CFP_VMW(13) CFP_VMW(14) CFP_VMW(16) CFP_VMW(20) CFP_VMW(44) CFP_VMW(45) CFP_VMW(46)
        CFP_VMW(48)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef CFP_VMW
}

// ---- encoder GEMM of both tiles of a pair, weights through the ring ---------------
// The three-term bf16 weight fragments (policy_tile.h, "map bytes on the bf16 matrix
// pipe") are streamed like the gate weights: K block kb+3 requested into the ring
// and block kb+1 read back while block kb multiplies.  Its 16-byte elements and its
// 6 KiB per wave and block are those of the gate mirror, so ring_dma serves both.
template <bool ONE>
__device__ __forceinline__ void encoder_gemm_split_ring(const FwdArgs& a, const float* ldsX,
                                                        const float* ldsY, f4* ring,
                                                        const Lane& L, f16v (&acc)[4]) {
    static_assert(kKb16Split == 50 && CFP_OBS_MAP == 16 * 49 + 8, "block schedule below");
    const uint32_t* rx = reinterpret_cast<const uint32_t*>(ldsX) + L.l32 * RS;
    const uint32_t* ry = reinterpret_cast<const uint32_t*>(ldsY) + L.l32 * RS;
    // the fp32 tail's weights first: older than every ring request, used last
    const f4* wq = a.we_pk + (size_t)(L.wave * 2) * 64;
    constexpr int KB8_STRIDE = 4 * 2 * 64;
    f4 tb0[7], tb1[7];
#pragma unroll
    for (int t = 0; t < 7; t++) {
        const f4* p = wq + (size_t)(kKbMap + t) * KB8_STRIDE;
        tb0[t] = p[L.lane_u];
        tb1[t] = (p + 64)[L.lane_u];
    }
    asm volatile("" ::: "memory");
    const f4* wp = reinterpret_cast<const f4*>(a.we_s3) + (size_t)(L.wave * 6) * 64;
    ring_preload(ring, wp, L);
    EncDw cur = encs_bytes(rx, ry, 0, L.half);
    EncS bl[2];
    // block 0 landed: the preload's blocks 1 and 2 (6 requests each) are the only younger
    // operations -- the tail fragments above were requested before the preload
    vm_wait(12);
#pragma unroll
    for (int i = 0; i < 6; i++)
        bl[0].b[i] = __builtin_bit_cast(u4, ring[i * 64 + L.lane_u]);
#pragma unroll
    for (int kb = 0; kb < kKb16Split; kb++) {
        const int cb = kb & 1, nb = cb ^ 1;
        if (kb + 3 < kKb16Split)
            ring_dma(wp, kb + 3, ring + (kb % kRingSlots) * kRingSlotF4, L,
                     __uint_as_float(bl[cb].b[5].w));
        EncDw nxt = cur;
        if (kb + 1 < kKb16Split) {
            // block kb+1 landed; younger: blocks kb+2 and kb+3 (12), near the end the one
            // block still to come (6) or nothing -- the loop issues no other vector memory
            vm_wait(kb + 3 < kKb16Split ? 12 : (kb + 2 < kKb16Split ? 6 : 0));
            const f4* slot = ring + ((kb + 1) % kRingSlots) * kRingSlotF4 + L.lane_u;
#pragma unroll
            for (int i = 0; i < 6; i++) bl[nb].b[i] = __builtin_bit_cast(u4, slot[i * 64]);
            nxt = encs_bytes(rx, ry, kb + 1, L.half);
        }
        u4 ax = bytes_to_bf16x8(cur.x0, cur.x1), ay = bytes_to_bf16x8(cur.y0, cur.y1);
        if (kb == kKb16Split - 1 && L.half) {   // features 792..799 are not map bytes
            ax = u4{0u, 0u, 0u, 0u};
            ay = u4{0u, 0u, 0u, 0u};
        }
        encs_mma<ONE>(acc, ax, ay, bl[cb]);
        cur = nxt;
        __builtin_amdgcn_sched_barrier(0);
    }
    // tail floats 8t + 4*half + j of the record (51 valid, then zeros) on the fp32 MFMA
    const float* fx = reinterpret_cast<const float*>(rx) + (CFP_OBS_MAP / 4) + 4 * L.half;
    const float* fy = reinterpret_cast<const float*>(ry) + (CFP_OBS_MAP / 4) + 4 * L.half;
#pragma unroll
    for (int t = 0; t < 7; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float x = fx[8 * t + j], y = fy[8 * t + j];
            acc[0] = mfma(x, tb0[t][j], acc[0]);
            acc[1] = mfma(x, tb1[t][j], acc[1]);
            if (!ONE) {
                acc[2] = mfma(y, tb0[t][j], acc[2]);
                acc[3] = mfma(y, tb1[t][j], acc[3]);
            }
        }
    }
}

// ---- classic-game encoder for a pair of tiles (64 envs) ----------------------------
// encode_obs_kernel (craftax_classic.cu:1714-1751): h0 = b_enc + W_enc^T x with
// x = 63 view cells x (one-hot of 17 block ids + 4 mob bits) followed by 22 scalar
// features.  The 1323 cell features are 0/1, exact in bf16, so they run like the
// full game's byte features: three bf16 MFMAs per product against the three-term
// split of the fp32 weights, weights streamed through the ring.  The A operand
// needs no arithmetic: the pair's 64 x 1323 feature bits are packed once into
// LDS (cell c = 21 bits at bit 21c), a lane's eight features of a K block are one
// byte of that, and a 256-entry LDS table turns the byte into eight bf16 0/1.
// The 22 scalar features (inventory and intrinsics / 10, direction one-hot, light,
// sleeping) follow on the fp32 MFMA (3 K blocks of 8).  Block ids must be 0..16.
constexpr int kClsEnvs = 2 * kTileEnvs;
// byte layout inside the (not yet used) x tiles
constexpr int kClsOffRecY = kTileEnvs * CFP_CLASSIC_REC_BYTES;
constexpr int kClsOffBits = ClsLayout<kClsEnvs>::offBits;
constexpr int kClsOffLut = ClsLayout<kClsEnvs>::offLut;
constexpr int kClsOffSv = ClsLayout<kClsEnvs>::offSv;
static_assert(kClsOffBits == 2 * kClsOffRecY, "the pair's records lie back to back");
static_assert(ClsLayout<kClsEnvs>::end <= 2 * LDS_FLOATS * 4, "classic tables fit the x tiles");

__device__ __forceinline__ void classic_encoder_gemm(const FwdArgs& a, const uint8_t* base,
                                                     f4* ring, const Lane& L, f16v (&acc)[4]) {
    const uint8_t* bx = base + kClsOffBits + L.l32 * (kClsBitRow * 4) + L.half;
    const uint8_t* by = bx + kTileEnvs * (kClsBitRow * 4);
    const u4* lut = reinterpret_cast<const u4*>(base + kClsOffLut);
    // the scalar features' weights first: older than every ring request, used last
    const f4* wq = a.we_pk + (size_t)(L.wave * 2) * 64;
    constexpr int KB8_STRIDE = 4 * 2 * 64;
    f4 tb0[kClsTailKb], tb1[kClsTailKb];
#pragma unroll
    for (int t = 0; t < kClsTailKb; t++) {
        const f4* p = wq + (size_t)t * KB8_STRIDE;
        tb0[t] = p[L.lane_u];
        tb1[t] = (p + 64)[L.lane_u];
    }
    asm volatile("" ::: "memory");
    const f4* wp = reinterpret_cast<const f4*>(a.we_s3) + (size_t)(L.wave * 6) * 64;
    ring_preload(ring, wp, L);
    // eight features of K block kb for this lane = byte 2*kb + half of the env's row
    uint32_t mx = bx[0], my = by[0];
    u4 ax = lut[mx], ay = lut[my];
    mx = bx[2];
    my = by[2];
    EncS bl[2];
    vm_wait(12);   // block 0 landed; younger: the preload's blocks 1 and 2
#pragma unroll
    for (int i = 0; i < 6; i++) bl[0].b[i] = __builtin_bit_cast(u4, ring[i * 64 + L.lane_u]);
#pragma unroll
    for (int kb = 0; kb < kClsKb16; kb++) {
        const int cb = kb & 1, nb = cb ^ 1;
        if (kb + 3 < kClsKb16)
            ring_dma(wp, kb + 3, ring + (kb % kRingSlots) * kRingSlotF4, L,
                     __uint_as_float(bl[cb].b[5].w));
        u4 nx = ax, ny = ay;
        if (kb + 1 < kClsKb16) {
            // block kb+1 landed; younger: the blocks requested since (12, 6 or none)
            vm_wait(kb + 3 < kClsKb16 ? 12 : (kb + 2 < kClsKb16 ? 6 : 0));
            const f4* slot = ring + ((kb + 1) % kRingSlots) * kRingSlotF4 + L.lane_u;
#pragma unroll
            for (int i = 0; i < 6; i++) bl[nb].b[i] = __builtin_bit_cast(u4, slot[i * 64]);
            nx = lut[mx];          // block kb+1
            ny = lut[my];
            if (kb + 2 < kClsKb16) {
                mx = bx[2 * (kb + 2)];
                my = by[2 * (kb + 2)];
            }
        }
        encs_mma(acc, ax, ay, bl[cb]);
        ax = nx;
        ay = ny;
        __builtin_amdgcn_sched_barrier(0);
    }
    const float* fx = reinterpret_cast<const float*>(base + kClsOffSv) + L.l32 * kClsSv + 4 * L.half;
    const float* fy = fx + kTileEnvs * kClsSv;
#pragma unroll
    for (int t = 0; t < kClsTailKb; t++) {
        const f4 x = *reinterpret_cast<const f4*>(fx + 8 * t);
        const f4 y = *reinterpret_cast<const f4*>(fy + 8 * t);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc[0] = mfma(x[j], tb0[t][j], acc[0]);
            acc[1] = mfma(x[j], tb1[t][j], acc[1]);
            acc[2] = mfma(y[j], tb0[t][j], acc[2]);
            acc[3] = mfma(y[j], tb1[t][j], acc[3]);
        }
    }
}

// DO_K: accN[6] += x_K . W_l^T for the tile whose x tile is `xs4K`.  On entry the
//       ring holds (has been asked for) K blocks 0..2, requested by ring_preload,
//       followed, when DO_E (or PX = 32), by the 32 loads of state_load and nothing else.
//       While block kb is multiplied, block kb+1 is read from its slot into the
//       other half of bl[2][6] and block kb+3 is requested into the slot block kb
//       was read from one block earlier: LDS latency is covered by one block
//       (1536 matrix-pipe cycles), L2 latency by two.
// DO_E: the gate/blend epilogue of the OTHER tile from accO[6], one element next
//       to each K block: element kb's ~35 vector instructions, its two LDS
//       accesses and its state / r_state stores issue in the shadow of the 24
//       MFMAs.  The block is branch-free (a branch would split it and leave the
//       epilogue behind the MFMAs).  The state values were requested before the
//       phase (st[32]); in-loop state loads would sit in front of the weight
//       requests in the in-order return queue with their HBM latency.
template <bool DO_K, bool DO_E, int MODE, int PX = 0>   // PX: loads that follow the preload when !DO_E
__device__ __forceinline__ void gru_phase(f16v (&accN)[6], const f16v (&accO)[6], f4* ring,
                                          const f4* xs4K, const f4* wp, float* xsE,
                                          const StateIO& io, const float (&st)[32],
                                          const Lane& L) {
    // Vector-memory operations complete in issue order, so "block b has landed"
    // is "at most N operations are outstanding", N = those issued after b's six:
    // the later requests, the S stores each epilogue block issues, and in the
    // first blocks the P state loads that follow the preload.
    constexpr int S = !DO_E ? 0 : (MODE == kModeTrain ? 4 : (MODE == kModeRecord ? 2 : 1));
    constexpr int P = DO_E ? 32 : PX;
    f4 aq[2];
    f4 bl[2][6];
    if (DO_K) {
        aq[0] = xs4K[L.arow4];
        vm_wait(12 + P);   // block 0 landed; blocks 1, 2 and the state loads may be in flight
#pragma unroll
        for (int t = 0; t < 6; t++) bl[0][t] = ring[t * 64 + L.lane_u];
    }
#pragma unroll
    for (int kb = 0; kb < kKbHid; kb++) {
        const int cb = kb & 1, nb = cb ^ 1;
        float* xp = nullptr;
        float xv = 0.0f;
        if (DO_E) {
            xp = xsE + (acc_row(kb % 16) + 4 * L.half) * XS + L.wave * 64 + (kb / 16) * 32 + L.l32;
            xv = *xp;
        }
        if (DO_K) {
            if (kb + 3 < kKbHid)
                ring_dma(wp, kb + 3, ring + (kb % kRingSlots) * kRingSlotF4, L, bl[cb][5][3]);
            if (kb + 1 < kKbHid) {
                // block kb+1 landed?  younger: blocks kb+2, kb+3 and what lies between
                if (kb + 3 < kKbHid) vm_wait(12 + (kb >= 2 ? 2 * S : P + kb * S));
                else if (kb + 2 < kKbHid) vm_wait(6 + 2 * S);
                else vm_wait(2 * S);
                const f4* slot = ring + ((kb + 1) % kRingSlots) * kRingSlotF4 + L.lane_u;
#pragma unroll
                for (int t = 0; t < 6; t++) bl[nb][t] = slot[t * 64];
                aq[nb] = xs4K[L.arow4 + 2 * (kb + 1)];
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int t = 0; t < 6; t++)
                    accN[t] = mfma(aq[cb][j], bl[cb][t][j], accN[t]);
        }
        if (DO_E) {
            const int ut = kb / 16, r = kb % 16;
            const float s = (MODE != kModeTrain && ((io.tmask >> r) & 1u)) ? 0.0f : st[kb];
            if (MODE == kModeRecord)
                __builtin_nontemporal_store(s, (io.rs_base + st_off(kb)) + L.loff);
            const float zh = accO[0 + ut][r];
            const float zg = accO[2 + ut][r];
            const float zp = accO[4 + ut][r];
            if (MODE == kModeTrain) {
                float* pp = io.pre_base + (acc_row(r) * CFP_GRU + ut * 32);
                __builtin_nontemporal_store(zh, pp + L.loff3);
                __builtin_nontemporal_store(zg, (pp + CFP_HIDDEN) + L.loff3);
                __builtin_nontemporal_store(zp, (pp + 2 * CFP_HIDDEN) + L.loff3);
            }
            const float sg = sigmoid_fast(zg);
            float sh = sigmoid_fast(zh);
            asm volatile("" : "+v"(sh));   // keep g(zh) a select, not a branch
            const float gh = zh >= 0.0f ? zh + 0.5f : sh;
            const float out = s + sg * (gh - s);
            const float p = sigmoid_fast(zp);
            const float hn = p * out + (1.0f - p) * xv;
            *xp = hn;
            if (MODE == kModeTrain)
                __builtin_nontemporal_store(hn, (io.rs_base + st_off(kb)) + L.loff);
            else
                __builtin_nontemporal_store(out, (io.st_base + st_off(kb)) + L.loff);
        }
        // Issue order of the block: the epilogue's vector instructions two per MFMA.
        if (DO_K) {
#pragma unroll
            for (int q = 0; q < 24; q++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                  // one MFMA
                if (q == 0 && DO_E) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // x value
                // next block's six weight fragments and x fragment, back to back
                if (q == 1) __builtin_amdgcn_sched_group_barrier(0x100, 7, 0);
                if (DO_E) {
                    __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);              // two VALU
                    if (q == 21) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                    if (q == 22)
                        __builtin_amdgcn_sched_group_barrier(
                            0x040, MODE == kModeTrain ? 4 : (MODE == kModeRecord ? 2 : 1), 0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

}  // namespace

// SINGLE: one tile per workgroup instead of a pair, for batches of at most one tile per
// CU (a rollout of a few thousand envs): twice as many CUs work, and a layer is its K
// phase followed by its epilogue instead of the two tiles' interleave.  Encoder and
// heads still run their two-tile code with an all-zero second tile.
template <int VARIANT, int MODE, bool SINGLE>
__global__ __launch_bounds__(kFwdThreads, 1) void k_policy_forward(FwdArgs a) {
    __shared__ __attribute__((aligned(16))) float lds_all[2][LDS_FLOATS];
    __shared__ __attribute__((aligned(16))) float red_all[2][kRedFloats];
    __shared__ float term_all[2][kTileEnvs];
    // the per-wave weight rings (encoder and MinGRU phases), 72 KiB
    __shared__ __attribute__((aligned(16))) f4 aux[kRingF4];
    // classic game: record bytes and the encoder's tables sit in the x tiles until the
    // encoder's result replaces them
    constexpr int kCrecBytes = kTileEnvs * CFP_CLASSIC_REC_BYTES;
    static_assert(kCrecBytes == kClsOffRecY, "record layout of the classic tables");
    uint8_t* const cbase = reinterpret_cast<uint8_t*>(&lds_all[0][0]);
    uint8_t* const crec_all[2] = {cbase, cbase + kClsOffRecY};

    // rollout step in one launch: the draw's offset, requested before anything else (older
    // than every weight request, so no wait of the ring protocol depends on it)
    uint64_t draw_step = 0;
    if (SINGLE && MODE == kModeRecord && a.s_act) draw_step = *a.s_step;
    const int tiles = a.n / kTileEnvs;
    constexpr int TS = SINGLE ? 1 : 2;   // tiles per unit of work ("pair")
    const int pairs = (tiles + TS - 1) / TS;
    const bool classic = VARIANT == 1 && a.rec;
    const bool full_rec = VARIANT == 0 && a.rec;

    // Full-game records travel one pair ahead through registers: requested while
    // the previous pair runs its last epilogue, written into LDS at the pair's start.
    RecRegs pre[2];
    // tile -> its records / terminal flags.  Window recompute: tile = 32 columns of
    // one step t (the minibatch is a multiple of 32 envs), records in the slab row.
    auto slab_env = [&](size_t c0) {   // first env of the tile as an index into [T][n_all]
        const size_t tr = c0 / (size_t)a.tr_mb;
        return ((size_t)a.tr_t0 + tr) * a.tr_n_all + a.tr_env_start + (c0 - tr * a.tr_mb);
    };
    auto rec_of = [&](int tile) {
        const size_t c0 = (size_t)tile * kTileEnvs;
        return a.rec + (MODE == kModeTrain ? slab_env(c0) : c0) * CFP_REC_BYTES;
    };
    auto term_of = [&](int tile) -> const float* {
        return (MODE != kModeTrain && a.terminals) ? a.terminals + (size_t)tile * kTileEnvs
                                                   : nullptr;
    };
    if (full_rec && (int)blockIdx.x < pairs) {
        const int tid0 = threadIdx.x;
        rec_fetch(rec_of(TS * blockIdx.x), term_of(TS * blockIdx.x), pre[0], tid0);
        if (!SINGLE && 2 * (int)blockIdx.x + 1 < tiles)
            rec_fetch(rec_of(2 * blockIdx.x + 1), term_of(2 * blockIdx.x + 1), pre[1], tid0);
    }
    for (int pair = blockIdx.x; pair < pairs; pair += gridDim.x) {
        // Lane constants are re-derived per pair from an opaque copy of the thread
        // index: hoisted out of this loop, the dozens of per-lane addresses they
        // feed would stay live across every phase and spill.
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        Lane L;
        L.lane_u = (unsigned)(tid & 63);
        L.half = (tid & 63) >> 5;
        L.l32 = tid & 31;
        L.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        L.arow4 = L.l32 * XS4 + L.half;
        L.loff = (unsigned)((4 * L.half) * CFP_HIDDEN + L.l32);
        L.loff3 = (unsigned)((4 * L.half) * CFP_GRU + L.l32);
        const int nt = L.wave & 1;   // head: row tile
        const int kh = L.wave >> 1;  // head: K half
        // tile X = 2*pair always exists; tile Y may be past the end (odd tile count)
        const bool hasY = !SINGLE && 2 * pair + 1 < tiles;
        size_t e0[2] = {(size_t)(TS * pair) * kTileEnvs, (size_t)(TS * pair + 1) * kTileEnvs};

        // ---- stage both tiles (a missing Y is a zero tile that is computed but
        // never read from or written to the caller's buffers) --------------------
        if (full_rec) rec_scatter(pre[0], lds_all[0], term_all[0], tid);
        else stage_tile<VARIANT>(a, e0[0], lds_all[0], crec_all[0], term_all[0], tid);
        if (hasY) {
            if (full_rec) rec_scatter(pre[1], lds_all[1], term_all[1], tid);
            else stage_tile<VARIANT>(a, e0[1], lds_all[1], crec_all[1], term_all[1], tid);
        } else {
            for (int i = tid; i < LDS_FLOATS; i += kFwdThreads) lds_all[1][i] = 0.0f;
            if (tid < kTileEnvs) term_all[1][tid] = 0.0f;
            if (VARIANT == 1)
                for (int i = tid; i < kCrecBytes; i += kFwdThreads) crec_all[1][i] = 0;
        }
        __syncthreads();

        unsigned tmask[2] = {0u, 0u};
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (term_all[s][acc_row(r) + 4 * L.half] != 0.0f) tmask[s] |= 1u << r;

        // ---- encoders ----------------------------------------------------------
        if (classic || full_rec) {
            f16v eacc[4];
#pragma unroll
            for (int t = 0; t < 4; t++) eacc[t] = zero16();
            f4* const ring = aux + L.wave * (kRingSlots * kRingSlotF4);
            if (classic) {
                classic_prepare<kClsEnvs>(cbase, tid);
                classic_encoder_gemm(a, cbase, ring, L, eacc);
            } else {
                encoder_gemm_split_ring<SINGLE>(a, lds_all[0], lds_all[1], ring, L, eacc);
            }
            __syncthreads();   // every wave is done with the record bytes / tables
#pragma unroll
            for (int s = 0; s < (SINGLE ? 1 : 2); s++)
#pragma unroll
                for (int ut = 0; ut < 2; ut++) {
                    const float bias = a.b_enc[L.wave * 64 + ut * 32 + L.l32];
                    float* xrow = lds_all[s] + (4 * L.half) * XS + L.wave * 64 + ut * 32 + L.l32;
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        xrow[acc_row(r) * XS] = eacc[2 * s + ut][r] + bias;
                }
        }
        __syncthreads();
        if (a.rec && a.h_enc_out) {
            copy_tile_out(lds_all[0], a.h_enc_out + e0[0] * CFP_HIDDEN, tid);
            if (hasY) copy_tile_out(lds_all[1], a.h_enc_out + e0[1] * CFP_HIDDEN, tid);
        }

        // next pair's records -> registers (no-op past the last pair of this workgroup)
        auto fetch_next = [&]() {
            const int np = pair + (int)gridDim.x;
            if (np < pairs) {
                rec_fetch(rec_of(TS * np), term_of(TS * np), pre[0], tid);
                if (!SINGLE && 2 * np + 1 < tiles)
                    rec_fetch(rec_of(2 * np + 1), term_of(2 * np + 1), pre[1], tid);
            }
        };
        if (full_rec && a.layers == 0) fetch_next();

        // ---- MinGRU layers, the two tiles software-pipelined -------------------------
        // phase q = 0 .. 2L:  K(tile q&1, layer q/2)  woven with  epi(tile (q-1)&1, layer (q-1)/2)
        // Before the barrier that ends phase q, the first two weight blocks and
        // the state of phase q+1 are requested, in that order.
        if (a.layers > 0) {
            f16v accO[6], accN[6];
            float st[32];
            f4* const bq = aux + L.wave * (kRingSlots * kRingSlotF4);   // this wave's ring
            const size_t wl = kGruPackFloats / 4;   // f4 per layer of the mirror
            const f4* wp0 = a.wg_pk + (size_t)(L.wave * 6) * 64;
            auto state_io = [&](int q) {
                const int s = (q - 1) & 1, l = (q - 1) >> 1;
                StateIO c;
                c.pre_base = nullptr;
                if (MODE == kModeTrain) {
                    // stored state of (t, layer l, env) -> this layer's pre / output tiles
                    const size_t se = slab_env(e0[s]);
                    const size_t tt = se / a.tr_n_all, ee = se - tt * a.tr_n_all;
                    c.st_base = a.state + ((tt * a.layers + l) * a.tr_n_all + ee) * CFP_HIDDEN +
                                L.wave * 64;
                    c.rs_base = a.tr_x[l + 1] + e0[s] * CFP_HIDDEN + L.wave * 64;
                    c.pre_base = a.tr_pre[l] + e0[s] * CFP_GRU + L.wave * 64;
                    if (s == 1 && !hasY) {
                        c.st_base = c.rs_base = g_void_tile + L.wave * 64;
                        c.pre_base = g_void_pre + L.wave * 64;
                    }
                } else if (s == 0 || hasY) {
                    const size_t off = (size_t)l * a.layer_stride + e0[s] * CFP_HIDDEN + L.wave * 64;
                    c.st_base = a.state + off;
                    c.rs_base = MODE == kModeRecord ? a.r_state + off : nullptr;
                } else {
                    c.st_base = g_void_tile + L.wave * 64;
                    c.rs_base = g_void_tile + L.wave * 64;
                }
                c.tmask = tmask[s];
                return c;
            };
            const int Q = 2 * a.layers;
            if (SINGLE) {
                // one tile: K phase, then its epilogue, layer by layer; the state is
                // requested right behind the first weight blocks, as in the pair schedule
                if (full_rec) fetch_next();
#pragma unroll 1
                for (int l = 0; l < a.layers; l++) {
                    const StateIO io1 = state_io(2 * l + 1);
                    ring_preload(bq, wp0 + (size_t)l * wl, L);
                    state_load(io1, st, L);   // behind the weights: lands under the K phase
#pragma unroll
                    for (int t = 0; t < 6; t++) accO[t] = zero16();
                    gru_phase<true, false, MODE, 32>(accO, accO, bq,
                                                 reinterpret_cast<const f4*>(lds_all[0]),
                                                 wp0 + (size_t)l * wl, nullptr, io1, st, L);
                    __syncthreads();   // every wave has read the layer input
                    gru_phase<false, true, MODE>(accN, accO, bq, nullptr, nullptr, lds_all[0], io1,
                                                 st, L);
                    __syncthreads();
                }
            } else {
#pragma unroll
            for (int t = 0; t < 6; t++) accO[t] = zero16();
            ring_preload(bq, wp0, L);
            StateIO io = state_io(1);
            gru_phase<true, false, MODE>(accO, accO, bq, reinterpret_cast<const f4*>(lds_all[0]),
                                           wp0, nullptr, io, st, L);
            ring_preload(bq, wp0, L);
            state_load(io, st, L);
            __syncthreads();
#pragma unroll 1
            for (int q = 1; q < Q; q++) {
#pragma unroll
                for (int t = 0; t < 6; t++) accN[t] = zero16();
                gru_phase<true, true, MODE>(accN, accO, bq,
                                              reinterpret_cast<const f4*>(lds_all[q & 1]),
                                              wp0 + (size_t)(q >> 1) * wl, lds_all[(q - 1) & 1],
                                              io, st, L);
                io = state_io(q + 1);
                if (q + 1 < Q) ring_preload(bq, wp0 + (size_t)((q + 1) >> 1) * wl, L);
                state_load(io, st, L);
                __syncthreads();
#pragma unroll
                for (int t = 0; t < 6; t++) accO[t] = accN[t];
            }
            if (full_rec) fetch_next();
            gru_phase<false, true, MODE>(accN, accO, bq, nullptr, nullptr, lds_all[(Q - 1) & 1],
                                           io, st, L);
            __syncthreads();
            }
            if (a.h3_out) {
                copy_tile_out(lds_all[0], a.h3_out + e0[0] * CFP_HIDDEN, tid);
                if (hasY) copy_tile_out(lds_all[1], a.h3_out + e0[1] * CFP_HIDDEN, tid);
            }
        }

        // ---- heads: wave = (row tile nt, K half kh), both tiles -----------------------
        if (a.do_head) {
            // both tiles share each weight fragment; their MFMAs alternate, so no MFMA
            // waits for the one before it on the same accumulator
            f16v hacc[2] = {zero16(), zero16()};
            const f4* wp = a.wav_pk + (size_t)nt * 64;
            const f4* xsX = reinterpret_cast<const f4*>(lds_all[0]);
            const f4* xsY = reinterpret_cast<const f4*>(lds_all[1]);
            f4 hb[kKbHid / 2];
#pragma unroll
            for (int i = 0; i < kKbHid / 2; i++)
                hb[i] = (wp + (size_t)(kh * (kKbHid / 2) + i) * 128)[L.lane_u];
#pragma unroll
            for (int i = 0; i < kKbHid / 2; i++) {
                const int kb = kh * (kKbHid / 2) + i;
                const f4 ax = xsX[L.arow4 + 2 * kb];
                const f4 ay = xsY[L.arow4 + 2 * kb];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    hacc[0] = mfma(ax[j], hb[i][j], hacc[0]);
                    if (!SINGLE) hacc[1] = mfma(ay[j], hb[i][j], hacc[1]);
                }
            }
            if (kh == 1) {
#pragma unroll
                for (int s = 0; s < (SINGLE ? 1 : 2); s++) {
                    float* red = red_all[s] + (nt * 16) * 64 + L.lane_u;
#pragma unroll
                    for (int r = 0; r < 16; r++) red[r * 64] = hacc[s][r];
                }
            }
            __syncthreads();
            if (kh == 0) {
                const int arow = nt * 32 + L.l32;
                const int avs = a.actions + 1;     // 44, or 18 for the classic game
                if (arow < avs) {
                    const float bias = arow < a.actions ? a.b_a[arow] : a.b_v[0];
#pragma unroll
                    for (int s = 0; s < 2; s++) {
                        if (s == 1 && !hasY) continue;
                        const float* red = red_all[s] + (nt * 16) * 64 + L.lane_u;
                        float* av_base = a.av_out + e0[s] * avs;
                        const int aoff = (4 * L.half) * avs + arow;
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const float v = hacc[s][r] + red[r * 64] + bias;
                            (av_base + acc_row(r) * avs)[aoff] = v;
                            // rollout step in one launch: the rows stay in LDS for the draw
                            // (the x tiles are free: every wave is past its head MFMAs)
                            if (SINGLE && MODE == kModeRecord && a.s_act)
                                lds_all[0][(acc_row(r) + 4 * L.half) * avs + arow] = v;
                        }
                    }
                }
            }
            // ---- the draw behind the heads (one tile per workgroup, recording mode): sixteen
            // lanes per env run the sampler's code (sample_row.h: same operations in the same
            // order as k_value_sample), lanes 0 and 1 of a group each finish one of the tile's
            // two halves, and the last workgroup bumps the step counter
            if (SINGLE && MODE == kModeRecord && a.s_act) {   // uniform over the launch
                __syncthreads();
                const int sub = tid % kSampleLanes, grp = tid / kSampleLanes;   // 16 groups
                const int avs = a.actions + 1;
                float mx[2];
#pragma unroll
                for (int part = 0; part < 2; part++) {
                    const int env = grp + 16 * part;
                    mx[part] = sample_spread(lds_all[0] + env * avs, lds_all[1] + env * kMaxActions,
                                             a.actions, sub, true);
                }
                __syncthreads();
                if (sub < 2) {
                    const int env = grp + 16 * sub;
                    sample_draw<CFP_ACTIONS>(lds_all[0] + env * avs, lds_all[1] + env * kMaxActions,
                                             sub == 0 ? mx[0] : mx[1], a.actions, (int)e0[0] + env,
                                             a.s_seed, draw_step, a.s_env_actions, a.s_act, a.s_logp,
                                             a.s_value);
                }
                __syncthreads();
                if (tid == 0) bump_by_last_group(a.s_ticket, a.s_step, gridDim.x);
            }
        }
        __syncthreads();   // LDS tiles and partials are free for the next pair
    }
}

static int num_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
            v > 0)
            cus = v;
        else
            cus = 256;
    }
    return cus;
}

// Does launch_forward run the instantiation that also draws the actions (FwdArgs::s_act)?
bool forward_draws(const FwdArgs& a) {
    const int tiles = a.n / kTileEnvs;
    return a.s_act && a.s_logp && a.s_step && a.s_ticket && a.variant == 0 && !a.train &&
           !a.bf16 && a.rec && a.r_state && a.do_head && a.layers > 0 && a.n % kTileEnvs == 0 &&
           tiles > 1 && tiles <= num_cus();
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
    CFP_REQUIRE(!a.tr_bf16 || (a.bf16 && a.train),
                "bf16 storage of the window recompute needs the bf16-input kernel");
    if (a.bf16) return launch_forward_bf16(a, st);
    CFP_REQUIRE(!(a.rs_bf16 && (a.r_state || a.train)),
                "a bf16 state slab is written and read by the bf16-input forward only "
                "(cfp_policy_set_gemm_bf16 / cfp_set_gemm_bf16)");
    if (forward_t16_ok(a)) return launch_forward_t16(a, st);
    // persistent: one workgroup per CU, each walking tile pairs round-robin; a full-game
    // batch of at most one tile per CU runs one tile per workgroup instead
    const int tiles = a.n / kTileEnvs;
    const int pairs = (tiles + 1) / 2;
    const int grid = pairs < num_cus() ? pairs : num_cus();
    const dim3 g(grid), b(kFwdThreads);
    const bool single = a.variant == 0 && !a.train && tiles <= num_cus() && tiles > 1;
    CFP_REQUIRE(!a.s_act || forward_draws(a),
                "the draw behind the heads needs full-game records, r_state and one tile per CU");
    if (a.train) {
        CFP_REQUIRE(a.variant == 0 && a.rec && a.state && a.layers > 0 && !a.r_state &&
                        a.tr_mb > 0 && a.tr_mb % kTileEnvs == 0 && a.h_enc_out == a.tr_x[0],
                    "window recompute: bad arguments");
        hipLaunchKernelGGL((k_policy_forward<0, kModeTrain, false>), g, b, 0, st, a);
    } else if (a.variant == 1) {
        if (a.r_state) hipLaunchKernelGGL((k_policy_forward<1, kModeRecord, false>), g, b, 0, st, a);
        else hipLaunchKernelGGL((k_policy_forward<1, kModePlain, false>), g, b, 0, st, a);
    } else if (single) {
        const dim3 g1(tiles);
        if (a.r_state) hipLaunchKernelGGL((k_policy_forward<0, kModeRecord, true>), g1, b, 0, st, a);
        else hipLaunchKernelGGL((k_policy_forward<0, kModePlain, true>), g1, b, 0, st, a);
    } else {
        if (a.r_state) hipLaunchKernelGGL((k_policy_forward<0, kModeRecord, false>), g, b, 0, st, a);
        else hipLaunchKernelGGL((k_policy_forward<0, kModePlain, false>), g, b, 0, st, a);
    }
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

// Map rows of W_enc as three bf16 terms per weight, MFMA 32x32x16 order: one
// 16-byte element (eight bf16) per lane, K block of 16 and term; lane l carries
// k = 16*kb + 8*(l/32) + j of column l%32 of its 32-wide tile.  Features past the
// map (the fp32 tail runs on the fp32 mirror) carry zeros.
__global__ void k_pack_enc_split(const float* __restrict__ W_enc, __bf16* __restrict__ out,
                                 int total, int nfeat) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int j = idx & 7, lane = (idx >> 3) & 63, q = idx >> 9;
    int s = q % 3, ut = (q / 3) & 1, wave = (q / 6) & 3, kb = q / 24;
    int unit = wave * 64 + ut * 32 + (lane & 31);
    int f = 16 * kb + 8 * (lane >> 5) + j;
    const float w = f < nfeat ? W_enc[(size_t)f * CFP_HIDDEN + unit] : 0.0f;
    const __bf16 hi = (__bf16)w;
    const float r1 = w - (float)hi;
    const __bf16 mid = (__bf16)r1;
    const __bf16 lo = (__bf16)(r1 - (float)mid);
    out[idx] = s == 0 ? hi : (s == 1 ? mid : lo);
}

int launch_pack_enc_split(const float* params, int layers, int variant, uint16_t* we_s3,
                          hipStream_t st) {
    const Arena ar = arena_of(variant, layers);
    // full game: the 792 map bytes; classic: the 1323 cell features
    const int nfeat = variant == 0 ? CFP_OBS_MAP : kClsBits;
    const int total = (variant == 0 ? kKb16Split : kClsKb16) * 4 * 6 * 64 * 8;
    hipLaunchKernelGGL(k_pack_enc_split, dim3((total + 255) / 256), dim3(256), 0, st,
                       params + ar.w_enc, reinterpret_cast<__bf16*>(we_s3), total, nfeat);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

// Classic game: the 22 scalar features' rows of W_enc (features 1323..1344, padded to
// 24) as three fp32 K blocks in the order of k_pack_enc.
__global__ void k_pack_enc_classic_tail(const float* __restrict__ W_enc,
                                        float* __restrict__ out) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= kClsTailKb * 2048) return;
    int j = idx & 3, lane = (idx >> 2) & 63, ut = (idx >> 8) & 1,
        wave = (idx >> 9) & 3, kb = idx >> 11;
    int unit = wave * 64 + ut * 32 + (lane & 31);
    int f = kClsBits + kKBlock * kb + 4 * (lane >> 5) + j;
    out[idx] = f < CFP_CLASSIC_OBS ? W_enc[(size_t)f * CFP_HIDDEN + unit] : 0.0f;
}

int launch_pack_weights(const float* params, int layers, int variant, float* we_pk,
                        float* wg_pk, float* wav_pk, hipStream_t st) {
    const Arena ar = arena_of(variant, layers);
    if (variant == 0) {
        const int enc_total = (kKbEnc + kEncPadBlocks) * 2048;
        hipLaunchKernelGGL(k_pack_enc, dim3((enc_total + 255) / 256), dim3(256), 0,
                           st, params + ar.w_enc, we_pk, enc_total);
    } else {
        hipLaunchKernelGGL(k_pack_enc_classic_tail, dim3((kClsTailKb * 2048 + 255) / 256),
                           dim3(256), 0, st, params + ar.w_enc, we_pk);
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
