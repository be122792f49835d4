// Tile-level device helpers shared by the fp32 and bf16 fused forward kernels:
// LDS tile geometry, record staging, the classic-game gather encoder, tile
// copies.  Internal to the library (included by the .hip files only).
#pragma once

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
    for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads)
        d4[i] = xs4[(i >> 6) * XS4 + (i & 63)];
}

// Stage one tile's inputs into LDS: the records (full game: contiguous 16-byte
// loads, rows re-strided to an odd dword count so that 32 envs reading the same
// feature hit 32 different banks; classic: a plain copy) or the given layer-0
// input, plus the terminal flags.
template <int VARIANT>
__device__ __forceinline__ void stage_tile(const FwdArgs& a, size_t e0, float* lds,
                                           uint8_t* crec, float* term_s, int tid) {
    if (tid < kTileEnvs)
        term_s[tid] = a.terminals ? a.terminals[e0 + tid] : 0.0f;
    if (VARIANT == 1 && a.rec) {
        constexpr int TILE_V4 = kTileEnvs * CFP_CLASSIC_REC_BYTES / 16;   // 296
        const u4* src = reinterpret_cast<const u4*>(a.rec + e0 * CFP_CLASSIC_REC_BYTES);
        u4* dst = reinterpret_cast<u4*>(crec);
        for (int i = tid; i < TILE_V4; i += kFwdThreads) dst[i] = src[i];
    } else if (VARIANT == 0 && a.rec) {
        uint32_t* rs = reinterpret_cast<uint32_t*>(lds);
        const u4* src = reinterpret_cast<const u4*>(a.rec + e0 * CFP_REC_BYTES);
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
    } else {
        const f4* src = reinterpret_cast<const f4*>(a.x0 + e0 * CFP_HIDDEN);
        f4* xs4 = reinterpret_cast<f4*>(lds);
        if (a.x0_add_bias) {   // k_add_bias (craftax_full.cu:10056) folded into the staging
            const f4* b4 = reinterpret_cast<const f4*>(a.b_enc);
            for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads) {
                const f4 v = src[i], b = b4[i & 63];
                xs4[(i >> 6) * XS4 + (i & 63)] = f4{v[0] + b[0], v[1] + b[1], v[2] + b[2], v[3] + b[3]};
            }
        } else {
            for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads)
                xs4[(i >> 6) * XS4 + (i & 63)] = src[i];
        }
    }
}

// Full-game record staging split in two so that the HBM latency of the next
// pair's records can be spent under the current pair's last phases: rec_fetch
// requests a tile's 31 872 bytes (8 x 16 bytes per thread) into registers,
// rec_scatter writes them into the LDS rows (stride RS dwords) later.
constexpr int kRecV4PerThread = (TILE_REC_V4 + kFwdThreads - 1) / kFwdThreads;   // 8

struct RecRegs {
    u4 v[kRecV4PerThread];
    float term;   // terminal flag of env `tid` of the tile (threads 0..31)
};

__device__ __forceinline__ void rec_fetch(const uint8_t* rec_tile, const float* term_tile,
                                          RecRegs& r, int tid) {
    const u4* src = reinterpret_cast<const u4*>(rec_tile);
#pragma unroll
    for (int j = 0; j < kRecV4PerThread; j++) {
        const int i = tid + kFwdThreads * j;
        if (i < TILE_REC_V4) r.v[j] = __builtin_nontemporal_load(src + i);
    }
    r.term = (tid < kTileEnvs && term_tile) ? term_tile[tid] : 0.0f;
}

__device__ __forceinline__ void rec_scatter(const RecRegs& r, float* lds, float* term_s, int tid) {
    uint32_t* rs = reinterpret_cast<uint32_t*>(lds);
#pragma unroll
    for (int j = 0; j < kRecV4PerThread; j++) {
        const int i = tid + kFwdThreads * j;
        if (i < TILE_REC_V4) {
            const uint32_t w[4] = {r.v[j].x, r.v[j].y, r.v[j].z, r.v[j].w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int d = 4 * i + c;
                const int row = d / REC_DW;
                const int col = d - row * REC_DW;
                rs[row * RS + col] = w[c];
            }
        }
    }
    if (tid < kTileEnvs * (RS - REC_DW)) {
        const int row = tid / (RS - REC_DW);
        const int c = tid - row * (RS - REC_DW);
        rs[row * RS + REC_DW + c] = 0u;   // features 843..847 read as 0.0f
    }
    if (tid < kTileEnvs) term_s[tid] = r.term;
}


// ---- classic-game encoder tables ---------------------------------------------------
// The 1323 cell features (63 view cells x (one-hot of 17 block ids + 4 mob bits)) are
// 0/1: an env's features are packed into a row of bits (cell c = 21 bits at bit 21c), a
// lane's eight features of a 16-wide K block are one byte of that row, and a 256-entry
// table turns the byte into eight bf16 0/1.  The 22 scalar features (inventory and
// intrinsics / 10, direction one-hot, light, sleeping) sit beside them as floats.
// Layout for ENVS envs inside a byte region that starts with their 148-byte records.
constexpr int kClsCells = 63, kClsCh = 21;
constexpr int kClsBits = kClsCells * kClsCh;                 // 1323
constexpr int kClsKb16 = (kClsBits + 15) / 16;               // 83
constexpr int kClsBitRow = 44;                               // dwords per env (42 used)
constexpr int kClsSv = 24;                                   // scalar features per env, padded
constexpr int kClsTailKb = kClsSv / 8;                       // 3 fp32 K blocks
template <int ENVS>
struct ClsLayout {
    static constexpr int offBits = ENVS * CFP_CLASSIC_REC_BYTES;
    static constexpr int offLut = offBits + ENVS * kClsBitRow * 4;
    static constexpr int offSv = offLut + 256 * 16;
    static constexpr int end = offSv + ENVS * kClsSv * 4;
    static_assert(offBits % 16 == 0 && offLut % 16 == 0 && offSv % 16 == 0, "alignment");
};

// Bit rows, byte -> 8 x bf16 table and scalar rows from the records at `base`
// (all 256 threads; ends with a barrier).  Block ids must be 0..16.
template <int ENVS>
__device__ __forceinline__ void classic_prepare(uint8_t* base, int tid) {
    using LY = ClsLayout<ENVS>;
    uint32_t* bits = reinterpret_cast<uint32_t*>(base + LY::offBits);
    u4* lut = reinterpret_cast<u4*>(base + LY::offLut);
    float* sv = reinterpret_cast<float*>(base + LY::offSv);
    for (int i = tid; i < ENVS * kClsBitRow; i += kFwdThreads) bits[i] = 0u;
    {
        u4 v;
        uint32_t d[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = (((unsigned)tid >> (2 * i)) & 1u) * 0x3F80u |
                   (((unsigned)tid >> (2 * i + 1)) & 1u) * 0x3F800000u;
        v.x = d[0]; v.y = d[1]; v.z = d[2]; v.w = d[3];
        lut[tid] = v;
    }
    for (int i = tid; i < ENVS * kClsSv; i += kFwdThreads) {
        const int e = i / kClsSv, f = i - e * kClsSv;
        const uint8_t* o = base + e * CFP_CLASSIC_REC_BYTES + 2 * kClsCells;
        float v = 0.0f;
        if (f < 16) v = (float)(int8_t)o[f] / 10.0f;                  // inventory, intrinsics
        else if (f < 20) v = (int8_t)o[16] == f - 15 ? 1.0f : 0.0f;   // direction 1..4
        else if (f == 20) v = *reinterpret_cast<const float*>(o + 18);   // light
        else if (f == 21) v = o[17] ? 1.0f : 0.0f;                    // sleeping
        sv[i] = v;
    }
    __syncthreads();   // rows are zero before the bits go in
    for (int i = tid; i < ENVS * kClsCells; i += kFwdThreads) {
        const int e = i / kClsCells, cell = i - e * kClsCells;
        const uint8_t* o = base + e * CFP_CLASSIC_REC_BYTES;
        const uint32_t v = ((1u << (o[cell] & 31u)) & 0x1FFFFu) | ((o[kClsCells + cell] & 15u) << 17);
        const int bit = kClsCh * cell, dw = bit >> 5, sh = bit & 31;
        uint32_t* row = bits + e * kClsBitRow;
        atomicOr(row + dw, v << sh);
        if (sh > 32 - kClsCh) atomicOr(row + dw + 1, v >> (32 - sh));
    }
    __syncthreads();
}

// Lane-constant context of one wave.
struct Lane {
    unsigned lane_u;   // 0..63
    int half;          // lane / 32
    int l32;           // lane % 32
    int wave;          // 0..3, scalar
    int arow4;         // f4 index of this lane's A fragment in an x tile, + 2*kb
    unsigned loff;     // lane offset (floats) into a [32][256] state tile row set
    unsigned loff3;    // likewise into a [32][768] pre-activation tile
};

constexpr int kEncPairs = kKbEnc / 2;                 // 53 steps of two K blocks
constexpr int kMapPairs = kKbMap / 2;                 // 49 all-map steps (blocks 0..97)
__device__ __forceinline__ f16v mfma(float a, float b, f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ f16v zero16() {
    f16v z;
#pragma unroll
    for (int i = 0; i < 16; i++) z[i] = 0.0f;
    return z;
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ f16v mfma16(const u4& a, const u4& b, f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// v = hi + mid + lo exactly, each with at most 8 significant bits; packed as bf16
// pairs (element 2p in the low half).
__device__ __forceinline__ void split3(const float (&v)[8], u4& hi, u4& mid, u4& lo) {
    uint32_t h[4], m[4], l[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const float v0 = v[2 * p], v1 = v[2 * p + 1];
        const float r0 = v0 - __uint_as_float(__float_as_uint(v0) & 0xffff0000u);
        const float r1 = v1 - __uint_as_float(__float_as_uint(v1) & 0xffff0000u);
        const float l0 = r0 - __uint_as_float(__float_as_uint(r0) & 0xffff0000u);
        const float l1 = r1 - __uint_as_float(__float_as_uint(r1) & 0xffff0000u);
        h[p] = __builtin_amdgcn_perm(__float_as_uint(v1), __float_as_uint(v0), 0x07060302u);
        m[p] = __builtin_amdgcn_perm(__float_as_uint(r1), __float_as_uint(r0), 0x07060302u);
        l[p] = __builtin_amdgcn_perm(__float_as_uint(l1), __float_as_uint(l0), 0x07060302u);
    }
    hi = u4{h[0], h[1], h[2], h[3]};
    mid = u4{m[0], m[1], m[2], m[3]};
    lo = u4{l[0], l[1], l[2], l[3]};
}

// Eight fp32 -> eight bf16, round to nearest even.
__device__ __forceinline__ u4 round_bf16x8(const float (&v)[8]) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
    const f4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
    const u2_t lo = __builtin_bit_cast(u2_t, __builtin_convertvector(a, bf16x4_t));
    const u2_t hi = __builtin_bit_cast(u2_t, __builtin_convertvector(b, bf16x4_t));
    return u4{lo.x, lo.y, hi.x, hi.y};
}

// Two record bytes -> two bf16 (0..255 are exact in bf16: the upper half of the
// fp32 encoding).
__device__ __forceinline__ uint32_t bytes_to_bf16x2(uint32_t w, int i) {
    const float lo = (float)((w >> (16 * i)) & 0xffu);
    const float hi = (float)((w >> (16 * i + 8)) & 0xffu);
    // upper halves of hi and lo in one byte permute: {hi[3], hi[2], lo[3], lo[2]}
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

__device__ __forceinline__ u4 bytes_to_bf16x8(uint32_t w0, uint32_t w1) {
    u4 r;
    r.x = bytes_to_bf16x2(w0, 0);
    r.y = bytes_to_bf16x2(w0, 1);
    r.z = bytes_to_bf16x2(w1, 0);
    r.w = bytes_to_bf16x2(w1, 1);
    return r;
}

// ---- encoder GEMM of both tiles of a pair, map bytes on the bf16 matrix pipe -------
// 792 of the 843 features are record bytes, exact in bf16.  An fp32 weight is
// exactly the sum of three bf16 numbers (hi = bf16(w), mid = bf16(w - hi),
// lo = w - hi - mid: 3 x 8 significant bits), so byte x weight is the sum of three
// bf16 x bf16 products, each exact in the fp32 the MFMA accumulates in: the same
// arithmetic as an fp32 FMA chain up to the order of the roundings, at
// 3 x 32 cycles of v_mfma_f32_32x32x16_bf16 per 16 features instead of 8 x 64 of
// v_mfma_f32_32x32x2_f32.  K = 792 as 50 blocks of 16 (the upper half of block 49
// is fed zeros); the 51 fp32 tail features follow on the fp32 MFMA (7 K blocks of
// 8 from the fp32 mirror).
struct EncS { u4 b[6]; };   // (unit tile 0|1) x (hi, mid, lo)
struct EncDw { uint32_t x0, x1, y0, y1; };

__device__ __forceinline__ EncDw encs_bytes(const uint32_t* rx, const uint32_t* ry, int kb,
                                            int half) {
    EncDw r;
    r.x0 = rx[4 * kb + 2 * half];
    r.x1 = rx[4 * kb + 2 * half + 1];
    r.y0 = ry[4 * kb + 2 * half];
    r.y1 = ry[4 * kb + 2 * half + 1];
    return r;
}

// ONE: the second tile does not exist (one tile per workgroup); its products are left out.
template <bool ONE = false>
__device__ __forceinline__ void encs_mma(f16v (&acc)[4], const u4& ax, const u4& ay,
                                         const EncS& w) {
#pragma unroll
    for (int s = 0; s < 3; s++)
#pragma unroll
        for (int ut = 0; ut < 2; ut++) {
            acc[ut] = mfma16(ax, w.b[3 * ut + s], acc[ut]);
            if (!ONE) acc[2 + ut] = mfma16(ay, w.b[3 * ut + s], acc[2 + ut]);
        }
}

}  // namespace
}  // namespace cfp
