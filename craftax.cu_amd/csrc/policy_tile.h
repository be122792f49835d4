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
#pragma unroll
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
        for (int i = tid; i < kTileEnvs * CFP_HIDDEN / 4; i += kFwdThreads)
            xs4[(i >> 6) * XS4 + (i & 63)] = src[i];
    }
}

// Classic-game encoder (encode_obs_kernel, craftax_classic.cu:1714-1751): the
// observation is one-hot per view cell, so h0 is b_enc plus a sum of W_enc
// rows selected by the record bytes, in feature order.  Thread k owns hidden
// unit k and walks the tile's 32 envs; the record bytes are LDS broadcasts and
// every W_enc row read is one coalesced 1 KiB line set from L2.
__device__ __forceinline__ void classic_encode_tile(const FwdArgs& a, const uint8_t* crec,
                                                    float* lds, int tid) {
    constexpr int CELLS = 63, CH = 21, NBLK = 17;
    const float* W = a.w_enc;            // uniform base, [tid] applied at each load
    const unsigned k = (unsigned)tid;
    const float bias = a.b_enc[tid];
    for (int e = 0; e < kTileEnvs; e++) {
        const uint8_t* o = crec + e * CFP_CLASSIC_REC_BYTES;
        float hv = bias;
        for (int cell = 0; cell < CELLS; cell++) {
            hv += (W + (size_t)(cell * CH + (int8_t)o[cell]) * CFP_HIDDEN)[k];
            const uint32_t m = o[CELLS + cell];
            if (m) {
                const float* wm = W + (size_t)(cell * CH + NBLK) * CFP_HIDDEN;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (m & (1u << j)) hv += (wm + (size_t)j * CFP_HIDDEN)[k];
            }
        }
        int f = CELLS * CH;
#pragma unroll
        for (int j = 0; j < 16; j++, f++)
            hv = fmaf((float)(int8_t)o[2 * CELLS + j] / 10.0f, (W + (size_t)f * CFP_HIDDEN)[k], hv);
        const int dir = (int8_t)o[2 * CELLS + 16];
#pragma unroll
        for (int d = 1; d <= 4; d++, f++)
            hv = fmaf(dir == d ? 1.0f : 0.0f, (W + (size_t)f * CFP_HIDDEN)[k], hv);
        const float sleeping = o[2 * CELLS + 17] ? 1.0f : 0.0f;
        const float light = *reinterpret_cast<const float*>(o + 2 * CELLS + 18);
        hv = fmaf(light, (W + (size_t)f * CFP_HIDDEN)[k], hv); f++;
        hv = fmaf(sleeping, (W + (size_t)f * CFP_HIDDEN)[k], hv);
        lds[e * XS + tid] = hv;
    }
}

// Lane-constant context of one wave.
struct Lane {
    unsigned lane_u;   // 0..63
    int half;          // lane / 32
    int l32;           // lane % 32
    int wave;          // 0..3, scalar
    int arow4;         // f4 index of this lane's A fragment in an x tile, + 2*kb
    unsigned loff;     // lane offset (floats) into a [32][256] state tile row set
};

}  // namespace
}  // namespace cfp
