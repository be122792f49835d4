// fp32 GEMMs of the PPO update on the bf16 matrix pipe.
//
// An fp32 number is exactly hi + mid + lo with three bf16 numbers (8 + 8 + 8 significand
// bits, split3), so a product a*b is exactly the sum of the nine products of their
// parts, each of which is exact in fp32 (8 x 8 bits).  Nine v_mfma_f32_32x32x16_bf16
// with fp32 accumulation therefore add up the same exact products as the fp32 MFMA --
// with one accumulator rounding per 16 products instead of per 2 -- and take 9/16 of
// its pipe time.  The reference runs these GEMMs as cublasSgemm behind cu_gemm_dw
// and cu_gemm_dh (craftax_full.cu:11642-11666).
// TERMS = 8 leaves out lo*lo alone (|lo| < 2^-15 |a| with truncated parts: below 2^-30 of a
// product).  TERMS = 6 leaves out mid*lo, lo*mid and lo*lo: with truncated parts |mid| < 2^-7 |a|
// and |lo| < 2^-15 |a|, so at most 2^-21 of |a*b| per product (about 2^-24 on average,
// always towards zero), the size of the roundings the fp32 accumulation of those
// products makes anyway, for two thirds of the MFMAs.  Opt-in.
// TERMS = 1 is the seam's bf16-input mode (operands rounded to nearest even, one
// product) on the same kernels: same loads and pipeline, a ninth of the MFMAs.
//
// k_dw_x9: dW[rows][256] += sum_c dpre[c][row] * x[c][unit], K = window columns.
//   grid      : ceil(rows / 128) row groups x S splits of the columns; the groups of a
//               split sit on one XCD and share x through its L2
//   workgroup : 8 waves; wave w owns units 32w..32w+31 and the group's four 32-row
//               blocks (4 accumulators)
//   K loop    : 64 columns per iteration (4 K steps of 16).  dpre side through LDS:
//               every wave fetches two (K step, row block) pieces -- 8 columns per
//               lane, each load a coalesced 128-byte row piece -- splits them and
//               stores three ready MFMA fragments each.  x side private to the wave,
//               split in registers.  Same software pipeline as the record-fed
//               encoder kernel.
//   output    : per-split partial sums, folded in a fixed order.
#include <mutex>

#include "policy_tile.h"

// W mirror of cfp_gemm_dh_noalloc (below): the split, MFMA-ordered copy of W that
// k_dh_x9 reads, for K up to 768 rows -- 48 K steps x 24 fragments x 64 lanes x 16 bytes.
// Every GPU the library runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[(CFP_GRU / 16) * 24 * 64 * 16];

namespace cfp {
namespace {

// The operand parts a kernel multiplies: TERMS = 9, 8 or 6 -> the exact triple; TERMS = 1 ->
// the operand rounded to bf16 (the bf16-input mode of the seam), one product.
template <int TERMS>
__device__ __forceinline__ void parts_of(const float (&v)[8], u4 (&p)[3]) {
    if (TERMS == 1) {
        p[0] = round_bf16x8(v);
        p[1] = p[0];
        p[2] = p[0];
    } else {
        split3(v, p[0], p[1], p[2]);
    }
}
template <int TERMS>
__device__ __forceinline__ constexpr bool term_used(int i, int j) {
    return TERMS == 9 || (TERMS == 8 && i + j <= 3) || (TERMS == 6 && i + j <= 2) || (TERMS == 1 && i == 0 && j == 0);
}

constexpr int kX9Threads = 512;
constexpr int kX9Blocks = 4;               // 32-row blocks per row group
constexpr int kX9GroupRows = 32 * kX9Blocks;
constexpr int kX9IterCols = 64;
constexpr int kX9Xcds = 8;

// DP16 / X16: that operand is stored as bf16 (bf16-input mode only, TERMS = 1).  A dword
// then holds two adjacent rows (units) of one column, so a lane that loads dword n of a
// 64-row span gets rows 2n and 2n+1: the even rows form one 32-row MFMA block and the
// odd rows the next -- a permutation of rows (units), undone where the result is stored.
//   dpre: wave w loads K step w/2 of the row-block pair w%2 (one load set instead of two)
//   x   : waves 2m and 2m+1 both load the 64 units 64m .. 64m+63 and keep the even /
//         the odd ones
template <int TERMS, bool DP16 = false, bool X16 = false>
__global__ __launch_bounds__(kX9Threads) void k_dw_x9(
    const float* __restrict__ dpre, int ldp, int rows, const float* __restrict__ x,
    float* __restrict__ part, int cols, int iters_per_split, int n_wg, int groups) {
    static_assert(TERMS == 1 || (!DP16 && !X16), "bf16 storage goes with bf16 inputs");
    // [buffer][K step][3 * row block + part][lane]: 96 KiB
    __shared__ u4 stage[2][4][3 * kX9Blocks][64];
    const int xcd = (int)(blockIdx.x % kX9Xcds), q = (int)(blockIdx.x / kX9Xcds);
    const int lin = xcd * (int)(gridDim.x / kX9Xcds) + q;
    if (lin >= n_wg) return;
    const int split = lin / groups, gi = lin - split * groups;
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int total_iters = (cols + kX9IterCols - 1) / kX9IterCols;
    const int it0 = split * iters_per_split;
    const int it1 = min(total_iters, it0 + iters_per_split);
    // this wave stages row block pb of K steps pk and pk + 2 (DP16: K step w / 2 of the
    // row-block pair w % 2)
    const int pk = DP16 ? w >> 1 : w >> 2, pb = DP16 ? 2 * (w & 1) : w & 3;

    // Branch-free body: loads past the last column go to the last 8 columns and the
    // dpre side of such columns is zeroed (cols % 8 == 0, so 8-column groups are all
    // in or all out).
    // rows past the last one read the last row; their results are not stored
    const float* dp_lane = dpre + min(gi * kX9GroupRows + 32 * pb + n, rows - 1);
    auto dp_load = [&](int it, int ks, float (&v)[8]) {
        const int cc = min(it * kX9IterCols + ks * 16 + 8 * g, cols - 8);
        const float* p = dp_lane + (size_t)cc * ldp;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = p[(size_t)j * ldp];
    };
    auto dp_store = [&](int it, int ks, int buf, const float (&v)[8]) {
        const bool in = it * kX9IterCols + ks * 16 + 8 * g < cols;
        float e[8];
#pragma unroll
        for (int j = 0; j < 8; j++) e[j] = in ? v[j] : 0.0f;
        u4 p[3];
        parts_of<TERMS>(e, p);
        stage[buf][ks][3 * pb + 0][lane] = p[0];
        if (TERMS > 1) {
            stage[buf][ks][3 * pb + 1][lane] = p[1];
            stage[buf][ks][3 * pb + 2][lane] = p[2];
        }
    };
    // bf16 dpre: dword n of the pair's 64 rows, eight columns
    const uint32_t* dp16_lane = reinterpret_cast<const uint32_t*>(dpre) +
                                (gi * kX9GroupRows + 32 * pb) / 2 + n;
    auto dp_load16 = [&](int it, float (&v)[8]) {
        const int cc = min(it * kX9IterCols + pk * 16 + 8 * g, cols - 8);
        const uint32_t* p = dp16_lane + (size_t)cc * (ldp / 2);
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = __uint_as_float(p[(size_t)j * (ldp / 2)]);
    };
    // eight dwords of bf16 pairs -> the fragment of the even (odd) halves
    auto pack16 = [&](const float (&v)[8], bool odd, bool in) {
        uint32_t d[4];
#pragma unroll
        for (int p = 0; p < 4; p++)
            d[p] = __builtin_amdgcn_perm(__float_as_uint(v[2 * p + 1]), __float_as_uint(v[2 * p]),
                                         odd ? 0x07060302u : 0x05040100u);
        return in ? u4{d[0], d[1], d[2], d[3]} : u4{0u, 0u, 0u, 0u};
    };
    auto dp_store16 = [&](int it, int buf, const float (&v)[8]) {
        const bool in = it * kX9IterCols + pk * 16 + 8 * g < cols;
        stage[buf][pk][3 * pb][lane] = pack16(v, false, in);
        stage[buf][pk][3 * (pb + 1)][lane] = pack16(v, true, in);
    };
    const float* x_lane = X16 ? reinterpret_cast<const float*>(
                                    reinterpret_cast<const uint32_t*>(x) + 32 * (w >> 1) + n)
                              : x + 32 * w + n;
    constexpr int kXRow = X16 ? CFP_HIDDEN / 2 : CFP_HIDDEN;   // dwords per column of x
    auto x_load = [&](int it, int ks, float (&v)[8]) {
        const int cc = min(it * kX9IterCols + ks * 16 + 8 * g, cols - 8);
        const float* p = x_lane + (size_t)cc * kXRow;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = p[j * kXRow];
    };
    auto x_parts = [&](const float (&v)[8], u4 (&p)[3]) {
        if (X16) {
            p[0] = pack16(v, (w & 1) != 0, true);
            p[1] = p[0];
            p[2] = p[0];
        } else {
            parts_of<TERMS>(v, p);
        }
    };
    auto frag_load = [&](int buf, int ks, int pair, u4 (&a)[6]) {
#pragma unroll
        for (int i = 0; i < 6; i++) a[i] = stage[buf][ks][6 * pair + i][lane];
    };

    f16v acc[kX9Blocks];
#pragma unroll
    for (int b = 0; b < kX9Blocks; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = 0.0f;

    // How far ahead the operands are requested.  The split kernels are bound by the matrix
    // pipe: x three K steps and dpre one iteration ahead cover the latency.  With one
    // product per operand pair an iteration is 16 MFMAs and the kernel is bound by HBM:
    // requests one iteration ahead make an iteration last one memory latency, so x goes
    // seven K steps and dpre two iterations ahead.
    constexpr int kXRing = TERMS == 1 ? 8 : 4, kXAhead = kXRing - 1;
    constexpr int kDpAhead = TERMS == 1 ? 2 : 1;
    if (it0 < it1) {
        const int itl = it1 - 1;
        float d0[kDpAhead][8], d1[kDpAhead][8];   // dpre of iteration it0 + r in slot r % kDpAhead
        float raw[kXRing][8];                     // x of K step G = 4 r + ks in slot G % kXRing
        auto dp_fetch = [&](int it, float (&e0)[8], float (&e1)[8]) __attribute__((always_inline)) {
            if (DP16) {
                dp_load16(it, e0);
            } else {
                dp_load(it, pk, e0);
                dp_load(it, pk + 2, e1);
            }
        };
        auto dp_stage = [&](int it, int buf, const float (&e0)[8], const float (&e1)[8])
                            __attribute__((always_inline)) {
            if (DP16) {
                dp_store16(it, buf, e0);
            } else {
                dp_store(it, pk, buf, e0);
                dp_store(it, pk + 2, buf, e1);
            }
        };
#pragma unroll
        for (int j = 0; j < kDpAhead; j++) dp_fetch(min(it0 + j, itl), d0[j], d1[j]);
#pragma unroll
        for (int j = 0; j < kXAhead; j++) x_load(min(it0 + j / 4, itl), j % 4, raw[j]);
        dp_stage(it0, 0, d0[0], d1[0]);
        __syncthreads();
        u4 a[2][6];
        frag_load(0, 0, 0, a[0]);
        u4 bs[3];
        x_parts(raw[0], bs);
        // par = (it - it0) & 1, a literal at every call of the one-product kernels, where it
        // selects registers; the LDS buffer everywhere
        auto iteration = [&](int it, const int par) __attribute__((always_inline)) {
            const int buf = par;
            const int itn = min(it + 1, itl);
            // the slot of this iteration's dpre (staged during the previous one)
            dp_fetch(min(it + kDpAhead, itl), d0[par % kDpAhead], d1[par % kDpAhead]);
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const int G = 4 * par + ks;   // K step modulo the ring
                x_load(min(it + (ks + kXAhead) / 4, itl), (ks + kXAhead) % 4,
                       raw[(G + kXAhead) % kXRing]);
                u4 ns[3];
                x_parts(raw[(G + 1) % kXRing], ns);
#pragma unroll
                for (int pr = 0; pr < 2; pr++) {
                    const int cur = pr, nxt = pr ^ 1;
                    if (pr < 1) {
                        frag_load(buf, ks, 1, a[nxt]);
                    } else if (ks < 3) {
                        frag_load(buf, ks + 1, 0, a[nxt]);
                    } else {
                        // this wave's last read of the current buffer is in flight or
                        // done; the barrier's wait covers it
                        dp_stage(itn, buf ^ 1, d0[(par + 1) % kDpAhead], d1[(par + 1) % kDpAhead]);
                        __syncthreads();
                        frag_load(buf ^ 1, 0, 0, a[nxt]);
                    }
                    const int b = 2 * pr;
#pragma unroll
                    for (int i = 0; i < 3; i++)
#pragma unroll
                        for (int j = 0; j < 3; j++) {
                            if (!term_used<TERMS>(i, j)) continue;
                            acc[b] = mfma16(a[cur][i], bs[j], acc[b]);
                            acc[b + 1] = mfma16(a[cur][3 + i], bs[j], acc[b + 1]);
                        }
                }
                bs[0] = ns[0]; bs[1] = ns[1]; bs[2] = ns[2];
                // six products: left free, the scheduler hoists enough of the next K steps'
                // LDS reads to take 215 registers, and above 208 the reverse sweep that
                // runs under this kernel finds no room on the CU
                if (TERMS == 6) __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (TERMS == 1) {
            int it = it0;
            for (; it + 1 < it1; it += 2) {
                iteration(it, 0);
                iteration(it + 1, 1);
            }
            if (it < it1) iteration(it, 0);
        } else {
            // four ring slots and one dpre slot: the parity only selects the LDS buffer.
            // (Not unrolled: the split kernels have to stay within 208 registers, or
            // the reverse sweep that runs under them finds no room on the CU.)
            for (int it = it0; it < it1; it++) iteration(it, (it - it0) & 1);
        }
    }
    // undo the even / odd permutations of bf16-stored operands
    const int unit = X16 ? 64 * (w >> 1) + 2 * n + (w & 1) : 32 * w + n;
    float* o = part + ((size_t)split * rows + gi * kX9GroupRows) * CFP_HIDDEN + unit;
#pragma unroll
    for (int b = 0; b < kX9Blocks; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int i = acc_row(r) + 4 * g;
            const int row = DP16 ? 64 * (b >> 1) + 2 * i + (b & 1) : 32 * b + i;
            if (gi * kX9GroupRows + row < rows) o[(size_t)row * CFP_HIDDEN] = acc[b][r];
        }
}

// k_dh_x9: dh[c][u] (+)= sum_k dpre[c][k] * W[k][u] for 256 units, K = m3 (multiple of 16);
// also the gate-forward shape y = x . W^T, 256 output rows at a time (gemm_fwd_x9).
//   workgroup : 256 columns; wave w owns columns 32w..32w+31 of them and all 256 units
//               (8 accumulators).  Its dpre fragment of a K step is 32 contiguous
//               bytes per lane, split in registers one step ahead.
//   W         : split once into an MFMA-ordered mirror (k_pack_w_x9: [K step][unit tile]
//               [part][lane] 16-byte fragments); every step the eight waves copy its 24
//               fragments into LDS (3 each) and all read them back, two at a time, one
//               group of 6 MFMAs ahead of their use.  One barrier per step, placed
//               before the step's last group so that the next step's first fragments
//               are on their way while it runs.
constexpr int kDhThreads = 512;
constexpr int kDhTileCols = 256;
constexpr int kDhFrags = 24;   // 8 unit tiles x 3 parts per K step

__global__ void k_pack_w_x9(const float* __restrict__ W, long sk, long su, u4* __restrict__ out,
                            int total, int rounded, int krows) {   // W(k, u) = W[k*sk + u*su], 0 from row krows on
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int lane = idx & 63, f = (idx >> 6) % kDhFrags, s = idx / (64 * kDhFrags);
    const int t = f / 3, part = f - 3 * t, n = lane & 31, g = lane >> 5;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int k = 16 * s + 8 * g + j;
        v[j] = k < krows ? W[(long)k * sk + (long)(32 * t + n) * su] : 0.0f;
    }
    u4 h, m, l;
    split3(v, h, m, l);
    if (rounded) h = round_bf16x8(v);   // bf16-input mode: part 0 is the rounded operand
    out[idx] = part == 0 ? h : (part == 1 ? m : l);
}

// A16: dpre is stored as bf16 (bf16-input mode): a lane's eight values of a K step are
// the MFMA operand as they lie in memory.
// O16: dh is a bf16 array (ldc counts bf16 elements).  A lane holds unit n of each of
// the eight 32-unit tiles; neighbouring lanes swap one value per pair of tiles, after
// which an even lane owns units n, n+1 of the even tile and an odd lane units n-1, n of
// the odd tile: one 4-byte access per lane, row and pair of tiles.
__device__ __forceinline__ float swap_with_neighbour(float v) { return __shfl_xor(v, 1, 64); }
__device__ __forceinline__ uint32_t pack_bf16_pair(float lo, float hi) {   // nearest even
    typedef float f2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{lo, hi}, bf16x2_t));
}

// AROW: the rows of dpre are `lda` floats apart with lda any number (rows only 4-byte
// aligned) and hold kvalid <= m3 values: a lane fetches its eight values of a K step as
// single dwords and reads what lies past kvalid as zero (the encoder product from an fp32
// feature matrix: 843 features a row).
template <int TERMS, bool A16 = false, bool O16 = false, bool AROW = false>
__global__ __launch_bounds__(kDhThreads) void k_dh_x9(const float* __restrict__ dpre, int m3,
                                                      const u4* __restrict__ wm,
                                                      float* __restrict__ dh, int ldc, int cols,
                                                      int accumulate, int lda, int kvalid) {
    __shared__ u4 stage[2][kDhFrags][64];   // 48 KiB
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int steps = m3 / 16;
    const int cb = (int)blockIdx.x * kDhTileCols + 32 * w;
    const bool live = cb < cols;               // cols % 32 == 0: blocks are whole
    const int cbc = live ? cb : cols - 32;     // idle waves still stage W and meet the barriers
    static_assert(TERMS == 1 || !A16, "bf16 storage goes with bf16 inputs");
    static_assert(!AROW || (!A16 && !O16), "row-strided A is an fp32 operand");
    const float* a_lane = dpre + (size_t)(cbc + n) * (AROW ? lda : m3) + 8 * g;
    const u4* a16_lane = reinterpret_cast<const u4*>(
        reinterpret_cast<const uint16_t*>(dpre) + (size_t)(cbc + n) * m3 + 8 * g);
    auto a_load = [&](int s, float (&v)[8]) {
        if (A16) {   // eight bf16 = 16 bytes, kept as raw bits in the first four slots
            const u4 q = a16_lane[2 * s];
            v[0] = __uint_as_float(q.x); v[1] = __uint_as_float(q.y);
            v[2] = __uint_as_float(q.z); v[3] = __uint_as_float(q.w);
            return;
        }
        if (AROW) {
            // rows are only 4-byte aligned: eight dwords (sixteen-byte loads on a dword boundary
            // measured 4 % slower), what lies past kvalid reads as zero and is never touched
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = 16 * s + 8 * g + j < kvalid ? a_lane[16 * s + j] : 0.0f;
            return;
        }
        const f4* p = reinterpret_cast<const f4*>(a_lane + 16 * s);
        const f4 x0 = p[0], x1 = p[1];
#pragma unroll
        for (int j = 0; j < 4; j++) { v[j] = x0[j]; v[4 + j] = x1[j]; }
    };
    auto a_parts = [&](const float (&v)[8], u4 (&p)[3]) {
        if (A16) {
            p[0] = u4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]),
                      __float_as_uint(v[3])};
            p[1] = p[0];
            p[2] = p[0];
        } else {
            parts_of<TERMS>(v, p);
        }
    };
    // wave w stages the three parts of W for (tile pair w / 2, half w % 2); with one
    // product only the first part is used
    constexpr int kWParts = TERMS == 1 ? 1 : 3;
    const u4* w_lane = wm + (size_t)3 * w * 64 + lane;
    auto w_load = [&](int s, u4 (&b)[3]) {
#pragma unroll
        for (int i = 0; i < kWParts; i++) b[i] = w_lane[((size_t)s * kDhFrags + i) * 64];
    };
    auto w_store = [&](int buf, const u4 (&b)[3]) {
#pragma unroll
        for (int i = 0; i < kWParts; i++) stage[buf][3 * w + i][lane] = b[i];
    };
    // group q of a step: unit tiles 2*(q/3), 2*(q/3)+1, part q%3 of W
    auto frag_load = [&](int buf, int q, u4 (&b)[2]) {
        const int tp = q / 3, j = q - 3 * tp;
        b[0] = stage[buf][6 * tp + j][lane];
        b[1] = stage[buf][6 * tp + 3 + j][lane];
    };

    static_assert(TERMS == 1 || !O16, "bf16 storage goes with bf16 inputs");
    float* o_lane = dh + (size_t)(cbc + 4 * g) * ldc + n;
    // O16: the lane's dword of a pair of tiles (ldc even, n - odd even: 4-byte aligned)
    const bool odd = n & 1;
    uint32_t* o16_lane = reinterpret_cast<uint32_t*>(
        reinterpret_cast<uint16_t*>(dh) + (size_t)(cbc + 4 * g) * ldc + (odd ? 32 + n - 1 : n));
    // The accumulators start at zero; the old contents of dh are fetched one 32-unit tile
    // (O16: one pair of tiles) per K step during the first steps and added a step later, so
    // that the fetch runs under the MFMAs instead of in front of them (every workgroup of
    // a round starts at once: loads in front of the loop are a phase nothing runs beside).
    // The epilogue is stores only.  The launcher asks for enough K steps.
    constexpr int kSpreadMax = O16 ? 4 : 8;
    const bool spread = accumulate != 0;
    f16v acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = 0.0f;
    f16v held;   // O16: sixteen dwords of two bf16 as raw bits
    auto old_fetch = [&](int i) {   // tile i, or pair of tiles i
#pragma unroll
        for (int r = 0; r < 16; r++) {
            if (O16)
                held[r] = __uint_as_float(o16_lane[((size_t)acc_row(r) * ldc + 64 * i) >> 1]);
            else
                held[r] = o_lane[(size_t)acc_row(r) * ldc + 32 * i];
        }
    };
    // (macros, not lambdas over references: the accumulators must stay in registers)
#define CFP_DH_OLD_ADD(EVEN, OTHER)                                                                \
    _Pragma("unroll") for (int r = 0; r < 16; r++) {                                               \
        if (O16) {                                                                                 \
            const uint32_t d = __float_as_uint(held[r]);                                           \
            const float lo = __uint_as_float(d << 16), hi = __uint_as_float(d & 0xffff0000u);      \
            /* even lane: lo is its own unit of the even tile, hi the neighbour's; */              \
            /* odd lane: hi is its own unit of the odd tile, lo the neighbour's */                 \
            const float got = swap_with_neighbour(odd ? lo : hi);                                  \
            acc[EVEN][r] += odd ? got : lo;                                                        \
            acc[OTHER][r] += odd ? hi : got;                                                       \
        } else {                                                                                   \
            acc[EVEN][r] += held[r];                                                               \
        }                                                                                          \
    }
#define CFP_DH_OLD_ADD_AT(I)                                                                       \
    do {   /* I is uniform over the workgroup */                                                   \
        if (O16) {                                                                                 \
            switch (I) {                                                                           \
                case 0: CFP_DH_OLD_ADD(0, 1) break;                                                \
                case 1: CFP_DH_OLD_ADD(2, 3) break;                                                \
                case 2: CFP_DH_OLD_ADD(4, 5) break;                                                \
                default: CFP_DH_OLD_ADD(6, 7) break;                                               \
            }                                                                                      \
        } else {                                                                                   \
            switch (I) {                                                                           \
                case 0: CFP_DH_OLD_ADD(0, 0) break;                                                \
                case 1: CFP_DH_OLD_ADD(1, 1) break;                                                \
                case 2: CFP_DH_OLD_ADD(2, 2) break;                                                \
                case 3: CFP_DH_OLD_ADD(3, 3) break;                                                \
                case 4: CFP_DH_OLD_ADD(4, 4) break;                                                \
                case 5: CFP_DH_OLD_ADD(5, 5) break;                                                \
                case 6: CFP_DH_OLD_ADD(6, 6) break;                                                \
                default: CFP_DH_OLD_ADD(7, 7) break;                                               \
            }                                                                                      \
        }                                                                                          \
    } while (0)

    // dpre is requested kAhead K steps ahead of its MFMAs.  The split kernels are bound by
    // the matrix pipe and two steps cover the latency; with one product per operand pair
    // the kernel is bound by HBM, and a workgroup (the only one on its CU) has to keep
    // about 48-64 KiB in flight: 6 steps of 8 KiB (bf16 dpre) or 4 of 16 KiB (fp32 dpre).
    // Loads return in issue order, so W (an L2 hit) comes back no sooner than the dpre
    // request in front of it: W travels through registers equally far ahead.
    constexpr int kAhead = TERMS != 1 ? 2 : (A16 ? 6 : 4);
    constexpr int kWAhead = TERMS != 1 ? 1 : kAhead;   // W(s + 1) is staged during step s
    static_assert(kAhead % kWAhead == 0, "one literal selects both rings");
    float raw[kAhead][8];
    u4 wring[kWAhead][3];
    const int last = steps - 1;
#pragma unroll
    for (int j = 0; j < kWAhead; j++) w_load(min(j, last), wring[j]);
#pragma unroll
    for (int j = 0; j < kAhead; j++) a_load(min(j, last), raw[j]);
    w_store(0, wring[0]);
    w_load(min(kWAhead, last), wring[0]);
    u4 as[3];
    a_parts(raw[0], as);
    __syncthreads();
    u4 b[2][2];
    frag_load(0, 0, b[0]);
    // slot = s % kAhead as a literal at every call: it selects registers
    auto k_step = [&](int s, const int slot) __attribute__((always_inline)) {
        const int buf = slot & 1;
        static_assert(kAhead % 2 == 0, "the W stage buffer follows the slot's parity");
        // raw[slot] held step s (already split): refill it kAhead steps ahead
        a_load(min(s + kAhead, last), raw[slot]);
        u4 ns[3];
        a_parts(raw[(slot + 1) % kAhead], ns);
#pragma unroll
        for (int q = 0; q < 12; q++) {
            const int cur = q & 1, nxt = cur ^ 1;
            if (q < 11) {
                frag_load(buf, q + 1, b[nxt]);
            } else {
                // next step's W parts: everyone is past its reads of the other buffer
                // (they precede the previous barrier)
                w_store(buf ^ 1, wring[(slot + 1) % kWAhead]);   // W(s + 1)
                __syncthreads();
                w_load(min(s + 1 + kWAhead, last), wring[(slot + 1) % kWAhead]);
                frag_load(buf ^ 1, 0, b[nxt]);
            }
            const int t = 2 * (q / 3);
#pragma unroll
            for (int i = 0; i < 3; i++) {
                if (!term_used<TERMS>(i, q % 3)) continue;
                acc[t] = mfma16(as[i], b[cur][0], acc[t]);
                acc[t + 1] = mfma16(as[i], b[cur][1], acc[t + 1]);
            }
        }
        as[0] = ns[0]; as[1] = ns[1]; as[2] = ns[2];
    };
    int s0 = 0;
    if (spread) {
        // the first steps as straight-line code: the tile an old value is added to is a
        // compile-time register index.  The peel runs on to a multiple of kAhead, where
        // the loop below takes over with slot 0.
        constexpr int kPeel = (kSpreadMax + 1 + kAhead - 1) / kAhead * kAhead;
#pragma unroll
        for (int i = 0; i < kPeel; i++) {
            if (i > 0 && i <= kSpreadMax) CFP_DH_OLD_ADD_AT(i - 1);
            if (i < kSpreadMax) old_fetch(i);
            if (i <= kSpreadMax || i < steps) k_step(i, i % kAhead);   // steps > kSpreadMax
        }
        s0 = kPeel;
    }
    int sr = s0;   // a multiple of kAhead
    for (; sr + kAhead <= steps; sr += kAhead) {
#pragma unroll
        for (int j = 0; j < kAhead; j++) k_step(sr + j, j);
    }
#pragma unroll
    for (int j = 0; j < kAhead - 1; j++)
        if (sr + j < steps) k_step(sr + j, j);
    if (O16) {
        // the swap involves every lane of the wavefront: it comes before the early exit
#pragma unroll
        for (int tp = 0; tp < 4; tp++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float got =
                    swap_with_neighbour(odd ? acc[2 * tp][r] : acc[2 * tp + 1][r]);
                const uint32_t d = odd ? pack_bf16_pair(got, acc[2 * tp + 1][r])
                                       : pack_bf16_pair(acc[2 * tp][r], got);
                if (live) o16_lane[((size_t)acc_row(r) * ldc + 64 * tp) >> 1] = d;
            }
        return;
    }
    if (!live) return;
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            o_lane[(size_t)acc_row(r) * ldc + 32 * t] = acc[t][r];
}

#undef CFP_DH_OLD_ADD_AT
#undef CFP_DH_OLD_ADD

constexpr int kDhMaxK = CFP_GRU;
constexpr int kEncK = (CFP_OBS + 15) / 16 * 16;   // 848: the encoder's K, padded to whole steps
constexpr size_t kDhMirrorBytes = (size_t)(kDhMaxK / 16) * kDhFrags * 64 * sizeof(u4);   // 1.125 MiB
constexpr size_t kEncMirrorBytes = (size_t)(kEncK / 16) * kDhFrags * 64 * sizeof(u4);   // 1.24 MiB

}  // namespace

bool gemm_dh_x9_ok(int m3, int cols, const float* dpre) {
    return m3 >= 16 && m3 % 16 == 0 && m3 <= kDhMaxK && cols >= 32 && cols % 32 == 0 &&
           (reinterpret_cast<uintptr_t>(dpre) & 15u) == 0;
}

// out[cols][ldc] (+)= A[cols][K] . B, B(k, u) = B[k*sk + u*su] for 256 units
static int launch_dh_x9(int K, int cols, const float* B, long sk, long su, const float* A,
                        float* out, int ldc, bool accumulate, int terms, u4* g_w_x9,
                        hipStream_t st, bool a16 = false, bool o16 = false) {
    CFP_REQUIRE((!a16 && !o16) || terms == 1,
                "k_dh_x9: bf16-stored operands need the bf16-input mode");
    CFP_REQUIRE(!o16 || ldc % 2 == 0, "k_dh_x9: a bf16 result needs an even row length");
    // the old contents are fetched during the first nine K steps
    CFP_REQUIRE(!accumulate || K >= 160, "k_dh_x9: accumulating needs K >= 160 (got %d)", K);
    CFP_REQUIRE(g_w_x9, "k_dh_x9: no mirror buffer for W");
    const int total = (K / 16) * kDhFrags * 64;
    hipLaunchKernelGGL(k_pack_w_x9, dim3((total + 255) / 256), dim3(256), 0, st, B, sk, su, g_w_x9,
                       total, terms == 1 ? 1 : 0, K);
    const dim3 grid((cols + kDhTileCols - 1) / kDhTileCols);
    const int acc = accumulate ? 1 : 0;
    if (a16 && o16)
        hipLaunchKernelGGL((k_dh_x9<1, true, true>), grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    else if (o16)
        hipLaunchKernelGGL((k_dh_x9<1, false, true>), grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    else if (a16)
        hipLaunchKernelGGL((k_dh_x9<1, true>), grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    else if (terms == 1)
        hipLaunchKernelGGL(k_dh_x9<1>, grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    else if (terms == 6)
        hipLaunchKernelGGL(k_dh_x9<6>, grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    else if (terms == 8)
        hipLaunchKernelGGL(k_dh_x9<8>, grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    else
        hipLaunchKernelGGL(k_dh_x9<9>, grid, dim3(kDhThreads), 0, st, A, K, g_w_x9, out, ldc, cols, acc, 0, 0);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

size_t dh_mirror_bytes() { return kDhMirrorBytes; }
size_t enc_mirror_bytes() { return kEncMirrorBytes; }

// Encoder product from an fp32 feature matrix: h[cols][256] = xobs[cols][843] . W_enc[843][256]
// (cu_gemm_enc_fwd, craftax_full.cu:11616) on the split kernels: K = 848 in 53 steps, rows of
// xobs ldx floats apart, features 843..847 read as zero on both sides.
bool gemm_enc_fwd_x9_ok(int cols, const float* xobs) {
    return cols >= 32 && cols % 32 == 0 && (reinterpret_cast<uintptr_t>(xobs) & 3u) == 0;
}
int gemm_enc_fwd_x9(int cols, const float* W_enc, const float* xobs, int ldx, float* h, int terms,
                    u4* enc_mirror, hipStream_t st) {
    CFP_REQUIRE(gemm_enc_fwd_x9_ok(cols, xobs) && W_enc && h && enc_mirror && ldx >= CFP_OBS,
                "gemm_enc_fwd_x9: columns must be a multiple of 32 and the matrix 4-byte aligned");
    const int total = (kEncK / 16) * kDhFrags * 64;
    hipLaunchKernelGGL(k_pack_w_x9, dim3((total + 255) / 256), dim3(256), 0, st, W_enc, (long)CFP_HIDDEN, 1L,
                       enc_mirror, total, terms == 1 ? 1 : 0, CFP_OBS);
    const dim3 grid((cols + kDhTileCols - 1) / kDhTileCols);
    if (terms == 1)
        hipLaunchKernelGGL((k_dh_x9<1, false, false, true>), grid, dim3(kDhThreads), 0, st, xobs, kEncK, enc_mirror, h,
                           CFP_HIDDEN, cols, 0, ldx, CFP_OBS);
    else if (terms == 6)
        hipLaunchKernelGGL((k_dh_x9<6, false, false, true>), grid, dim3(kDhThreads), 0, st, xobs, kEncK, enc_mirror, h,
                           CFP_HIDDEN, cols, 0, ldx, CFP_OBS);
    else if (terms == 8)
        hipLaunchKernelGGL((k_dh_x9<8, false, false, true>), grid, dim3(kDhThreads), 0, st, xobs, kEncK, enc_mirror, h,
                           CFP_HIDDEN, cols, 0, ldx, CFP_OBS);
    else
        hipLaunchKernelGGL((k_dh_x9<9, false, false, true>), grid, dim3(kDhThreads), 0, st, xobs, kEncK, enc_mirror, h,
                           CFP_HIDDEN, cols, 0, ldx, CFP_OBS);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int gemm_dh_x9(int m3, int cols, const float* W, const float* dpre, float* dh, bool accumulate,
               int terms, u4* w_mirror, hipStream_t st, bool dpre_bf16, bool dh_bf16) {
    CFP_REQUIRE(gemm_dh_x9_ok(m3, cols, dpre) && W && dh,
                "gemm_dh_x9: K must be a multiple of 16 up to %d and columns of 32", kDhMaxK);
    return launch_dh_x9(m3, cols, W, CFP_HIDDEN, 1, dpre, dh, CFP_HIDDEN, accumulate, terms, w_mirror,
                        st, dpre_bf16, dh_bf16);
}

// y[cols][m] = x[cols][k] . W[m][k]^T in slices of 256 output rows of W
bool gemm_fwd_x9_ok(int m, int cols, int k, const float* x) {
    return m >= CFP_HIDDEN && m % CFP_HIDDEN == 0 && gemm_dh_x9_ok(k, cols, x);
}

int gemm_fwd_x9(int m, int cols, int k, const float* W, const float* x, float* y, int terms,
                u4* w_mirror, hipStream_t st) {
    CFP_REQUIRE(gemm_fwd_x9_ok(m, cols, k, x) && W && y,
                "gemm_fwd_x9: m must be a multiple of 256, k of 16 up to %d, columns of 32", kDhMaxK);
    for (int j = 0; j < m / CFP_HIDDEN; j++)
        if (launch_dh_x9(k, cols, W + (size_t)j * CFP_HIDDEN * k, 1, k, x, y + j * CFP_HIDDEN, m,
                         false, terms, w_mirror, st))
            return 1;
    return 0;
}

}  // namespace cfp

// Device address of `scratch` on each GPU, resolved on the first call made with that GPU
// current: the array's name is only a host-side handle, each device has its own copy.
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

extern "C" int cfp_gemm_dh_noalloc(int m3, int cols, const float* d_W, const float* d_dpre,
                                   float* d_dh, void* stream) {
    using namespace cfp;
    static_assert(sizeof(scratch) == kDhMirrorBytes, "scratch holds one W mirror");
    CFP_REQUIRE(m3 > 0 && cols > 0 && d_W && d_dpre && d_dh, "cfp_gemm_dh_noalloc: bad argument");
    CFP_REQUIRE(m3 <= kDhMaxK, "cfp_gemm_dh_noalloc: m3 = %d exceeds the %d rows its W mirror holds",
                m3, kDhMaxK);
    CFP_REQUIRE(gemm_dh_x9_ok(m3, cols, d_dpre),
                "cfp_gemm_dh_noalloc: m3 must be a multiple of 16, cols of 32 and dpre 16-byte "
                "aligned (got m3 = %d, cols = %d)", m3, cols);
    int dev = -1;
    CFP_HIP_TRY(hipGetDevice(&dev));
    CFP_REQUIRE(dev >= 0 && dev < kMaxDevices, "cfp_gemm_dh_noalloc: device index %d out of range", dev);
    void* ptr = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        if (!g_scratch_ptr[dev]) {
            void* p = nullptr;
            CFP_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            CFP_REQUIRE(p, "cfp_gemm_dh_noalloc: no device address for the W mirror");
            g_scratch_ptr[dev] = p;
        }
        ptr = g_scratch_ptr[dev];
    }
    // same arithmetic as cfp_gemm_dh runs for this shape: nine exact partial products
    // unless the process-wide switches ask for six, or for bf16 inputs
    const int terms = gemm_split_terms() ? gemm_split_terms() : 9;
    return gemm_dh_x9(m3, cols, d_W, d_dpre, d_dh, false, terms, reinterpret_cast<u4*>(ptr),
                      (hipStream_t)stream);
}

namespace cfp {

bool gemm_dw_x9_ok(int rows, int cols) {
    return rows > 0 && cols >= 8 && cols % 8 == 0;
}

int gemm_dw_x9(int rows, int cols, const float* x, const float* dpre, int ld_dpre, float* dW,
               int terms, const SeamWork& sw, hipStream_t st, int rows_first, float* dW_rest,
               bool dpre_bf16, bool x_bf16) {
    CFP_REQUIRE((!dpre_bf16 && !x_bf16) || terms == 1,
                "gemm_dw_x9: bf16-stored operands need the bf16-input mode");
    CFP_REQUIRE(!dpre_bf16 || (rows % kX9GroupRows == 0 && ld_dpre % 2 == 0),
                "gemm_dw_x9: bf16-stored dpre needs whole groups of %d rows", kX9GroupRows);
    CFP_REQUIRE(gemm_dw_x9_ok(rows, cols) && x && dpre && dW && ld_dpre >= rows &&
                    (!dW_rest || (rows_first > 0 && rows_first < rows)),
                "gemm_dw_x9: columns must be a multiple of 8");
    // GEMMs that overlap each other need split workspaces of their own
    float* work = sw.dw_part;
    const size_t work_floats = sw.dw_part_floats;
    CFP_REQUIRE(work, "gemm_dw_x9: no split workspace");
    const int groups = (rows + kX9GroupRows - 1) / kX9GroupRows;
    const int total_iters = (cols + kX9IterCols - 1) / kX9IterCols;
    int splits = 256 / groups;   // one workgroup per CU
    const int cap = (int)(work_floats / ((size_t)rows * CFP_HIDDEN));
    if (splits > cap) splits = cap;
    if (splits > total_iters) splits = total_iters;
    CFP_REQUIRE(splits >= 1, "gemm_dw_x9: split workspace too small for %d rows", rows);
    const int ips = (total_iters + splits - 1) / splits;
    splits = (total_iters + ips - 1) / ips;
    const int n_wg = splits * groups;
    const int grid = (n_wg + kX9Xcds - 1) / kX9Xcds * kX9Xcds;
    if (dpre_bf16 && x_bf16)
        hipLaunchKernelGGL((k_dw_x9<1, true, true>), dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre,
                           rows, x, work, cols, ips, n_wg, groups);
    else if (x_bf16)
        hipLaunchKernelGGL((k_dw_x9<1, false, true>), dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre,
                           rows, x, work, cols, ips, n_wg, groups);
    else if (dpre_bf16)
        hipLaunchKernelGGL((k_dw_x9<1, true, false>), dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre,
                           rows, x, work, cols, ips, n_wg, groups);
    else if (terms == 1)
        hipLaunchKernelGGL(k_dw_x9<1>, dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre, rows, x,
                           work, cols, ips, n_wg, groups);
    else if (terms == 6)
        hipLaunchKernelGGL(k_dw_x9<6>, dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre, rows, x,
                           work, cols, ips, n_wg, groups);
    else if (terms == 8)
        hipLaunchKernelGGL(k_dw_x9<8>, dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre, rows, x,
                           work, cols, ips, n_wg, groups);
    else
        hipLaunchKernelGGL(k_dw_x9<9>, dim3(grid), dim3(kX9Threads), 0, st, dpre, ld_dpre, rows, x,
                           work, cols, ips, n_wg, groups);
    CFP_HIP_TRY(hipGetLastError());
    // rows [0, rows_first) are added onto dW, the others (if any) onto dW_rest
    const long count = (long)rows * CFP_HIDDEN;
    const long first = dW_rest ? (long)rows_first * CFP_HIDDEN : count;
    if (launch_splitk_reduce(dW, work, first, count, splits, st)) return 1;
    if (first < count)
        return launch_splitk_reduce(dW_rest, work + first, count - first, count, splits, st);
    return 0;
}

}  // namespace cfp
