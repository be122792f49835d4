// The dense-math seam: fp32 MFMA GEMMs behind the reference's wrapper
// signatures cu_gemm_fwd / cu_gemm_enc_fwd / cu_gemm_dh / cu_gemm_dw /
// cu_gemv_dwv (craftax_full.cu:11604-11666), which there forward to
// cublasSgemm / cublasSgemv.  The fused forward does not go through these;
// they serve the PPO update and unfused parity tests.
//
// One kernel covers all four shapes: C[i][j] (+)= sum_k A(i,k) * B(k,j) with
// element strides for both operands, so "transposes" are just strides.
//   workgroup tile 128 x 128 x 32, 4 waves as 2 x 2, each wave 64 x 64
//   (2 x 2 accumulators of v_mfma_f32_32x32x2_f32).
//   An operand whose K dimension is the unit-stride one in memory sits in LDS as
//   [row][k] (36-float rows) and a lane's fragment for an 8-wide K block
//   (k = 8b + 4*(lane/32) + j) is one 16-byte read; an operand whose row
//   dimension is unit-stride sits as [k][row] (132-float rows) and the fragment
//   is four 4-byte reads (two ds_read2).  Either way global loads and LDS
//   writes are 16 bytes per lane and coalesced -- nothing is transposed on
//   the way in.  The next K tile is fetched into registers while the current
//   one is multiplied.  Edges are zero-filled, so M, N, K are arbitrary;
//   operands whose base or leading dimension is not 16-byte aligned take a
//   scalar-load path of the same kernel.
//   Workgroup ids are remapped to the XCDs (tile_of_block below).
// dW = dpre^T x has K = window columns (>= 16k) and a small output, so K is
// split over grid.y into a workspace and summed in a fixed order by a second
// kernel: run-to-run bitwise stable, unlike float atomics.
#include <mutex>

#include "cfp_common.h"

namespace cfp {
namespace {

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int LDK = BK + 4;    // [row][k] layout: floats per row
constexpr int LDR = BM + 4;    // [k][row] layout: floats per k
constexpr int OPER_FLOATS = BM * LDK > BK * LDR ? BM * LDK : BK * LDR;
constexpr int GEMM_THREADS = 256;
constexpr int kXcds = 8;

struct GemmArgs {
    const float* A; long sa_i, sa_k;   // A(i,k) = A[i*sa_i + k*sa_k]
    const float* B; long sb_k, sb_j;   // B(k,j) = B[k*sb_k + j*sb_j]
    float* C; long ldc;                // C[i*ldc + j]; split z adds z*c_split
    long c_split;
    int M, N, K;
    int k_per_split;                   // multiple of BK
    int splits;                        // K splits (1 = none)
    int mt, nt;                        // tile counts
};

// Workgroup -> (output tile, K split).  The hardware deals workgroups to the eight
// XCDs round-robin, each XCD with its own L2.
//   no split: consecutive tiles (which share an A tile) go to the same XCD;
//   split K : every XCD takes whole splits -- all output tiles of the splits
//             s = xcd (mod 8), one split after the other -- so the A and B slices
//             of a split are fetched from HBM once and shared through that L2 by
//             the tiles that need them, and all eight XCDs are busy however few
//             output tiles there are.
__device__ __forceinline__ bool tile_of_block(const GemmArgs& g, int& tile, int& split) {
    const int total = g.mt * g.nt;
    const int xcd = (int)(blockIdx.x % kXcds), q = (int)(blockIdx.x / kXcds);
    if (g.splits == 1) {
        const int chunk = (total + kXcds - 1) / kXcds;
        tile = xcd * chunk + q;
        split = 0;
        return tile < total;
    }
    const int sl = q / total;
    tile = q - sl * total;
    split = sl * kXcds + xcd;
    return split < g.splits;
}

// Fetch this thread's share (4 x 16 bytes) of a [128 rows][32 k] operand tile.
// KFAST: k is unit-stride in memory; thread covers (row = v/8, k = 4*(v%8)..+3).
// else : row is unit-stride;        thread covers (k = v/32, row = 4*(v%32)..+3).
// VEC loads 16 bytes at once (the host checked alignment and that reading up to
// the next multiple of four along the unit-stride dimension stays inside the
// leading dimension); elements past the extent are zeroed either way.
template <bool KFAST, bool VEC>
__device__ __forceinline__ void fetch(f4 (&r)[4], const float* src, long s_row, long s_k,
                                      int row0, int nrows, int k0, int kend, int tid) {
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int v = tid + GEMM_THREADS * it;
        int row, k;
        if (KFAST) { row = row0 + (v >> 3); k = k0 + 4 * (v & 7); }
        else { k = k0 + (v >> 5); row = row0 + 4 * (v & 31); }
        f4 val = {0.0f, 0.0f, 0.0f, 0.0f};
        const int lim = KFAST ? kend - k : nrows - row;   // valid elements along the fast dim
        const bool in = KFAST ? row < nrows : k < kend;
        if (in && lim > 0) {
            const float* p = src + (long)row * s_row + (long)k * s_k;
            if (VEC) {
                val = *reinterpret_cast<const f4*>(p);
                if (lim < 4) {
#pragma unroll
                    for (int c = 1; c < 4; c++)
                        if (c >= lim) val[c] = 0.0f;
                }
            } else {
                const long step = KFAST ? s_k : s_row;
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (c < lim) val[c] = p[c * step];
            }
        }
        r[it] = val;
    }
}

template <bool KFAST>
__device__ __forceinline__ void stash(float* lds, const f4 (&r)[4], int tid) {
    f4* l4 = reinterpret_cast<f4*>(lds);
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int v = tid + GEMM_THREADS * it;
        if (KFAST) l4[(v >> 3) * (LDK / 4) + (v & 7)] = r[it];
        else l4[(v >> 5) * (LDR / 4) + (v & 31)] = r[it];
    }
}

// fragment of K block kb for the 32 rows starting at rb: k = 8*kb + 4*half + j
template <bool KFAST>
__device__ __forceinline__ f4 frag(const float* lds, int rb, int l32, int half, int kb) {
    if (KFAST)
        return reinterpret_cast<const f4*>(lds)[(rb + l32) * (LDK / 4) + 2 * kb + half];
    const float* p = lds + (8 * kb + 4 * half) * LDR + rb + l32;
    f4 r = {p[0], p[LDR], p[2 * LDR], p[3 * LDR]};
    return r;
}

template <bool A_KFAST, bool B_KFAST, bool ACCUM, bool VEC_A, bool VEC_B>
__global__ __launch_bounds__(GEMM_THREADS) void k_gemm(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) float As[OPER_FLOATS];
    __shared__ __attribute__((aligned(16))) float Bs[OPER_FLOATS];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    // XCD-aware tile id: hardware deals workgroups to the XCDs round-robin
    int tile, split;
    if (!tile_of_block(g, tile, split)) return;
    const int i0 = (tile / g.nt) * BM;
    const int j0 = (tile % g.nt) * BN;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);

    f16v acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

    f4 ra[4], rb[4];
    fetch<A_KFAST, VEC_A>(ra, g.A, g.sa_i, g.sa_k, i0, g.M, kbeg, kend, tid);
    fetch<B_KFAST, VEC_B>(rb, g.B, g.sb_j, g.sb_k, j0, g.N, kbeg, kend, tid);
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        __syncthreads();   // the previous tile has been read
        stash<A_KFAST>(As, ra, tid);
        stash<B_KFAST>(Bs, rb, tid);
        __syncthreads();
        if (k0 + BK < kend) {
            fetch<A_KFAST, VEC_A>(ra, g.A, g.sa_i, g.sa_k, i0, g.M, k0 + BK, kend, tid);
            fetch<B_KFAST, VEC_B>(rb, g.B, g.sb_j, g.sb_k, j0, g.N, k0 + BK, kend, tid);
        }
#pragma unroll
        for (int kb = 0; kb < BK / 8; kb++) {
            f4 af[2], bf[2];
#pragma unroll
            for (int a = 0; a < 2; a++) af[a] = frag<A_KFAST>(As, wm * 64 + a * 32, l32, half, kb);
#pragma unroll
            for (int b = 0; b < 2; b++) bf[b] = frag<B_KFAST>(Bs, wn * 64 + b * 32, l32, half, kb);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int b = 0; b < 2; b++)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            af[a][j], bf[b][j], acc[a][b], 0, 0, 0);
        }
    }

    float* C = g.C + (long)split * g.c_split;
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int j = j0 + wn * 64 + b * 32 + l32;
            if (j >= g.N) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = i0 + wm * 64 + a * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (i < g.M) {
                    float* c = C + (long)i * g.ldc + j;
                    if (ACCUM) *c += acc[a][b][r];
                    else *c = acc[a][b][r];
                }
            }
        }
}

// ---- bf16-input / fp32-accumulate form of the same GEMM ----------------------------
// (the reference's CF_GEMM_BF16 wrappers, craftax_full.cu:11688-11756).  Operands
// stay fp32 in memory; they are rounded to bf16 (nearest even) on their way into
// LDS, where both sit as [row][k] with 80-byte rows so that a lane's fragment for
// v_mfma_f32_32x32x16_bf16 (eight consecutive k of one row) is one 16-byte read.
// An operand whose K dimension is unit-stride arrives as four consecutive k
// (one 8-byte LDS write); one whose row dimension is unit-stride arrives as four
// rows of one k and is transposed by four 2-byte writes.  At bf16 rates the
// kernel is bound by this staging and by HBM, not by the matrix pipe.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
constexpr int LDB = 40;   // bf16 per LDS row: 32 k + 8 pad

template <bool KFAST>
__device__ __forceinline__ void stash_bf16(__bf16* lds, const f4 (&r)[4], int tid) {
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int v = tid + GEMM_THREADS * it;
        const bf16x4 h = __builtin_convertvector(r[it], bf16x4);
        if (KFAST) {
            *reinterpret_cast<bf16x4*>(lds + (v >> 3) * LDB + 4 * (v & 7)) = h;
        } else {
            __bf16* q = lds + (4 * (v & 31)) * LDB + (v >> 5);
#pragma unroll
            for (int c = 0; c < 4; c++) q[c * LDB] = h[c];
        }
    }
}

template <bool A_KFAST, bool B_KFAST, bool ACCUM, bool VEC_A, bool VEC_B>
__global__ __launch_bounds__(GEMM_THREADS) void k_gemm_bf16(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) __bf16 As[BM * LDB];
    __shared__ __attribute__((aligned(16))) __bf16 Bs[BN * LDB];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    int tile, split;
    if (!tile_of_block(g, tile, split)) return;
    const int i0 = (tile / g.nt) * BM;
    const int j0 = (tile % g.nt) * BN;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);

    f16v acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

    f4 ra[4], rb[4];
    fetch<A_KFAST, VEC_A>(ra, g.A, g.sa_i, g.sa_k, i0, g.M, kbeg, kend, tid);
    fetch<B_KFAST, VEC_B>(rb, g.B, g.sb_j, g.sb_k, j0, g.N, kbeg, kend, tid);
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        __syncthreads();
        stash_bf16<A_KFAST>(As, ra, tid);
        stash_bf16<B_KFAST>(Bs, rb, tid);
        __syncthreads();
        if (k0 + BK < kend) {
            fetch<A_KFAST, VEC_A>(ra, g.A, g.sa_i, g.sa_k, i0, g.M, k0 + BK, kend, tid);
            fetch<B_KFAST, VEC_B>(rb, g.B, g.sb_j, g.sb_k, j0, g.N, k0 + BK, kend, tid);
        }
#pragma unroll
        for (int kb = 0; kb < BK / 16; kb++) {
            bf16x8 af[2], bf[2];
#pragma unroll
            for (int a = 0; a < 2; a++)
                af[a] = *reinterpret_cast<const bf16x8*>(As + (wm * 64 + a * 32 + l32) * LDB +
                                                          16 * kb + 8 * half);
#pragma unroll
            for (int b = 0; b < 2; b++)
                bf[b] = *reinterpret_cast<const bf16x8*>(Bs + (wn * 64 + b * 32 + l32) * LDB +
                                                          16 * kb + 8 * half);
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[b], acc[a][b],
                                                                        0, 0, 0);
        }
    }

    float* C = g.C + (long)split * g.c_split;
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int j = j0 + wn * 64 + b * 32 + l32;
            if (j >= g.N) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = i0 + wm * 64 + a * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (i < g.M) {
                    float* c = C + (long)i * g.ldc + j;
                    if (ACCUM) *c += acc[a][b][r];
                    else *c = acc[a][b][r];
                }
            }
        }
}

// dst[i] += sum_z part[z*stride + i] in a fixed order: the splits are dealt to four
// thread groups (contiguous quarters), each walks its quarter with four independent
// running sums (z = 0, 1, 2, 3 mod 4), and the sixteen sums are folded in one fixed
// tree -- enough loads in flight to run at memory speed, run-to-run bitwise stable.
constexpr int kReduceOut = 64;   // outputs per workgroup of 256 threads
__global__ __launch_bounds__(256) void k_splitk_reduce(float* __restrict__ dst,
                                                       const float* __restrict__ part,
                                                       long count, long stride, int splits) {
    __shared__ float fold[4][kReduceOut];
    const int o = threadIdx.x & (kReduceOut - 1), zg = threadIdx.x / kReduceOut;
    const long i = (long)blockIdx.x * kReduceOut + o;
    const int per = (splits + 3) / 4;
    const int z0 = zg * per, z1 = min(splits, z0 + per);
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    if (i < count) {
        const float* p = part + i;
        int z = z0;
        for (; z + 4 <= z1; z += 4) {
            s0 += p[(long)z * stride];
            s1 += p[(long)(z + 1) * stride];
            s2 += p[(long)(z + 2) * stride];
            s3 += p[(long)(z + 3) * stride];
        }
        for (; z < z1; z++) s0 += p[(long)z * stride];
    }
    fold[zg][o] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (zg == 0 && i < count)
        dst[i] += (fold[0][o] + fold[1][o]) + (fold[2][o] + fold[3][o]);
}

// dWv[k] += sum_c x[c][k] * dv[c].  Stage 1: workgroup z owns a contiguous slice
// of columns, thread k walks it (each column is one coalesced 1 KiB row of x)
// and leaves part[z][k]; stage 2 is k_splitk_reduce, slices in ascending order,
// so the sum is run-to-run bitwise stable.
constexpr int kGemvSlices = 256;
__global__ __launch_bounds__(256) void k_gemv_dwv_partial(const float* __restrict__ x,
                                                          const float* __restrict__ dv,
                                                          float* __restrict__ part, int cols,
                                                          int cols_per_slice) {
    const int c0 = blockIdx.x * cols_per_slice;
    const int c1 = min(cols, c0 + cols_per_slice);
    const int k = threadIdx.x;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    int c = c0;
    for (; c + 4 <= c1; c += 4) {
        s0 = fmaf(x[(size_t)c * CFP_HIDDEN + k], dv[c], s0);
        s1 = fmaf(x[(size_t)(c + 1) * CFP_HIDDEN + k], dv[c + 1], s1);
        s2 = fmaf(x[(size_t)(c + 2) * CFP_HIDDEN + k], dv[c + 2], s2);
        s3 = fmaf(x[(size_t)(c + 3) * CFP_HIDDEN + k], dv[c + 3], s3);
    }
    for (; c < c1; c++) s0 = fmaf(x[(size_t)c * CFP_HIDDEN + k], dv[c], s0);
    part[(size_t)blockIdx.x * CFP_HIDDEN + k] = (s0 + s1) + (s2 + s3);
}

// 16-byte loads need an aligned base, a leading dimension that is a multiple
// of four floats and room to read up to the next multiple of four along the
// unit-stride dimension.
static bool vec_ok(const float* p, long ld, int fast_extent) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0 && ld % 4 == 0 &&
           ld >= (long)((fast_extent + 3) / 4 * 4);
}

// Process-wide switch of the seam's GEMMs to bf16 inputs, like the reference's
// g_gemm_bf16 (craftax_full.cu:11306-11316).
int g_gemm_bf16 = 0;
// fp32 operands split into bf16 triples for the update's shapes (gemm_x9.hip)
int g_gemm_split = 1;
// A trainer with a mode of its own overrides both for the calls it issues: the override
// belongs to the issuing thread and lasts for one entry point (GemmModeScope).
thread_local int t_gemm_bf16 = -1, t_gemm_split = -1;
inline int eff_bf16() { return t_gemm_bf16 >= 0 ? t_gemm_bf16 : g_gemm_bf16; }
inline int eff_split() { return t_gemm_split >= 0 ? t_gemm_split : g_gemm_split; }
// partial products per product on those kernels: bf16 inputs -> 1 (rounded operands)
inline int split_terms() { return eff_bf16() ? 1 : (eff_split() == 2 ? 6 : (eff_split() == 3 ? 8 : 9)); }

template <bool A_KFAST, bool B_KFAST, bool ACCUM>
int launch_gemm(const GemmArgs& g, dim3 grid, bool va, bool vb, hipStream_t st) {
    const dim3 blk(GEMM_THREADS);
    if (eff_bf16()) {
        if (va && vb) hipLaunchKernelGGL((k_gemm_bf16<A_KFAST, B_KFAST, ACCUM, true, true>), grid, blk, 0, st, g);
        else if (va) hipLaunchKernelGGL((k_gemm_bf16<A_KFAST, B_KFAST, ACCUM, true, false>), grid, blk, 0, st, g);
        else if (vb) hipLaunchKernelGGL((k_gemm_bf16<A_KFAST, B_KFAST, ACCUM, false, true>), grid, blk, 0, st, g);
        else hipLaunchKernelGGL((k_gemm_bf16<A_KFAST, B_KFAST, ACCUM, false, false>), grid, blk, 0, st, g);
        CFP_HIP_TRY(hipGetLastError());
        return 0;
    }
    if (va && vb) hipLaunchKernelGGL((k_gemm<A_KFAST, B_KFAST, ACCUM, true, true>), grid, blk, 0, st, g);
    else if (va) hipLaunchKernelGGL((k_gemm<A_KFAST, B_KFAST, ACCUM, true, false>), grid, blk, 0, st, g);
    else if (vb) hipLaunchKernelGGL((k_gemm<A_KFAST, B_KFAST, ACCUM, false, true>), grid, blk, 0, st, g);
    else hipLaunchKernelGGL((k_gemm<A_KFAST, B_KFAST, ACCUM, false, false>), grid, blk, 0, st, g);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

template <bool A_KFAST, bool B_KFAST>
int run_gemm(GemmArgs g, int splits, bool accum, hipStream_t st) {
    g.mt = (g.M + BM - 1) / BM;
    g.nt = (g.N + BN - 1) / BN;
    const int total = g.mt * g.nt;
    g.splits = splits;
    const dim3 grid(splits == 1 ? (total + kXcds - 1) / kXcds * kXcds
                                : kXcds * total * ((splits + kXcds - 1) / kXcds));
    const bool va = A_KFAST ? vec_ok(g.A, g.sa_i, g.K) : vec_ok(g.A, g.sa_k, g.M);
    const bool vb = B_KFAST ? vec_ok(g.B, g.sb_j, g.K) : vec_ok(g.B, g.sb_k, g.N);
    if (accum) return launch_gemm<A_KFAST, B_KFAST, true>(g, grid, va, vb, st);
    return launch_gemm<A_KFAST, B_KFAST, false>(g, grid, va, vb, st);
}

// Split-K workspace of a dW GEMM: room for 128 splits of the largest one (843 rows).
constexpr int kMaxSplits = 128;
constexpr size_t kDwWorkFloats = (size_t)kMaxSplits * CFP_OBS * CFP_HIDDEN;
// The raw C entry points' shared workspace (the reference pre-warms cuBLAS's
// workspaces before capturing a graph, craftax_full.cu:12094-12122: here
// cfp_seam_reserve does that).
std::mutex g_seam_mu;
SeamWork g_seam;
bool g_seam_ready = false;

}  // namespace
}  // namespace cfp

using namespace cfp;

namespace cfp {

int gemm_enc_fwd_ld(int cols, const float* d_W_enc, const float* d_xobs, int ldx, float* d_h,
                    hipStream_t st) {
    CFP_REQUIRE(cols > 0 && d_W_enc && d_xobs && d_h && ldx >= CFP_OBS,
                "cfp_gemm_enc_fwd: bad argument");
    GemmArgs g{};
    g.A = d_xobs; g.sa_i = ldx; g.sa_k = 1;
    g.B = d_W_enc; g.sb_k = CFP_HIDDEN; g.sb_j = 1;
    g.C = d_h; g.ldc = CFP_HIDDEN; g.c_split = 0;
    g.M = cols; g.N = CFP_HIDDEN; g.K = CFP_OBS;
    g.k_per_split = (CFP_OBS + BK - 1) / BK * BK;
    return run_gemm<true, false>(g, 1, false, st);
}

// cu_gemm_dh with an accumulate switch: dh[cols][256] (+)= dpre[cols][m3] . W[m3][256]
int seam_work_create(SeamWork* w) {
    *w = SeamWork{};
    hipError_t e = hipMalloc((void**)&w->w_mirror, dh_mirror_bytes());
    if (e == hipSuccess) e = hipMalloc((void**)&w->dw_part, kDwWorkFloats * sizeof(float));
    if (e == hipSuccess)
        e = hipMalloc((void**)&w->gemv_part, (size_t)kGemvSlices * CFP_HIDDEN * sizeof(float));
    if (e != hipSuccess) {
        set_error("GEMM workspace allocation failed: %s", hipGetErrorString(e));
        seam_work_destroy(w);
        return 1;
    }
    w->dw_part_floats = kDwWorkFloats;
    return 0;
}

void seam_work_destroy(SeamWork* w) {
    (void)hipFree(w->w_mirror);
    (void)hipFree(w->dw_part);
    (void)hipFree(w->gemv_part);
    *w = SeamWork{};
}

const SeamWork* seam_default() {
    std::lock_guard<std::mutex> lock(g_seam_mu);
    if (!g_seam_ready) {
        if (seam_work_create(&g_seam)) return nullptr;
        g_seam_ready = true;
    }
    return &g_seam;
}

int gemm_dh_acc(int m3, int cols, const float* d_W, const float* d_dpre, float* d_dh,
                bool accumulate, const SeamWork& sw, hipStream_t st) {
    CFP_REQUIRE(m3 > 0 && cols > 0 && d_W && d_dpre && d_dh, "cfp_gemm_dh: bad argument");
    if (eff_split() && gemm_dh_x9_ok(m3, cols, d_dpre) && (!accumulate || m3 >= 160))
        return gemm_dh_x9(m3, cols, d_W, d_dpre, d_dh, accumulate, split_terms(), sw.w_mirror, st);
    GemmArgs g{};
    g.A = d_dpre; g.sa_i = m3; g.sa_k = 1;
    g.B = d_W; g.sb_k = CFP_HIDDEN; g.sb_j = 1;
    g.C = d_dh; g.ldc = CFP_HIDDEN; g.c_split = 0;
    g.M = cols; g.N = CFP_HIDDEN; g.K = m3;
    g.k_per_split = (m3 + BK - 1) / BK * BK;
    return run_gemm<true, false>(g, 1, accumulate, st);
}

int launch_splitk_reduce(float* dst, const float* part, long count, long stride, int splits,
                         hipStream_t st) {
    hipLaunchKernelGGL(k_splitk_reduce, dim3((unsigned)((count + kReduceOut - 1) / kReduceOut)),
                       dim3(256), 0, st, dst, part, count, stride, splits);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int gemm_dw_ld(int rows, int cols, const float* d_x, const float* d_dpre, int ld_dpre,
               float* d_dW, const SeamWork& sw, hipStream_t st) {
    CFP_REQUIRE(rows > 0 && rows <= CFP_OBS && cols > 0 && d_x && d_dpre && d_dW &&
                    ld_dpre >= rows,
                "cfp_gemm_dw: bad argument (rows must be in 1..%d)", CFP_OBS);
    if (eff_split() && gemm_dw_x9_ok(rows, cols))
        return gemm_dw_x9(rows, cols, d_x, d_dpre, ld_dpre, d_dW, split_terms(), sw, st);
    // enough workgroups to fill 256 CUs: tiles(M) * tiles(N=2) * splits
    const int tiles = ((rows + BM - 1) / BM) * (CFP_HIDDEN / BN);
    int splits = (2048 + tiles - 1) / tiles;   // measured: 128 splits of the gate dW beat 64 by 3 %
    const int kblocks = (cols + BK - 1) / BK;
    if (splits > kblocks) splits = kblocks;
    // the workspace holds kMaxSplits slices of the largest dW; a smaller one may use more
    int max_splits = (int)(sw.dw_part_floats / ((size_t)rows * CFP_HIDDEN));
    if (max_splits > 4 * kMaxSplits) max_splits = 4 * kMaxSplits;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    const int k_per_split = ((kblocks + splits - 1) / splits) * BK;
    splits = (cols + k_per_split - 1) / k_per_split;
    GemmArgs g{};
    g.A = d_dpre; g.sa_i = 1; g.sa_k = ld_dpre;
    g.B = d_x; g.sb_k = CFP_HIDDEN; g.sb_j = 1;
    g.ldc = CFP_HIDDEN;
    g.M = rows; g.N = CFP_HIDDEN; g.K = cols;
    g.k_per_split = k_per_split;
    if (splits == 1) {
        g.C = d_dW; g.c_split = 0;
        return run_gemm<false, false>(g, 1, true, st);
    }
    CFP_REQUIRE(sw.dw_part, "cfp_gemm_dw: no split workspace");
    g.C = sw.dw_part;
    g.c_split = (long)rows * CFP_HIDDEN;
    if (run_gemm<false, false>(g, splits, false, st) != 0) return 1;
    const long count = (long)rows * CFP_HIDDEN;
    return launch_splitk_reduce(d_dW, sw.dw_part, count, count, splits, st);
}

int gemm_split_terms() { return eff_split() ? split_terms() : 0; }
int gemm_mode_bf16() { return eff_bf16(); }
int gemm_mode_split() { return eff_split(); }
GemmModeScope::GemmModeScope(int bf16, int split) : old_bf16(t_gemm_bf16), old_split(t_gemm_split) {
    if (bf16 >= 0) t_gemm_bf16 = bf16;
    if (split >= 0) t_gemm_split = split;
}
GemmModeScope::~GemmModeScope() {
    t_gemm_bf16 = old_bf16;
    t_gemm_split = old_split;
}

int gemm_dw_two(int rows_a, int rows_b, int cols, const float* d_x, const float* d_dpre,
                int ld_dpre, float* d_dW_a, float* d_dW_b, const SeamWork& sw, hipStream_t st) {
    CFP_REQUIRE(rows_a > 0 && rows_b > 0 && ld_dpre >= rows_a + rows_b && d_dW_a && d_dW_b,
                "gemm_dw_two: bad argument");
    if (eff_split() && gemm_dw_x9_ok(rows_a + rows_b, cols))
        return gemm_dw_x9(rows_a + rows_b, cols, d_x, d_dpre, ld_dpre, d_dW_a, split_terms(), sw, st,
                          rows_a, d_dW_b);
    if (gemm_dw_ld(rows_a, cols, d_x, d_dpre, ld_dpre, d_dW_a, sw, st)) return 1;
    return gemm_dw_ld(rows_b, cols, d_x, d_dpre + rows_a, ld_dpre, d_dW_b, sw, st);
}

}  // namespace cfp

extern "C" {

int cfp_seam_reserve(void) { return seam_default() ? 0 : 1; }

int cfp_set_gemm_bf16(int on) {
    g_gemm_bf16 = on ? 1 : 0;
    return 0;
}
int cfp_get_gemm_bf16(void) { return g_gemm_bf16; }
int cfp_set_gemm_split(int mode) {
    CFP_REQUIRE(mode >= 0 && mode <= 3, "cfp_set_gemm_split: mode must be 0..3 (got %d)", mode);
    g_gemm_split = mode;
    return 0;
}
int cfp_get_gemm_split(void) { return g_gemm_split; }

int cfp_gemm_fwd(int m, int cols, int k, const float* d_W, const float* d_x,
                 float* d_y, void* stream) {
    CFP_REQUIRE(m > 0 && cols > 0 && k > 0 && d_W && d_x && d_y,
                "cfp_gemm_fwd: bad argument");
    if (eff_split() && gemm_fwd_x9_ok(m, cols, k, d_x)) {
        const SeamWork* sw = seam_default();
        if (!sw) return 1;
        return gemm_fwd_x9(m, cols, k, d_W, d_x, d_y, split_terms(), sw->w_mirror,
                           (hipStream_t)stream);
    }
    GemmArgs g{};
    g.A = d_x; g.sa_i = k; g.sa_k = 1;
    g.B = d_W; g.sb_k = 1; g.sb_j = k;
    g.C = d_y; g.ldc = m; g.c_split = 0;
    g.M = cols; g.N = m; g.K = k;
    g.k_per_split = (k + BK - 1) / BK * BK;
    return run_gemm<true, true>(g, 1, false, (hipStream_t)stream);
}

int cfp_gemm_enc_fwd(int cols, const float* d_W_enc, const float* d_xobs,
                     float* d_h, void* stream) {
    return gemm_enc_fwd_ld(cols, d_W_enc, d_xobs, CFP_OBS, d_h, (hipStream_t)stream);
}

int cfp_gemm_dh(int m3, int cols, const float* d_W, const float* d_dpre,
                float* d_dh, void* stream) {
    const SeamWork* sw = seam_default();
    if (!sw) return 1;
    return gemm_dh_acc(m3, cols, d_W, d_dpre, d_dh, false, *sw, (hipStream_t)stream);
}

int cfp_gemm_dw(int rows, int cols, const float* d_x, const float* d_dpre,
                float* d_dW, void* stream) {
    const SeamWork* sw = seam_default();
    if (!sw) return 1;
    return gemm_dw_ld(rows, cols, d_x, d_dpre, rows, d_dW, *sw, (hipStream_t)stream);
}

int cfp_gemv_dwv(const float* d_x, const float* d_dv, float* d_dWv, int cols,
                 void* stream) {
    CFP_REQUIRE(cols > 0 && d_x && d_dv && d_dWv, "cfp_gemv_dwv: bad argument");
    hipStream_t st = (hipStream_t)stream;
    const SeamWork* sw = seam_default();
    if (!sw) return 1;
    float* const g_gemv_work = sw->gemv_part;
    int per = (cols + kGemvSlices - 1) / kGemvSlices;
    if (per < 32) per = 32;
    const int slices = (cols + per - 1) / per;
    hipLaunchKernelGGL(k_gemv_dwv_partial, dim3(slices), dim3(256), 0, st, d_x, d_dv,
                       g_gemv_work, cols, per);
    return launch_splitk_reduce(d_dWv, g_gemv_work, (long)CFP_HIDDEN, (long)CFP_HIDDEN, slices,
                                st);
}

}  // extern "C"
