// The dense-math seam: fp32 MFMA GEMMs behind the reference's wrapper
// signatures cu_gemm_fwd / cu_gemm_enc_fwd / cu_gemm_dh / cu_gemm_dw /
// cu_gemv_dwv (craftax_full.cu:11604-11666), which there forward to
// cublasSgemm / cublasSgemv.  The fused forward does not go through these;
// they serve the PPO update and unfused parity tests.
//
// One kernel covers all four shapes: C[i][j] (+)= sum_k A(i,k) * B(k,j) with
// element strides for both operands, so "transposes" are just strides.
//   workgroup tile 128 x 128 x 32, 4 waves as 2 x 2, each wave 64 x 64
//   (2 x 2 accumulators of v_mfma_f32_32x32x2_f32); operands are staged
//   through LDS as [row][k] with a 36-float row stride so that a lane's
//   16-byte fragment read (k = 4*(lane/32)+j of an 8-wide K block) is
//   conflict free.  Edges are zero-filled, so M, N, K are arbitrary.
// dW = dpre^T x has K = window columns (>= 16k) and a small output, so K is
// split over grid.z into a workspace and summed in a fixed order by a second
// kernel: run-to-run bitwise stable, unlike float atomics.
#include "cfp_common.h"

namespace cfp {
namespace {

constexpr int BM = 128, BN = 128, BK = 32, LDT = BK + 4;
constexpr int GEMM_THREADS = 256;

struct GemmArgs {
    const float* A; long sa_i, sa_k;   // A(i,k) = A[i*sa_i + k*sa_k]
    const float* B; long sb_k, sb_j;   // B(k,j) = B[k*sb_k + j*sb_j]
    float* C; long ldc;                // C[i*ldc + j]; split z adds z*c_split
    long c_split;
    int M, N, K;
    int k_per_split;                   // multiple of BK
};

// Stage a [128 rows][32 k] operand tile into LDS [row][k].  `kfast` says k is
// the unit-stride dimension in memory; lanes walk the unit-stride dimension so
// every wave-wide load covers whole 128-byte segments.
template <bool KFAST>
__device__ __forceinline__ void stage(float* lds, const float* src, long s_row,
                                      long s_k, int row0, int nrows, int k0,
                                      int kend, int tid) {
    if (KFAST) {
        const int kk = tid & 31;
        const int r0 = tid >> 5;
        const int k = k0 + kk;
        const bool kin = k < kend;
#pragma unroll
        for (int it = 0; it < BM / 8; it++) {
            const int r = r0 + 8 * it;
            const int row = row0 + r;
            float v = 0.0f;
            if (kin && row < nrows) v = src[(long)row * s_row + (long)k * s_k];
            lds[r * LDT + kk] = v;
        }
    } else {
        const int r = tid & 127;
        const int kq = tid >> 7;
        const int row = row0 + r;
        const bool rin = row < nrows;
#pragma unroll
        for (int it = 0; it < BK / 2; it++) {
            const int kk = kq + 2 * it;
            const int k = k0 + kk;
            float v = 0.0f;
            if (rin && k < kend) v = src[(long)row * s_row + (long)k * s_k];
            lds[r * LDT + kk] = v;
        }
    }
}

template <bool A_KFAST, bool B_KFAST, bool ACCUM>
__global__ __launch_bounds__(GEMM_THREADS) void k_gemm(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) float As[BM * LDT];
    __shared__ __attribute__((aligned(16))) float Bs[BN * LDT];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    const int i0 = blockIdx.x * BM;
    const int j0 = blockIdx.y * BN;
    const int kbeg = blockIdx.z * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);

    f16v acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

    const f4* As4 = reinterpret_cast<const f4*>(As);
    const f4* Bs4 = reinterpret_cast<const f4*>(Bs);
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        stage<A_KFAST>(As, g.A, g.sa_i, g.sa_k, i0, g.M, k0, kend, tid);
        stage<B_KFAST>(Bs, g.B, g.sb_j, g.sb_k, j0, g.N, k0, kend, tid);
        __syncthreads();
#pragma unroll
        for (int kb = 0; kb < BK / 8; kb++) {
            f4 af[2], bf[2];
#pragma unroll
            for (int a = 0; a < 2; a++)
                af[a] = As4[(wm * 64 + a * 32 + l32) * (LDT / 4) + 2 * kb + half];
#pragma unroll
            for (int b = 0; b < 2; b++)
                bf[b] = Bs4[(wn * 64 + b * 32 + l32) * (LDT / 4) + 2 * kb + half];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int b = 0; b < 2; b++)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            af[a][j], bf[b][j], acc[a][b], 0, 0, 0);
        }
        __syncthreads();
    }

    float* C = g.C + (long)blockIdx.z * g.c_split;
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

// dst[i] += sum_z part[z*stride + i], z ascending.
__global__ void k_splitk_reduce(float* __restrict__ dst,
                                const float* __restrict__ part, long count,
                                long stride, int splits) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float s = 0.0f;
    for (int z = 0; z < splits; z++) s += part[(long)z * stride + i];
    dst[i] += s;
}

// dWv[k] += sum_c x[c][k] * dv[c]: one workgroup per 64 units, 4 waves stride
// the columns, fixed-order LDS reduction.
__global__ __launch_bounds__(256) void k_gemv_dwv(const float* __restrict__ x,
                                                  const float* __restrict__ dv,
                                                  float* __restrict__ dWv,
                                                  int cols) {
    __shared__ float red[4][64];
    const int k = blockIdx.x * 64 + (threadIdx.x & 63);
    const int w = threadIdx.x >> 6;
    float s = 0.0f;
    for (int c = w; c < cols; c += 4)
        s = fmaf(x[(size_t)c * CFP_HIDDEN + k], dv[c], s);
    red[w][threadIdx.x & 63] = s;
    __syncthreads();
    if (w == 0)
        dWv[k] += (red[0][threadIdx.x] + red[1][threadIdx.x]) +
                  (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

template <bool A_KFAST, bool B_KFAST>
int run_gemm(GemmArgs g, int splits, bool accum, hipStream_t st) {
    dim3 grid((g.M + BM - 1) / BM, (g.N + BN - 1) / BN, splits);
    if (accum)
        hipLaunchKernelGGL((k_gemm<A_KFAST, B_KFAST, true>), grid,
                           dim3(GEMM_THREADS), 0, st, g);
    else
        hipLaunchKernelGGL((k_gemm<A_KFAST, B_KFAST, false>), grid,
                           dim3(GEMM_THREADS), 0, st, g);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

// Split-K workspace for cfp_gemm_dw: allocated once per process on first use
// (the reference pre-warms cuBLAS workspaces the same way before capturing a
// graph, craftax_full.cu:12094-12122).
constexpr int kMaxSplits = 64;
constexpr size_t kDwWorkFloats = (size_t)kMaxSplits * CFP_OBS * CFP_HIDDEN;
float* g_dw_work = nullptr;

}  // namespace
}  // namespace cfp

using namespace cfp;

extern "C" {

int cfp_gemm_fwd(int m, int cols, int k, const float* d_W, const float* d_x,
                 float* d_y, void* stream) {
    CFP_REQUIRE(m > 0 && cols > 0 && k > 0 && d_W && d_x && d_y,
                "cfp_gemm_fwd: bad argument");
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
    CFP_REQUIRE(cols > 0 && d_W_enc && d_xobs && d_h,
                "cfp_gemm_enc_fwd: bad argument");
    GemmArgs g{};
    g.A = d_xobs; g.sa_i = CFP_OBS; g.sa_k = 1;
    g.B = d_W_enc; g.sb_k = CFP_HIDDEN; g.sb_j = 1;
    g.C = d_h; g.ldc = CFP_HIDDEN; g.c_split = 0;
    g.M = cols; g.N = CFP_HIDDEN; g.K = CFP_OBS;
    g.k_per_split = (CFP_OBS + BK - 1) / BK * BK;
    return run_gemm<true, false>(g, 1, false, (hipStream_t)stream);
}

int cfp_gemm_dh(int m3, int cols, const float* d_W, const float* d_dpre,
                float* d_dh, void* stream) {
    CFP_REQUIRE(m3 > 0 && cols > 0 && d_W && d_dpre && d_dh,
                "cfp_gemm_dh: bad argument");
    GemmArgs g{};
    g.A = d_dpre; g.sa_i = m3; g.sa_k = 1;
    g.B = d_W; g.sb_k = CFP_HIDDEN; g.sb_j = 1;
    g.C = d_dh; g.ldc = CFP_HIDDEN; g.c_split = 0;
    g.M = cols; g.N = CFP_HIDDEN; g.K = m3;
    g.k_per_split = (m3 + BK - 1) / BK * BK;
    return run_gemm<true, false>(g, 1, false, (hipStream_t)stream);
}

int cfp_gemm_dw(int rows, int cols, const float* d_x, const float* d_dpre,
                float* d_dW, void* stream) {
    CFP_REQUIRE(rows > 0 && rows <= CFP_OBS && cols > 0 && d_x && d_dpre && d_dW,
                "cfp_gemm_dw: bad argument (rows must be in 1..%d)", CFP_OBS);
    hipStream_t st = (hipStream_t)stream;
    // enough workgroups to fill 256 CUs: tiles(M) * tiles(N=2) * splits
    const int tiles = ((rows + BM - 1) / BM) * (CFP_HIDDEN / BN);
    int splits = (1024 + tiles - 1) / tiles;
    const int kblocks = (cols + BK - 1) / BK;
    if (splits > kblocks) splits = kblocks;
    if (splits > kMaxSplits) splits = kMaxSplits;
    if (splits < 1) splits = 1;
    const int k_per_split = ((kblocks + splits - 1) / splits) * BK;
    splits = (cols + k_per_split - 1) / k_per_split;
    GemmArgs g{};
    g.A = d_dpre; g.sa_i = 1; g.sa_k = rows;
    g.B = d_x; g.sb_k = CFP_HIDDEN; g.sb_j = 1;
    g.ldc = CFP_HIDDEN;
    g.M = rows; g.N = CFP_HIDDEN; g.K = cols;
    g.k_per_split = k_per_split;
    if (splits == 1) {
        g.C = d_dW; g.c_split = 0;
        return run_gemm<false, false>(g, 1, true, st);
    }
    if (!g_dw_work)
        CFP_HIP_TRY(hipMalloc((void**)&g_dw_work, kDwWorkFloats * sizeof(float)));
    g.C = g_dw_work;
    g.c_split = (long)rows * CFP_HIDDEN;
    if (run_gemm<false, false>(g, splits, false, st) != 0) return 1;
    const long count = (long)rows * CFP_HIDDEN;
    hipLaunchKernelGGL(k_splitk_reduce, dim3((unsigned)((count + 255) / 256)),
                       dim3(256), 0, st, d_dW, g_dw_work, count, count, splits);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

int cfp_gemv_dwv(const float* d_x, const float* d_dv, float* d_dWv, int cols,
                 void* stream) {
    CFP_REQUIRE(cols > 0 && d_x && d_dv && d_dWv, "cfp_gemv_dwv: bad argument");
    hipLaunchKernelGGL(k_gemv_dwv, dim3(CFP_HIDDEN / 64), dim3(256), 0,
                       (hipStream_t)stream, d_x, d_dv, d_dWv, cols);
    CFP_HIP_TRY(hipGetLastError());
    return 0;
}

}  // extern "C"
