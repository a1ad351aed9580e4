// C += A * B for row-major panels with row strides.
// Upstream: Eigen `C.noalias() += A*B` / KokkosBlas::gemm on strided sub-block views, one call per
// arriving panel pair (src/backend_internal.hpp:113-133, src/executor_incremental.cpp:97-132).
// fp64 is the one dense contraction of the path, so it runs on the matrix cores
// (v_mfma_f64_16x16x4_f64): 64x64 workgroup tiles, four wavefronts of 32x32, K in steps of 16
// staged through double-buffered LDS. Other element types use a plain LDS-tiled kernel.
#include "common.h"

using namespace cnh;

namespace {

typedef double v4d __attribute__((ext_vector_type(4)));
typedef double v2d __attribute__((ext_vector_type(2)));

constexpr int PAD = 16;

// Workgroup ids are dealt round-robin to the 8 XCDs; give every XCD a contiguous run of logical
// tiles so that the workgroups sharing a B column panel also share one L2.
__device__ __forceinline__ int xcd_remap(int b, int nblocks) {
    if (nblocks % 8 != 0)
        return b;
    return (b % 8) * (nblocks / 8) + b / 8;
}

// WM x WN wavefronts per workgroup, each owning TM x TN tiles of 16x16; K advances BKT at a time.
// The fp64 matrix pipe needs two or more wavefronts per SIMD to stay busy (one wavefront issues at
// ~70% of the rate eight reach), hence the 8-wavefront shape for grids that give each CU a single
// workgroup. Global loads run two K steps ahead of the arithmetic (two register sets, one LDS
// buffer being filled while the other is read): one K step of matrix instructions is shorter than
// a trip to memory.
template <int WM, int WN, int TM, int TN, int BKT, bool FULL>
__global__ __launch_bounds__(WM * WN * 64) void gemm_f64_mfma(int M, int N, int K,
                                                              const double* __restrict__ A, int64_t lda,
                                                              const double* __restrict__ B, int64_t ldb,
                                                              double* __restrict__ C, int64_t ldc) {
    constexpr int NT = WM * WN * 64;
    constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
    constexpr int APT = BM * BKT / NT, BPT = BN * BKT / NT;   // doubles staged per lane
    static_assert(APT >= 2 && BPT >= 2 && APT % 2 == 0 && BPT % 2 == 0, "staging uses 128-bit loads");
    static_assert(BKT % APT == 0 && BN % BPT == 0, "a lane's run stays inside one row");
    // A stays row-major in LDS with rows of BKT + 1 doubles: the operand read of 16 consecutive
    // rows at one k then touches 16 different bank pairs. B is k-major with rows of BN + 16.
    constexpr int AP = BKT + 1;
    __shared__ double As[2][BM][AP];
    __shared__ __attribute__((aligned(16))) double Bs[2][BKT][BN + PAD];
    const int nbm = (M + BM - 1) / BM, nbn = (N + BN - 1) / BN;
    const int logical = xcd_remap(blockIdx.x, nbm * nbn);
    const int bn = logical / nbm, bm = logical - bn * nbm;
    const int m0 = bm * BM, n0 = bn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // staging assignment: A tile BM rows x BKT k (APT along k), B tile BKT k x BN (BPT along n)
    const int a_row = tid / (BKT / APT), a_k = (tid % (BKT / APT)) * APT;
    const int b_k = tid / (BN / BPT), b_n = (tid % (BN / BPT)) * BPT;

    auto fetch = [&](int k0, double (&ra)[APT], double (&rb)[BPT]) {
        const int gr = m0 + a_row;
        const int gk = k0 + a_k;
        if (FULL) {
#pragma unroll
            for (int j = 0; j < APT; j += 2) {
                const v2d v = *reinterpret_cast<const v2d*>(A + (int64_t)gr * lda + gk + j);
                ra[j] = v[0];
                ra[j + 1] = v[1];
            }
        } else {
#pragma unroll
            for (int j = 0; j < APT; ++j)
                ra[j] = (gr < M && gk + j < K) ? A[(int64_t)gr * lda + gk + j] : 0.0;
        }
        const int bk = k0 + b_k;
        const int gn = n0 + b_n;
        if (FULL) {
#pragma unroll
            for (int j = 0; j < BPT; j += 2) {
                const v2d v = *reinterpret_cast<const v2d*>(B + (int64_t)bk * ldb + gn + j);
                rb[j] = v[0];
                rb[j + 1] = v[1];
            }
        } else {
#pragma unroll
            for (int j = 0; j < BPT; ++j)
                rb[j] = (bk < K && gn + j < N) ? B[(int64_t)bk * ldb + gn + j] : 0.0;
        }
    };
    auto stage = [&](int buf, const double (&ra)[APT], const double (&rb)[BPT]) {
#pragma unroll
        for (int j = 0; j < APT; ++j)
            As[buf][a_row][a_k + j] = ra[j];
#pragma unroll
        for (int j = 0; j < BPT; j += 2)
            *reinterpret_cast<v2d*>(&Bs[buf][b_k][b_n + j]) = (v2d){rb[j], rb[j + 1]};
    };

    v4d acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            acc[i][j] = (v4d){0.0, 0.0, 0.0, 0.0};

    const int lr = lane & 15, lk = lane >> 4;
    auto multiply = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < BKT / 4; ++ks) {
            const int kk = ks * 4 + lk;
            double a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                a[i] = As[buf][(wm * TM + i) * 16 + lr][kk];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b[j] = Bs[buf][kk][(wn * TN + j) * 16 + lr];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    };

    // Step t multiplies LDS buffer t&1, which holds K slice t. Register set t&1 receives slice
    // t+2 while that runs; the other set (slice t+1, requested a step earlier) goes to LDS after it.
    const int nk = (K + BKT - 1) / BKT;
    double ra0[APT], rb0[BPT], ra1[APT], rb1[BPT];
    fetch(0, ra0, rb0);
    if (nk > 1)
        fetch(BKT, ra1, rb1);
    stage(0, ra0, rb0);
    __syncthreads();
    // At the top of every round LDS buffer 0 holds slice t and register set 1 slice t + 1.
    // The steady-state rounds carry no conditions, so that the compiler's wait counts leave the
    // younger pair of loads in flight while the older pair is stored.
    int t = 0;
    for (; t + 3 < nk; t += 2) {
        fetch((t + 2) * BKT, ra0, rb0);
        multiply(0);
        stage(1, ra1, rb1);
        __syncthreads();
        fetch((t + 3) * BKT, ra1, rb1);
        multiply(1);
        stage(0, ra0, rb0);
        __syncthreads();
    }
    if (t + 2 < nk)
        fetch((t + 2) * BKT, ra0, rb0);
    multiply(0);
    if (t + 1 < nk) {
        stage(1, ra1, rb1);
        __syncthreads();
        multiply(1);
        if (t + 2 < nk) {
            stage(0, ra0, rb0);
            __syncthreads();
            multiply(0);
        }
    }
    // D layout of the 16x16x4 f64 instruction (measured on gfx950): register r of a lane holds
    // row 4*r + lane/16, column lane % 16.
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + (wn * TN + j) * 16 + lr;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + (wm * TM + i) * 16 + r * 4 + lk;
                if (FULL || (row < M && col < N)) {
                    double* c = C + (int64_t)row * ldc + col;
                    *c = *c + acc[i][j][r];
                }
            }
        }
}

template <typename T>
struct Acc {
    typedef T type;
};
template <>
struct Acc<int32_t> {
    typedef uint32_t type;
};
template <>
struct Acc<int64_t> {
    typedef uint64_t type;
};

template <typename T>
__global__ __launch_bounds__(256) void gemm_tiled_generic(int M, int N, int K,
                                                          const T* __restrict__ A, int64_t lda,
                                                          const T* __restrict__ B, int64_t ldb,
                                                          T* __restrict__ C, int64_t ldc) {
    typedef typename Acc<T>::type U;
    __shared__ T As[16][17];
    __shared__ T Bs[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
    U acc = 0;
    for (int k0 = 0; k0 < K; k0 += 16) {
        As[ty][tx] = (row < M && k0 + tx < K) ? A[(int64_t)row * lda + k0 + tx] : (T)0;
        Bs[ty][tx] = (k0 + ty < K && col < N) ? B[(int64_t)(k0 + ty) * ldb + col] : (T)0;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k)
            acc += (U)As[ty][k] * (U)Bs[k][tx];
        __syncthreads();
    }
    if (row < M && col < N)
        C[(int64_t)row * ldc + col] = (T)((U)C[(int64_t)row * ldc + col] + acc);
}

template <typename T>
int run_generic(int M, int N, int K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C,
                int64_t ldc, hipStream_t st) {
    dim3 grid((N + 15) / 16, (M + 15) / 16);
    CNH_CHECK(grid.y <= 65535, -3, "cnh_gemm_acc: M too large for this element type");
    hipLaunchKernelGGL(gemm_tiled_generic<T>, grid, dim3(256), 0, st, M, N, K, (const T*)A, lda,
                       (const T*)B, ldb, (T*)C, ldc);
    CNH_HIP(hipGetLastError());
    return 0;
}

} // namespace

namespace {
struct GemmArgs {
    int M, N, K;
    const double* A;
    int64_t lda;
    const double* B;
    int64_t ldb;
    double* C;
    int64_t ldc;
};

template <int WM, int WN, int TM, int TN, int BKT>
int launch_mfma(const GemmArgs& g, bool aligned, hipStream_t st) {
    constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
    const int64_t blocks = (((int64_t)g.M + BM - 1) / BM) * (((int64_t)g.N + BN - 1) / BN);
    CNH_CHECK(blocks < (1ll << 31), -3, "cnh_gemm_acc: too many tiles");
    const bool full = aligned && g.M % BM == 0 && g.N % BN == 0 && g.K % BKT == 0;
    if (full)
        hipLaunchKernelGGL((gemm_f64_mfma<WM, WN, TM, TN, BKT, true>), dim3((unsigned)blocks),
                           dim3(WM * WN * 64), 0, st, g.M, g.N, g.K, g.A, g.lda, g.B, g.ldb, g.C, g.ldc);
    else
        hipLaunchKernelGGL((gemm_f64_mfma<WM, WN, TM, TN, BKT, false>), dim3((unsigned)blocks),
                           dim3(WM * WN * 64), 0, st, g.M, g.N, g.K, g.A, g.lda, g.B, g.ldb, g.C, g.ldc);
    CNH_HIP(hipGetLastError());
    return 0;
}
} // namespace

extern "C" int cnh_gemm_acc(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                            const void* B, int64_t ldb, void* C, int64_t ldc, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(M >= 0 && N >= 0 && K >= 0, -2, "cnh_gemm_acc: negative extent");
    CNH_CHECK(M < (1ll << 30) && N < (1ll << 30) && K < (1ll << 30), -3,
              "cnh_gemm_acc: extent too large");
    if (M == 0 || N == 0 || K == 0)
        return 0;
    CNH_CHECK(A && B && C, -2, "cnh_gemm_acc: null pointer");
    CNH_CHECK(lda >= K && ldb >= N && ldc >= N, -2, "cnh_gemm_acc: row stride shorter than the row");
    hipStream_t st = as_stream(s);
    switch (dtype) {
    case CNH_F64: {
        const bool aligned = (lda % 2 == 0) && (ldb % 2 == 0) && (((uintptr_t)A & 15) == 0) &&
                             (((uintptr_t)B & 15) == 0);
        const GemmArgs ga{(int)M, (int)N, (int)K, (const double*)A, lda, (const double*)B, ldb, (double*)C, ldc};
        // 64x64 tiles of four wavefronts when that gives every CU several workgroups; smaller
        // grids take 8 wavefronts per workgroup so that a CU with one workgroup still has two
        // wavefronts per SIMD.
        const int64_t blocks64 = ((M + 63) / 64) * ((N + 63) / 64);
        if (blocks64 >= 1024)
            return launch_mfma<2, 2, 2, 2, 16>(ga, aligned, st);
        return launch_mfma<2, 4, 2, 1, 16>(ga, aligned, st);
    }
    case CNH_F32: return run_generic<float>((int)M, (int)N, (int)K, A, lda, B, ldb, C, ldc, st);
    case CNH_I32: return run_generic<int32_t>((int)M, (int)N, (int)K, A, lda, B, ldb, C, ldc, st);
    case CNH_I64: return run_generic<int64_t>((int)M, (int)N, (int)K, A, lda, B, ldb, C, ldc, st);
    }
    return set_error(-2, "unknown dtype %d", dtype);
}
