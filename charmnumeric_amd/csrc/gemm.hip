// C += A * B for row-major panels with row strides.
// Upstream: Eigen `C.noalias() += A*B` / KokkosBlas::gemm on strided sub-block views, one call per
// arriving panel pair (src/backend_internal.hpp:113-133, src/executor_incremental.cpp:97-132).
// fp64 is the one dense contraction of the path, so it runs on the matrix cores
// (v_mfma_f64_16x16x4_f64): 64x64 workgroup tiles, K in steps of 16 staged through double-buffered
// LDS; four wavefronts of 32x32 on big grids, eight of 16x32 on smaller ones, and two such sets of
// eight sharing the K steps where a CU gets a single workgroup. Other element types use a plain
// LDS-tiled kernel.
#include "common.h"

#include <cstring>
#include <vector>

using namespace cnh;

namespace {

typedef int64_t cn_i64;
typedef int32_t cn_i32;
#define CN_GEMM_HEAD(...)                                                                             \
    template <int WM, int WN, int TM, int TN, int BKT, bool FULL, bool BUF = false, int KS = 1>       \
    __global__ __launch_bounds__(WM * WN * 64 * KS) void gemm_f64_mfma(__VA_ARGS__)
#define CN_GEMM_MORE_ARGS
#include "gemm_kernel.inc"

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

int check_job(const cnh_gemm_job& j) {
    CNH_CHECK(j.M >= 0 && j.N >= 0 && j.K >= 0, -2, "cnh_gemm_acc: negative extent");
    CNH_CHECK(j.M < (1ll << 30) && j.N < (1ll << 30) && j.K < (1ll << 30), -3,
              "cnh_gemm_acc: extent too large");
    if (j.M == 0 || j.N == 0 || j.K == 0)
        return 0;
    CNH_CHECK(j.A && j.B && j.C, -2, "cnh_gemm_acc: null pointer");
    CNH_CHECK(j.lda >= j.K && j.ldb >= j.N && j.ldc >= j.N, -2,
              "cnh_gemm_acc: row stride shorter than the row");
    return 0;
}

int compute_units() {
    static int cus[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 0;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            return 0;
        cus[dev] = n;
    }
    return cus[dev];
}

int g_gemm_buffer_loads = 1;   // option "gemm_buffer_loads"
int g_gemm_ksplit = 1;         // option "gemm_ksplit": two sets of wavefronts per workgroup on small grids

template <int WM, int WN, int TM, int TN, int BKT, bool KSPLIT = false>
int launch_chains(std::vector<GemmChain>& chains, const std::vector<GemmSeg>& segs, bool full,
                  int overwrite, hipStream_t st) {
    constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
    int64_t blocks = 0;
    for (GemmChain& c : chains) {
        c.nbm = (c.M + BM - 1) / BM;
        c.blk0 = (int32_t)blocks;
        blocks += (int64_t)c.nbm * ((c.N + BN - 1) / BN);
        CNH_CHECK(blocks < (1ll << 31), -3, "cnh_gemm_acc: too many tiles");
    }
    const GemmChain* dch = nullptr;
    const GemmSeg* dsg = nullptr;
    if (chains.size() > 1 || segs.size() > 1) {
        // one table: chains, then segments
        std::vector<unsigned char> table(chains.size() * sizeof(GemmChain) + segs.size() * sizeof(GemmSeg));
        std::memcpy(table.data(), chains.data(), chains.size() * sizeof(GemmChain));
        std::memcpy(table.data() + chains.size() * sizeof(GemmChain), segs.data(),
                    segs.size() * sizeof(GemmSeg));
        const void* dev = nullptr;
        if (int rc = desc_upload(table.data(), table.size(), st, &dev))
            return rc;
        dch = static_cast<const GemmChain*>(dev);
        dsg = reinterpret_cast<const GemmSeg*>(static_cast<const unsigned char*>(dev) +
                                               chains.size() * sizeof(GemmChain));
    }
    const int nch = (int)chains.size(), nb = (int)blocks;
    // buffer loads need a lane's offset inside its workgroup's block of A (BM rows) and K step of
    // B (BKT rows) to fit 31 bits
    bool buf = full && g_gemm_buffer_loads;
    for (const GemmSeg& sg : segs)
        buf = buf && (int64_t)BM * sg.lda * 8 < (1ll << 31) && (int64_t)BKT * sg.ldb * 8 < (1ll << 31);
    // two sets of wavefronts per workgroup where no CU gets more than one workgroup and every K
    // divides (256 x 2048 @ 2048 x 4096 under sustained load: 72.0 -> 66.2 us; with 384 or 512
    // workgroups on 256 CUs the split costs 4 %: its 106 KB of LDS keep a second workgroup off the CU)
    bool split = buf && KSPLIT && g_gemm_ksplit && blocks <= compute_units();
    for (const GemmSeg& sg : segs)
        split = split && sg.K % (2 * BKT) == 0;
    if (split)
        hipLaunchKernelGGL((gemm_f64_mfma<WM, WN, TM, TN, BKT, true, true, KSPLIT ? 2 : 1>), dim3((unsigned)blocks),
                           dim3(WM * WN * 64 * 2), 0, st, dch, nch, dsg, nb, chains[0], segs[0], overwrite);
    else if (buf)
        hipLaunchKernelGGL((gemm_f64_mfma<WM, WN, TM, TN, BKT, true, true>), dim3((unsigned)blocks),
                           dim3(WM * WN * 64), 0, st, dch, nch, dsg, nb, chains[0], segs[0], overwrite);
    else if (full)
        hipLaunchKernelGGL((gemm_f64_mfma<WM, WN, TM, TN, BKT, true>), dim3((unsigned)blocks),
                           dim3(WM * WN * 64), 0, st, dch, nch, dsg, nb, chains[0], segs[0], overwrite);
    else
        hipLaunchKernelGGL((gemm_f64_mfma<WM, WN, TM, TN, BKT, false>), dim3((unsigned)blocks),
                           dim3(WM * WN * 64), 0, st, dch, nch, dsg, nb, chains[0], segs[0], overwrite);
    CNH_HIP(hipGetLastError());
    return 0;
}

int run_f64_batch(int njobs, const cnh_gemm_job* jobs, int overwrite, hipStream_t st) {
    std::vector<GemmChain> chains;
    std::vector<std::vector<GemmSeg>> per_chain;
    bool full = true;
    for (int i = 0; i < njobs; ++i) {
        const cnh_gemm_job& j = jobs[i];
        if (j.M == 0 || j.N == 0 || j.K == 0)
            continue;
        size_t c = 0;
        for (; c < chains.size(); ++c)
            if (chains[c].C == j.C && chains[c].M == j.M && chains[c].N == j.N && chains[c].ldc == j.ldc)
                break;
        if (c == chains.size()) {
            chains.push_back(GemmChain{(double*)j.C, j.ldc, (int32_t)j.M, (int32_t)j.N, 0, 0, 0, 0});
            per_chain.emplace_back();
        }
        per_chain[c].push_back(GemmSeg{(const double*)j.A, j.lda, (const double*)j.B, j.ldb, (int32_t)j.K, 0});
        full = full && (j.M % 64 == 0) && (j.N % 64 == 0) && (j.K % 16 == 0) && (j.lda % 2 == 0) &&
               (j.ldb % 2 == 0) && (((uintptr_t)j.A & 15) == 0) && (((uintptr_t)j.B & 15) == 0);
    }
    if (chains.empty())
        return 0;
    std::vector<GemmSeg> segs;
    int64_t blocks64 = 0;
    for (size_t c = 0; c < chains.size(); ++c) {
        chains[c].seg0 = (int32_t)segs.size();
        chains[c].nseg = (int32_t)per_chain[c].size();
        segs.insert(segs.end(), per_chain[c].begin(), per_chain[c].end());
        blocks64 += (int64_t)((chains[c].M + 63) / 64) * ((chains[c].N + 63) / 64);
    }
    // 64x64 tiles of four wavefronts when that gives every CU several workgroups; smaller grids
    // take 8 wavefronts per workgroup so that a CU with one workgroup still has two per SIMD.
    // Measured on MI355X: big grids are fastest with 32x32 per wavefront (4096^3: 2.05 ms against
    // 2.07-2.13 for 16x64, 64x16 or the 8-wavefront shape); one-workgroup-per-CU grids with 16 rows
    // x 32 columns per wavefront (256x2048 @ 2048x4096: 86 us against 92 for 32 x 16).
    if (blocks64 >= 1024)
        return launch_chains<2, 2, 2, 2, 16>(chains, segs, full, overwrite, st);
    return launch_chains<4, 2, 1, 2, 16, true>(chains, segs, full, overwrite, st);
}

} // namespace

namespace {
// Issue rate of the fp64 matrix instruction with nothing else in the way: 8 wavefronts per CU,
// four independent accumulators each, operands in registers.
__global__ __launch_bounds__(512) void mfma_f64_probe(double* out, int iters, double a0, double b0) {
    v4d acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        acc[i] = (v4d){0.0, 0.0, 0.0, 0.0};
    const double a = a0 + threadIdx.x, b = b0 - threadIdx.x;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
    }
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}
} // namespace

namespace cnh {
void gemm_set_buffer_loads(int on) { g_gemm_buffer_loads = on; }
void gemm_set_ksplit(int on) { g_gemm_ksplit = on; }
int gemm_form(int64_t M, int64_t N, int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb) {
    const bool full = M > 0 && N > 0 && K > 0 && M % 64 == 0 && N % 64 == 0 && K % 16 == 0 && lda % 2 == 0 &&
                      ldb % 2 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)B & 15) == 0;
    const bool buf = full && g_gemm_buffer_loads && 64 * lda * 8 < (1ll << 31) && 16 * ldb * 8 < (1ll << 31);
    if (!buf)
        return 0;
    const int64_t blocks = (M / 64) * (N / 64);
    if (blocks >= 1024)
        return blocks < (1ll << 31) ? 3 : 0;
    return g_gemm_ksplit && blocks <= compute_units() && K % 32 == 0 ? 1 : 2;
}
} // namespace cnh

extern "C" int cnh_probe_mfma_f64(int iters, double* tflops) {
    CNH_CHECK(iters >= 1 && iters <= (1 << 20) && tflops != nullptr, -2, "cnh_probe_mfma_f64: bad argument");
    int dev = 0;
    hipDeviceProp_t prop;
    CNH_HIP(hipGetDevice(&dev));
    CNH_HIP(hipGetDeviceProperties(&prop, dev));
    const int blocks = prop.multiProcessorCount, threads = 512;
    double* out = nullptr;
    CNH_HIP(hipMalloc((void**)&out, (size_t)blocks * threads * sizeof(double)));
    hipEvent_t e0, e1;
    CNH_HIP(hipEventCreate(&e0));
    CNH_HIP(hipEventCreate(&e1));
    hipLaunchKernelGGL(mfma_f64_probe, dim3(blocks), dim3(threads), 0, nullptr, out, 64, 1.0, 2.0);   // warm-up
    CNH_HIP(hipEventRecord(e0, nullptr));
    hipLaunchKernelGGL(mfma_f64_probe, dim3(blocks), dim3(threads), 0, nullptr, out, iters, 1.0, 2.0);
    CNH_HIP(hipEventRecord(e1, nullptr));
    CNH_HIP(hipEventSynchronize(e1));
    float ms = 0.0f;
    CNH_HIP(hipEventElapsedTime(&ms, e0, e1));
    CNH_HIP(hipEventDestroy(e0));
    CNH_HIP(hipEventDestroy(e1));
    CNH_HIP(hipFree(out));
    const double flop = 2048.0 * 4.0 * iters * (double)blocks * (threads / 64);
    *tflops = ms > 0.0f ? flop / ((double)ms * 1e9) : 0.0;
    return 0;
}

extern "C" int cnh_gemm_batch(int dtype, int njobs, const cnh_gemm_job* jobs, int overwrite, cnh_stream s) {
    CNH_CHECK(njobs >= 0 && (njobs == 0 || jobs != nullptr), -2, "cnh_gemm_batch: bad job list");
    CNH_CHECK(!overwrite || dtype == CNH_F64, -3, "cnh_gemm_batch: overwriting products are fp64 only");
    for (int i = 0; i < njobs; ++i)
        if (int rc = check_job(jobs[i]))
            return rc;
    hipStream_t st = as_stream(s);
    if (dtype == CNH_F64)
        return run_f64_batch(njobs, jobs, overwrite ? 1 : 0, st);
    for (int i = 0; i < njobs; ++i) {
        const cnh_gemm_job& j = jobs[i];
        if (j.M == 0 || j.N == 0 || j.K == 0)
            continue;
        int rc;
        switch (dtype) {
        case CNH_F32: rc = run_generic<float>((int)j.M, (int)j.N, (int)j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc, st); break;
        case CNH_I32: rc = run_generic<int32_t>((int)j.M, (int)j.N, (int)j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc, st); break;
        case CNH_I64: rc = run_generic<int64_t>((int)j.M, (int)j.N, (int)j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc, st); break;
        default: return set_error(-2, "unknown dtype %d", dtype);
        }
        if (rc)
            return rc;
    }
    return 0;
}

extern "C" int cnh_gemm_acc_batch(int dtype, int njobs, const cnh_gemm_job* jobs, cnh_stream s) {
    return cnh_gemm_batch(dtype, njobs, jobs, 0, s);
}

extern "C" int cnh_gemm_acc(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                            const void* B, int64_t ldb, void* C, int64_t ldc, cnh_stream s) {
    const cnh_gemm_job job{M, N, K, A, lda, B, ldb, C, ldc};
    return cnh_gemm_acc_batch(dtype, 1, &job, s);
}
