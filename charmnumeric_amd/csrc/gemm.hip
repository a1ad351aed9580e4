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

// One C block and the panel products that accumulate into it, in order; a launch covers a list
// of such chains (a single product is a chain of one segment).
struct GemmSeg {
    const double* A;
    int64_t lda;
    const double* B;
    int64_t ldb;
    int32_t K, pad;
};
struct GemmChain {
    double* C;
    int64_t ldc;
    int32_t M, N;
    int32_t seg0, nseg; // segments [seg0, seg0 + nseg)
    int32_t blk0, nbm;  // first workgroup of the chain, tiles along M
};
static_assert(sizeof(GemmSeg) == 40 && sizeof(GemmChain) == 40, "descriptor tables are uploaded as bytes");

// WM x WN wavefronts per workgroup, each owning TM x TN tiles of 16x16; K advances BKT at a time.
// The fp64 matrix pipe needs two or more wavefronts per SIMD to stay busy (one wavefront issues at
// ~70% of the rate eight reach), hence the 8-wavefront shape for grids that give each CU a single
// workgroup. Global loads run two K steps ahead of the arithmetic (two register sets, one LDS
// buffer being filled while the other is read): one K step of matrix instructions is shorter than
// a trip to memory. A workgroup keeps its accumulators across the segments of its chain, so the
// panel products of one C block cost one pass over C however many K pieces they come in.
// KS = 2: the workgroup is two such sets of wavefronts; set g takes the K steps g, g + 2, ... of every
// segment into accumulators of its own (staging buffers of its own too), and at the end the second
// set hands its sums over through LDS and the first adds them, first + second, and stores. Twice
// the wavefronts per SIMD for grids that give a CU one workgroup; K must be a multiple of 2 * BKT.
template <int WM, int WN, int TM, int TN, int BKT, bool FULL, bool BUF = false, int KS = 1>
__global__ __launch_bounds__(WM * WN * 64 * KS) void gemm_f64_mfma(const GemmChain* __restrict__ chains,
                                                                   int nchains,
                                                                   const GemmSeg* __restrict__ segs,
                                                                   int nblocks, GemmChain only_chain,
                                                                   GemmSeg only_seg, int overwrite) {
    constexpr int NT = WM * WN * 64;   // lanes of one set
    constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
    constexpr int APT = BM * BKT / NT, BPT = BN * BKT / NT;   // doubles staged per lane
    static_assert(APT >= 2 && BPT >= 2 && APT % 2 == 0 && BPT % 2 == 0, "staging uses 128-bit loads");
    static_assert(BKT % APT == 0 && BN % BPT == 0, "a lane's run stays inside one row");
    // A stays row-major in LDS with rows of BKT + 1 doubles: the operand read of 16 consecutive
    // rows at one k then touches 16 different bank pairs. B is k-major with rows of BN + 16.
    constexpr int AP = BKT + 1;
    __shared__ double As_all[KS][2][BM][AP];
    __shared__ __attribute__((aligned(16))) double Bs_all[KS][2][BKT][BN + PAD];
    __shared__ double Cs[KS > 1 ? TM * TN * 4 : 1][KS > 1 ? NT : 1];
    const int set = KS > 1 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x / NT) : 0;   // the same for a whole wavefront
    double (*As)[BM][AP] = As_all[set];
    double (*Bs)[BKT][BN + PAD] = Bs_all[set];
    const int logical = xcd_remap(blockIdx.x, nblocks);
    // a lone product travels in the kernel arguments (chains == nullptr), lists in a table
    int ci = 0;
    if (chains != nullptr)
        while (ci + 1 < nchains && chains[ci + 1].blk0 <= logical)
            ++ci;
    const GemmChain ch = chains != nullptr ? chains[ci] : only_chain;
    const int M = ch.M, N = ch.N;
    const int local = logical - ch.blk0;
    const int bn = local / ch.nbm, bm = local - bn * ch.nbm;
    const int m0 = bm * BM, n0 = bn * BN;
    const int tid = KS > 1 ? (int)threadIdx.x % NT : (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // staging assignment: A tile BM rows x BKT k (APT along k), B tile BKT k x BN (BPT along n)
    const int a_row = tid / (BKT / APT), a_k = (tid % (BKT / APT)) * APT;
    const int b_k = tid / (BN / BPT), b_n = (tid % (BN / BPT)) * BPT;
    const int lr = lane & 15, lk = lane >> 4;

    v4d acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            acc[i][j] = (v4d){0.0, 0.0, 0.0, 0.0};

    for (int si = 0; si < ch.nseg; ++si) {
        const GemmSeg sg = chains != nullptr ? segs[ch.seg0 + si] : only_seg;
        const double* __restrict__ A = sg.A;
        const double* __restrict__ B = sg.B;
        const int64_t lda = sg.lda, ldb = sg.ldb;
        const int K = sg.K;
        if (si > 0)
            __syncthreads();   // the previous segment's last reads of LDS are done

        // BUF: buffer loads. The descriptor (base of this workgroup's rows of A, of its columns of
        // B, moved along K on the scalar unit) sits in scalar registers and a lane contributes one
        // 32-bit offset that never changes: no 64-bit address arithmetic on the vector unit, which
        // the fp64 matrix instructions compete with (3-6 % on the 256 x 2048 x 4096 product).
        typedef int v4i __attribute__((ext_vector_type(4)));
        const int a_off = BUF ? (int)((a_row * lda + a_k) * 8) : 0;
        const int b_off = BUF ? (int)((b_k * ldb + b_n) * 8) : 0;
        auto fetch = [&](int k0, double (&ra)[APT], double (&rb)[BPT]) {
            if (BUF) {
                const __amdgpu_buffer_rsrc_t da = __builtin_amdgcn_make_buffer_rsrc(
                    (void*)(A + (int64_t)m0 * lda + k0), 0, 0x7fffffff, 0x00020000);
                const __amdgpu_buffer_rsrc_t db = __builtin_amdgcn_make_buffer_rsrc(
                    (void*)(B + (int64_t)k0 * ldb + n0), 0, 0x7fffffff, 0x00020000);
#pragma unroll
                for (int j = 0; j < APT; j += 2) {
                    const v4i v = __builtin_amdgcn_raw_buffer_load_b128(da, a_off + j * 8, 0, 0);
                    v2d d;
                    __builtin_memcpy(&d, &v, 16);
                    ra[j] = d[0];
                    ra[j + 1] = d[1];
                }
#pragma unroll
                for (int j = 0; j < BPT; j += 2) {
                    const v4i v = __builtin_amdgcn_raw_buffer_load_b128(db, b_off + j * 8, 0, 0);
                    v2d d;
                    __builtin_memcpy(&d, &v, 16);
                    rb[j] = d[0];
                    rb[j + 1] = d[1];
                }
                return;
            }
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

        // Step t multiplies LDS buffer t&1, which holds K slice t. Register set t&1 receives
        // slice t+2 while that runs; the other set (slice t+1, requested a step earlier) goes to
        // LDS after it.
        const int nk = (K + BKT - 1) / BKT / KS;          // K steps of this set
        auto kof = [&](int step) { return (step * KS + set) * BKT; };
        double ra0[APT], rb0[BPT], ra1[APT], rb1[BPT];
        fetch(kof(0), ra0, rb0);
        if (nk > 1)
            fetch(kof(1), ra1, rb1);
        stage(0, ra0, rb0);
        __syncthreads();
        // At the top of every round LDS buffer 0 holds slice t and register set 1 slice t + 1.
        // The steady-state rounds carry no conditions, so that the compiler's wait counts leave
        // the younger pair of loads in flight while the older pair is stored.
        int t = 0;
        for (; t + 3 < nk; t += 2) {
            fetch(kof(t + 2), ra0, rb0);
            multiply(0);
            stage(1, ra1, rb1);
            __syncthreads();
            fetch(kof(t + 3), ra1, rb1);
            multiply(1);
            stage(0, ra0, rb0);
            __syncthreads();
        }
        if (t + 2 < nk)
            fetch(kof(t + 2), ra0, rb0);
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
    }
    if (KS > 1) {
        // the second set's sums go through LDS, lane to lane; the first set adds them to its own
        if (set == 1) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        Cs[(i * TN + j) * 4 + r][tid] = acc[i][j][r];
        }
        __syncthreads();
        if (set == 1)
            return;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[i][j][r] += Cs[(i * TN + j) * 4 + r][tid];
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
                    double* c = ch.C + (int64_t)row * ch.ldc + col;
                    *c = overwrite ? acc[i][j][r] : *c + acc[i][j][r];
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
