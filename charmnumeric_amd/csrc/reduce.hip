// Deterministic reductions: dot, sum, sum of squared differences, max |a-b|.
// Upstream REDUCE is a per-tile Eigen/KokkosBlas dot followed by a Charm++ reduction that adds
// the contributions one after the other (src/executor_reduce.cpp:8-119,
// src/executor_reducer.cpp:11-57). Here: stage 1 — every workgroup reduces a fixed slice with
// 128-bit loads, a wavefront shuffle tree and an LDS tree; stage 2 — one workgroup folds the
// slices of all tiles, in slot order, in a fixed tree. The workgroup
// count depends only on the element counts, so results never depend on scheduling.
#include "common.h"

#include <vector>

using namespace cnh;

namespace {

enum Mode { M_DOT = 0, M_SUM = 1, M_SUMSQ_DIFF = 2, M_MAXABS_DIFF = 3 };

struct Chunk {
    const void* a;
    const void* b;
    int64_t n;
    int64_t per_block; // elements per workgroup (multiple of 512)
    int32_t blk0;      // first stage-1 workgroup / first partial slot
    int32_t nblk;
};

constexpr int kThreads = 256;
// Stage 1 runs 512 lanes a workgroup and stage 2 one workgroup of 1024: over 2^24 doubles the pair took
// 23.6 us with 256 and 256, 22.9 us with 256 and 1024, 22.45 us with 512 and 1024 (stage 2 then reads
// its 2048 slots two to a lane instead of eight).
constexpr int kStage1Threads = 512;
constexpr int kStage2Threads = 1024;
constexpr int kMaxBlocksPerChunk = 65536;

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

template <typename A, int MODE>
__device__ __forceinline__ A combine(A x, A y) {
    if (MODE == M_MAXABS_DIFF)
        return x > y ? x : y;
    return x + y;
}

template <typename T, typename A, int MODE>
__device__ __forceinline__ A term(T a, T b) {
    if (MODE == M_DOT)
        return (A)a * (A)b;
    if (MODE == M_SUM)
        return (A)a;
    if (MODE == M_SUMSQ_DIFF) {
        A d = (A)a - (A)b;
        return d * d;
    }
    A d = (A)a - (A)b;
    return d < (A)0 ? (A)0 - d : d;
}

template <typename A>
__device__ __forceinline__ A shfl_down_any(A v, int off) {
    if (sizeof(A) == 8) {
        unsigned long long u;
        __builtin_memcpy(&u, &v, 8);
        unsigned lo = (unsigned)u, hi = (unsigned)(u >> 32);
        lo = __shfl_down(lo, off, 64);
        hi = __shfl_down(hi, off, 64);
        u = ((unsigned long long)hi << 32) | lo;
        A r;
        __builtin_memcpy(&r, &u, 8);
        return r;
    } else {
        unsigned u;
        __builtin_memcpy(&u, &v, 4);
        u = __shfl_down(u, off, 64);
        A r;
        __builtin_memcpy(&r, &u, 4);
        return r;
    }
}

// Wavefront shuffle tree, then an LDS tree over the wavefronts of the workgroup.
template <typename A, int MODE, int THREADS>
__device__ __forceinline__ A block_reduce(A v, A* lds) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
        v = combine<A, MODE>(v, shfl_down_any<A>(v, off));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0)
        lds[wave] = v;
    __syncthreads();
    constexpr int NW = THREADS / 64;
    if (threadIdx.x == 0) {
        A r = lds[0];
#pragma unroll
        for (int w = 1; w < NW; ++w)
            r = combine<A, MODE>(r, lds[w]);
        v = r;
    }
    __syncthreads();
    return v;
}

template <typename T, int MODE, int THREADS>
__device__ __forceinline__ typename Acc<T>::type slice_reduce(const T* a, const T* b, int64_t lo,
                                                               int64_t hi) {
    typedef typename Acc<T>::type A;
    constexpr int VEC = 16 / sizeof(T);
    typedef T P __attribute__((ext_vector_type(VEC)));
    constexpr int U = 4; // independent 128-bit loads in flight per operand
    A acc0 = 0, acc1 = 0;
    const bool two = MODE != M_SUM;
    const bool same = !two || a == b;
    const bool aligned = (((uintptr_t)(a + lo)) & 15) == 0 &&
                         (!two || (((uintptr_t)(b + lo)) & 15) == 0);
    int64_t i = lo + (int64_t)threadIdx.x * VEC;
    if (aligned) {
        const int64_t stride = (int64_t)THREADS * VEC;
        for (; i + (U - 1) * stride + VEC <= hi; i += U * stride) {
            P av[U], bv[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
                av[u] = __builtin_nontemporal_load(reinterpret_cast<const P*>(a + i + u * stride));
#pragma unroll
            for (int u = 0; u < U; ++u)
                bv[u] = same ? av[u]
                             : __builtin_nontemporal_load(reinterpret_cast<const P*>(b + i + u * stride));
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if (u & 1)
                        acc1 = combine<A, MODE>(acc1, term<T, A, MODE>(av[u][e], bv[u][e]));
                    else
                        acc0 = combine<A, MODE>(acc0, term<T, A, MODE>(av[u][e], bv[u][e]));
                }
        }
        for (; i + VEC <= hi; i += stride) {
            P a0 = *reinterpret_cast<const P*>(a + i);
            P b0 = a0;
            if (!same)
                b0 = *reinterpret_cast<const P*>(b + i);
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                acc0 = combine<A, MODE>(acc0, term<T, A, MODE>(a0[e], b0[e]));
        }
        // ragged end of the slice: fewer than VEC elements
        if (i < hi) {
            for (int64_t j = i; j < hi; ++j)
                acc0 = combine<A, MODE>(acc0, term<T, A, MODE>(a[j], two ? b[j] : a[j]));
        }
    } else {
        for (int64_t j = lo + threadIdx.x; j < hi; j += THREADS)
            acc0 = combine<A, MODE>(acc0, term<T, A, MODE>(a[j], two ? b[j] : a[j]));
    }
    return combine<A, MODE>(acc0, acc1);
}

// Stage 1 of one workgroup: reduce slice `rel` of chunk `c` into its slot.
template <typename T, int MODE>
__device__ __forceinline__ void stage1_body(const Chunk& c, int rel, typename Acc<T>::type* lds,
                                            typename Acc<T>::type* slot) {
    typedef typename Acc<T>::type A;
    const int64_t b0 = (int64_t)rel * c.per_block;
    const int64_t b1 = b0 + c.per_block < c.n ? b0 + c.per_block : c.n;
    A v = slice_reduce<T, MODE, kStage1Threads>((const T*)c.a, (const T*)c.b, b0, b1);
    v = block_reduce<A, MODE, kStage1Threads>(v, lds);
    if (threadIdx.x == 0)
        *slot = v;
}

// Stage 2 for one chunk: a fixed tree over its `nb` slots (every lane returns the value lane 0 holds
// only in lane 0).
template <typename T, int MODE>
__device__ __forceinline__ typename Acc<T>::type stage2_chunk(const typename Acc<T>::type* slots,
                                                               int nb, typename Acc<T>::type* lds) {
    typedef typename Acc<T>::type A;
    A v = 0;
    for (int i = threadIdx.x; i < nb; i += kStage2Threads)
        v = combine<A, MODE>(v, slots[i]);
    return block_reduce<A, MODE, kStage2Threads>(v, lds);
}

template <typename T, int MODE>
__global__ __launch_bounds__(kStage1Threads) void reduce_stage1(const Chunk* __restrict__ chunks,
                                                                int nchunk,
                                                                typename Acc<T>::type* __restrict__ partials) {
    typedef typename Acc<T>::type A;
    __shared__ A lds[kStage1Threads / 64];
    int lo = 0, hi = nchunk - 1;
    const int blk = blockIdx.x;
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (chunks[mid].blk0 <= blk)
            lo = mid;
        else
            hi = mid - 1;
    }
    const Chunk c = chunks[lo];
    stage1_body<T, MODE>(c, blk - c.blk0, lds, partials + blk);
}

// One workgroup folds the slots of all chunks (they are consecutive) in one pass: lane t takes slots
// t, t + 256, ... in that order, then the fixed tree. One trip to memory for all slots instead of
// one per chunk (a chunk at a time cost 4.6 us for the four partitions of 2^24 elements).
template <typename T, int MODE>
__global__ __launch_bounds__(kStage2Threads) void reduce_stage2(int nslots,
                                                                const typename Acc<T>::type* __restrict__ partials,
                                                                T* __restrict__ out) {
    typedef typename Acc<T>::type A;
    __shared__ A lds[kStage2Threads / 64];
    A v = stage2_chunk<T, MODE>(partials, nslots, lds);
    if (threadIdx.x == 0)
        *out = (T)v;
}

// The same two stages for a single chunk handed over by value: no descriptor table on the device.
template <typename T, int MODE>
__global__ __launch_bounds__(kStage1Threads) void reduce_stage1_one(const Chunk c,
                                                                    typename Acc<T>::type* __restrict__ partials) {
    typedef typename Acc<T>::type A;
    __shared__ A lds[kStage1Threads / 64];
    stage1_body<T, MODE>(c, blockIdx.x, lds, partials + blockIdx.x);
}

template <typename T, int MODE>
__global__ __launch_bounds__(kStage2Threads) void reduce_stage2_one(int nblk,
                                                                    const typename Acc<T>::type* __restrict__ partials,
                                                                    T* __restrict__ out) {
    typedef typename Acc<T>::type A;
    __shared__ A lds[kStage2Threads / 64];
    A v = stage2_chunk<T, MODE>(partials, nblk, lds);
    if (threadIdx.x == 0)
        *out = (T)v;
}

// Short single tile: one workgroup of 1024 lanes does everything in one launch.
template <typename T, int MODE>
__global__ __launch_bounds__(1024) void reduce_single(const T* __restrict__ a,
                                                      const T* __restrict__ b, int64_t n,
                                                      T* __restrict__ out) {
    typedef typename Acc<T>::type A;
    __shared__ A lds[1024 / 64];
    A v = slice_reduce<T, MODE, 1024>(a, b, 0, n);
    v = block_reduce<A, MODE, 1024>(v, lds);
    if (threadIdx.x == 0)
        *out = (T)v;
}

// Sequential sum of per-tile partials in index order (the upstream reducer's a += b loop).
template <typename T>
__global__ void reduce_final_seq(const T* __restrict__ partials, int n, T* __restrict__ out) {
    typedef typename Acc<T>::type A;
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        A acc = (A)partials[0];
        for (int i = 1; i < n; ++i)
            acc += (A)partials[i];
        *out = (T)acc;
    }
}

constexpr int64_t kSingleMax = 1 << 16;

// How one contiguous chunk is cut into stage-1 slices: about 8192 elements per workgroup, at most
// kMaxBlocksPerChunk workgroups, slice lengths a multiple of 512. Depends on n only.
Chunk plan_chunk(const void* a, const void* b, int64_t n, int blk0) {
    Chunk c;
    c.a = a;
    c.b = b;
    c.n = n;
    int64_t nb = (n + 8191) / 8192;
    if (nb < 1)
        nb = 1;
    if (nb > kMaxBlocksPerChunk)
        nb = kMaxBlocksPerChunk;
    int64_t per = (n + nb - 1) / nb;
    per = (per + 511) / 512 * 512;
    if (per < 512)
        per = 512;
    nb = n > 0 ? (n + per - 1) / per : 1;
    c.per_block = per;
    c.blk0 = blk0;
    c.nblk = (int)nb;
    return c;
}

template <typename T, int MODE>
int run_tiles(int n_tiles, const void* const* a, const void* const* b, const int64_t* n, void* out,
              hipStream_t st) {
    CNH_CHECK(n_tiles >= 1, -2, "reduction over %d tiles", n_tiles);
    CNH_CHECK(out != nullptr && a != nullptr && n != nullptr, -2, "null argument");
    const bool two = MODE != M_SUM;
    CNH_CHECK(!two || b != nullptr, -2, "null second operand");
    for (int t = 0; t < n_tiles; ++t) {
        CNH_CHECK(n[t] >= 0, -2, "tile %d has negative length", t);
        CNH_CHECK(n[t] == 0 || (a[t] != nullptr && (!two || b[t] != nullptr)), -2,
                  "tile %d has a null pointer", t);
    }
    if (n_tiles == 1 && n[0] <= kSingleMax) {
        hipLaunchKernelGGL((reduce_single<T, MODE>), dim3(1), dim3(1024), 0, st, (const T*)a[0],
                           (const T*)(two ? b[0] : a[0]), n[0], (T*)out);
        CNH_HIP(hipGetLastError());
        return 0;
    }
    std::vector<Chunk> chunks(n_tiles);
    int blocks = 0;
    for (int t = 0; t < n_tiles; ++t) {
        chunks[t] = plan_chunk(a[t], two ? b[t] : a[t], n[t], blocks);
        blocks += chunks[t].nblk;
    }
    typedef typename Acc<T>::type A;
    void* ws = nullptr;
    if (int rc = reduce_workspace(st, (size_t)blocks * sizeof(A), &ws))
        return rc;
    // The chunk table stays in device memory: handed over by value (8 chunks, 320 bytes of kernel
    // arguments) the same launch took 0.8 us longer.
    const void* dchunks = nullptr;
    if (int rc = desc_upload(chunks.data(), chunks.size() * sizeof(Chunk), st, &dchunks))
        return rc;
    hipLaunchKernelGGL((reduce_stage1<T, MODE>), dim3(blocks), dim3(kStage1Threads), 0, st,
                       (const Chunk*)dchunks, n_tiles, (A*)ws);
    CNH_HIP(hipGetLastError());
    hipLaunchKernelGGL((reduce_stage2<T, MODE>), dim3(1), dim3(kStage2Threads), 0, st, blocks, (const A*)ws,
                       (T*)out);
    CNH_HIP(hipGetLastError());
    return 0;
}

template <int MODE>
int dispatch_tiles(int dtype, int n_tiles, const void* const* a, const void* const* b,
                   const int64_t* n, void* out, hipStream_t st) {
    switch (dtype) {
    case CNH_F32: return run_tiles<float, MODE>(n_tiles, a, b, n, out, st);
    case CNH_F64: return run_tiles<double, MODE>(n_tiles, a, b, n, out, st);
    case CNH_I32: return run_tiles<int32_t, MODE>(n_tiles, a, b, n, out, st);
    case CNH_I64: return run_tiles<int64_t, MODE>(n_tiles, a, b, n, out, st);
    }
    return set_error(-2, "unknown dtype %d", dtype);
}

// ---- dot without any allocation ----
// Slots for the stage-1 partials of cnh_dot_partial_noalloc: part of the code object, so every
// device the library runs on holds its own copy from load until the process ends.
constexpr int kScratchSlots = 32768;                      // 256 KiB
constexpr int64_t kScratchMaxN = (int64_t)kScratchSlots * 8192;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned long long scratch[kScratchSlots];
void* g_scratch_ptr[kMaxDevices] = {};

template <typename T>
int run_dot_noalloc(int64_t n, const void* a, const void* b, void* out, void* slots, hipStream_t st) {
    typedef typename Acc<T>::type A;
    if (n <= kSingleMax) {
        hipLaunchKernelGGL((reduce_single<T, M_DOT>), dim3(1), dim3(1024), 0, st, (const T*)a,
                           (const T*)b, n, (T*)out);
        CNH_HIP(hipGetLastError());
        return 0;
    }
    const Chunk c = plan_chunk(a, b, n, 0);
    CNH_CHECK(c.nblk <= kScratchSlots, -3, "cnh_dot_partial_noalloc: %d partial slots needed, %d held",
              c.nblk, kScratchSlots);
    hipLaunchKernelGGL((reduce_stage1_one<T, M_DOT>), dim3(c.nblk), dim3(kStage1Threads), 0, st, c,
                       (A*)slots);
    CNH_HIP(hipGetLastError());
    hipLaunchKernelGGL((reduce_stage2_one<T, M_DOT>), dim3(1), dim3(kStage2Threads), 0, st, c.nblk,
                       (const A*)slots, (T*)out);
    CNH_HIP(hipGetLastError());
    return 0;
}

} // namespace

namespace {
// Folding the partials a kernel that reduced on the way left behind (one per wavefront, in launch
// order; sums, or maxima of non-negative values). Few of them: one workgroup, lane t takes slots
// t, t + 1024, ... in that order, then the fixed tree. Many: first every workgroup of a grid folds
// its own run of `per` consecutive slots the same way into one value, then one workgroup folds
// those. The grouping depends on n only.
template <bool MAXV>
__global__ __launch_bounds__(1024) void fold_slots(const double* __restrict__ slots, int64_t n,
                                                   double* __restrict__ out) {
    __shared__ double lds[1024 / 64];
    double v = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        const double o = slots[i];
        v = MAXV ? (o > v ? o : v) : v + o;
    }
    v = block_reduce<double, MAXV ? M_MAXABS_DIFF : M_SUM, 1024>(v, lds);
    if (threadIdx.x == 0)
        *out = v;
}
template <bool MAXV>
__global__ __launch_bounds__(kThreads) void fold_slots_runs(const double* __restrict__ slots, int64_t n,
                                                            int64_t per, double* __restrict__ runs) {
    __shared__ double lds[kThreads / 64];
    const int64_t lo = (int64_t)blockIdx.x * per, hi = lo + per < n ? lo + per : n;
    double v = 0.0;
    for (int64_t i = lo + threadIdx.x; i < hi; i += kThreads) {
        const double o = slots[i];
        v = MAXV ? (o > v ? o : v) : v + o;
    }
    v = block_reduce<double, MAXV ? M_MAXABS_DIFF : M_SUM, kThreads>(v, lds);
    if (threadIdx.x == 0)
        runs[blockIdx.x] = v;
}

// Several slot vectors at once (blockIdx.y picks the vector), each a sum or a maximum: the
// reductions a group kernel carried along are folded by the same one or two launches.
// Up to this many partials per vector one workgroup of 1024 lanes folds by itself (64 loads per
// lane, all in flight together); beyond it a grid folds runs first.
constexpr int64_t kFoldSingleMax = 8192;
struct FoldMany {
    double* vec[kFoldMaxVectors];
    double* out[kFoldMaxVectors];
    int maximum[kFoldMaxVectors];
};
__global__ __launch_bounds__(kThreads) void fold_many_runs(int64_t n, int64_t per, FoldMany f) {
    __shared__ double lds[kThreads / 64];
    const int q = blockIdx.y;
    const double* __restrict__ src = f.vec[q];
    const bool maxv = f.maximum[q] != 0;
    const int64_t lo = (int64_t)blockIdx.x * per, hi = lo + per < n ? lo + per : n;
    double v = 0.0;
    for (int64_t i = lo + threadIdx.x; i < hi; i += kThreads) {
        const double o = src[i];
        v = maxv ? (o > v ? o : v) : v + o;
    }
    v = maxv ? block_reduce<double, M_MAXABS_DIFF, kThreads>(v, lds) : block_reduce<double, M_SUM, kThreads>(v, lds);
    if (threadIdx.x == 0)
        f.vec[q][n + blockIdx.x] = v;
}
__global__ __launch_bounds__(1024) void fold_many(int64_t first, int64_t count, FoldMany f) {
    __shared__ double lds[1024 / 64];
    const int q = blockIdx.y;
    const double* __restrict__ src = f.vec[q] + first;
    const bool maxv = f.maximum[q] != 0;
    double v = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += 1024) {
        const double o = src[i];
        v = maxv ? (o > v ? o : v) : v + o;
    }
    v = maxv ? block_reduce<double, M_MAXABS_DIFF, 1024>(v, lds) : block_reduce<double, M_SUM, 1024>(v, lds);
    if (threadIdx.x == 0)
        *f.out[q] = v;
}

// The sum of n partial results in the order a group launch uses when it is handed them as a summed
// scalar (cnh_launch_group_sums): 256 lanes take running sums a lane stride apart, a butterfly
// combines the lanes of each wavefront, the four wavefronts are added left to right.
__global__ __launch_bounds__(256) void fold_sums_f64(const double* __restrict__ p, int n, double* __restrict__ out) {
    __shared__ double part[4];
    double v = 0;
    for (int j = threadIdx.x; j < n; j += 256)
        v += p[j];
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        v += __shfl_xor(v, m, 64);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0)
        *out = ((part[0] + part[1]) + part[2]) + part[3];
}
} // namespace

namespace cnh {
// Every vector holds n entries with room for kFoldRuns more behind them.
int reduce_slots_f64_many(int nvec, const int* maximum, double* const* vecs, int64_t n, double* const* outs,
                          hipStream_t st) {
    CNH_CHECK(vecs != nullptr && outs != nullptr && n >= 1 && nvec >= 1 && nvec <= kFoldMaxVectors, -2,
              "reduce_slots_f64_many: bad arguments");
    FoldMany f;
    for (int q = 0; q < kFoldMaxVectors; ++q) {
        f.vec[q] = q < nvec ? vecs[q] : nullptr;
        f.out[q] = q < nvec ? outs[q] : nullptr;
        f.maximum[q] = q < nvec ? maximum[q] : 0;
    }
    int64_t first = 0, count = n;
    if (n > kFoldSingleMax) {
        int64_t per = (n + kFoldRuns - 1) / kFoldRuns;
        per = (per + 1023) / 1024 * 1024;               // whole passes of a workgroup
        const int64_t runs = (n + per - 1) / per;
        hipLaunchKernelGGL(fold_many_runs, dim3((unsigned)runs, (unsigned)nvec), dim3(kThreads), 0, st, n, per, f);
        CNH_HIP(hipGetLastError());
        first = n;
        count = runs;
    }
    hipLaunchKernelGGL(fold_many, dim3(1, (unsigned)nvec), dim3(1024), 0, st, first, count, f);
    CNH_HIP(hipGetLastError());
    return 0;
}

// `slots` must have room for kFoldRuns more doubles behind its n entries (the run sums).
int reduce_slots_f64(bool maximum, double* slots, int64_t n, double* out, hipStream_t st) {
    CNH_CHECK(slots != nullptr && out != nullptr && n >= 1, -2, "reduce_slots_f64: bad arguments");
    const double* src = slots;
    int64_t count = n;
    if (n > 8192) {
        int64_t per = (n + kFoldRuns - 1) / kFoldRuns;
        per = (per + 1023) / 1024 * 1024;               // whole passes of a workgroup
        const int64_t runs = (n + per - 1) / per;
        double* tmp = slots + n;
        if (maximum)
            hipLaunchKernelGGL(fold_slots_runs<true>, dim3((unsigned)runs), dim3(kThreads), 0, st, slots, n, per, tmp);
        else
            hipLaunchKernelGGL(fold_slots_runs<false>, dim3((unsigned)runs), dim3(kThreads), 0, st, slots, n, per, tmp);
        CNH_HIP(hipGetLastError());
        src = tmp;
        count = runs;
    }
    if (maximum)
        hipLaunchKernelGGL(fold_slots<true>, dim3(1), dim3(1024), 0, st, src, count, out);
    else
        hipLaunchKernelGGL(fold_slots<false>, dim3(1), dim3(1024), 0, st, src, count, out);
    CNH_HIP(hipGetLastError());
    return 0;
}

// Called by cnh_init with `device` current: resolves this device's copy of the scratch array.
int reduce_scratch_init(int device) {
    CNH_CHECK(device >= 0 && device < kMaxDevices, -2, "device %d beyond the %d the scratch table holds",
              device, kMaxDevices);
    if (g_scratch_ptr[device])
        return 0;
    void* p = nullptr;
    CNH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    CNH_CHECK(p != nullptr, -100, "hipGetSymbolAddress returned a null scratch address");
    g_scratch_ptr[device] = p;
    return 0;
}
} // namespace cnh

extern "C" {

int cnh_dot_partial_noalloc(int dtype, int64_t n, const void* a, const void* b, void* out,
                            cnh_stream s) {
    // no lazy initialisation here: selecting a device and resolving the scratch symbol are not
    // things to do under a caller's graph capture
    CNH_CHECK(current_device() >= 0, -100, "cnh_dot_partial_noalloc: call cnh_init first");
    CNH_CHECK(out != nullptr && n >= 0, -2, "cnh_dot_partial_noalloc: bad arguments");
    CNH_CHECK(n == 0 || (a != nullptr && b != nullptr), -2, "cnh_dot_partial_noalloc: null operand");
    CNH_CHECK(n <= kScratchMaxN, -3,
              "cnh_dot_partial_noalloc: %lld elements exceed the maximum of %lld",
              (long long)n, (long long)kScratchMaxN);
    const int dev = current_device();
    void* slots = dev >= 0 && dev < kMaxDevices ? g_scratch_ptr[dev] : nullptr;
    CNH_CHECK(slots != nullptr, -100, "cnh_dot_partial_noalloc: scratch of device %d not resolved", dev);
    hipStream_t st = as_stream(s);
    switch (dtype) {
    case CNH_F32: return run_dot_noalloc<float>(n, a, b, out, slots, st);
    case CNH_F64: return run_dot_noalloc<double>(n, a, b, out, slots, st);
    case CNH_I32: return run_dot_noalloc<int32_t>(n, a, b, out, slots, st);
    case CNH_I64: return run_dot_noalloc<int64_t>(n, a, b, out, slots, st);
    }
    return set_error(-2, "unknown dtype %d", dtype);
}


int cnh_dot_tiles(int dtype, int n_tiles, const void* const* a, const void* const* b,
                  const int64_t* n, void* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    return dispatch_tiles<M_DOT>(dtype, n_tiles, a, b, n, out, as_stream(s));
}

int cnh_dot_partial(int dtype, int64_t n, const void* a, const void* b, void* partial_slot,
                    cnh_stream s) {
    const void* aa[1] = {a};
    const void* bb[1] = {b};
    int64_t nn[1] = {n};
    return cnh_dot_tiles(dtype, 1, aa, bb, nn, partial_slot, s);
}

int cnh_reduce_final(int dtype, int n_partials, const void* partials, void* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(n_partials >= 1 && partials && out, -2, "cnh_reduce_final: bad arguments");
    hipStream_t st = as_stream(s);
    switch (dtype) {
    case CNH_F32:
        hipLaunchKernelGGL(reduce_final_seq<float>, dim3(1), dim3(64), 0, st, (const float*)partials,
                           n_partials, (float*)out);
        break;
    case CNH_F64:
        hipLaunchKernelGGL(reduce_final_seq<double>, dim3(1), dim3(64), 0, st,
                           (const double*)partials, n_partials, (double*)out);
        break;
    case CNH_I32:
        hipLaunchKernelGGL(reduce_final_seq<int32_t>, dim3(1), dim3(64), 0, st,
                           (const int32_t*)partials, n_partials, (int32_t*)out);
        break;
    case CNH_I64:
        hipLaunchKernelGGL(reduce_final_seq<int64_t>, dim3(1), dim3(64), 0, st,
                           (const int64_t*)partials, n_partials, (int64_t*)out);
        break;
    default: return set_error(-2, "unknown dtype %d", dtype);
    }
    CNH_HIP(hipGetLastError());
    return 0;
}

int cnh_fold_sums(const void* partials, int64_t count, void* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(partials && out && count >= 1 && count <= (1 << 20), -2, "cnh_fold_sums: bad arguments");
    hipLaunchKernelGGL(fold_sums_f64, dim3(1), dim3(256), 0, as_stream(s), (const double*)partials, (int)count,
                       (double*)out);
    CNH_HIP(hipGetLastError());
    return 0;
}

int cnh_sum_tiles(int dtype, int n_tiles, const void* const* a, const int64_t* n, void* out,
                  cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    return dispatch_tiles<M_SUM>(dtype, n_tiles, a, nullptr, n, out, as_stream(s));
}

int cnh_sumsq_diff_tiles(int n_tiles, const void* const* a, const void* const* b, const int64_t* n,
                         void* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    return run_tiles<double, M_SUMSQ_DIFF>(n_tiles, a, b, n, out, as_stream(s));
}

int cnh_maxabs_diff_tiles(int n_tiles, const void* const* a, const void* const* b,
                          const int64_t* n, void* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    return run_tiles<double, M_MAXABS_DIFF>(n_tiles, a, b, n, out, as_stream(s));
}

} // extern "C"
