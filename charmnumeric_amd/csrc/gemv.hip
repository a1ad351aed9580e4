// Bandwidth-bound matvec over row-major tiles, and the 1-D partial accumulate.
// Upstream: every 2-D tile chare runs an Eigen GEMV on its sub-matrix and ships the partial rows
// to the 1-D owner, which adds them in arrival order (src/backend_internal.hpp:28-41,
// src/execute_node.cpp:116-273,489-583). Here one launch covers the whole tile grid: one
// wavefront per matrix row walks the column tiles in index order with 128-bit loads, so the
// matrix is read from HBM exactly once and the per-row sum has a fixed order.
#include "common.h"

#include <type_traits>
#include <vector>

using namespace cnh;

namespace {

struct ColTile {
    const void* base; // first element of tile (ti, tj)
    int64_t ld;       // row stride of that tile in elements
    int64_t ncols;    // columns held by that tile
    int64_t xoff;     // offset of its first column in x
};

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

template <typename A>
__device__ __forceinline__ A wave_sum(A v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        if (sizeof(A) == 8) {
            unsigned long long u;
            __builtin_memcpy(&u, &v, 8);
            unsigned lo = (unsigned)u, hi = (unsigned)(u >> 32);
            lo = __shfl_down(lo, off, 64);
            hi = __shfl_down(hi, off, 64);
            u = ((unsigned long long)hi << 32) | lo;
            A o;
            __builtin_memcpy(&o, &u, 8);
            v = v + o;
        } else {
            unsigned u;
            __builtin_memcpy(&u, &v, 4);
            u = __shfl_down(u, off, 64);
            A o;
            __builtin_memcpy(&o, &u, 4);
            v = v + o;
        }
    }
    return v;
}

constexpr int kWavesPerBlockDefault = 4;

// tiles[ti * ncol_tiles + tj]; row r belongs to tile row (r + row_shift) / tile_rows: a window that
// starts row_shift rows into its first tile row.
// Measured on MI355X (n = 16384, fp64): 4 loads in flight per lane 326 us, 8: 330-336, 2: 345;
// 1, 2 or 4 wavefronts per workgroup make no difference, 8 are slower. Large products take
// gemv_rows_xlds below instead.
template <typename T, bool VEC16, int kWavesPerBlock = 4, int kUnroll = 4>
__global__ __launch_bounds__(kWavesPerBlock * 64) void gemv_rows(const ColTile* __restrict__ tiles,
                                                                 int ncol_tiles, int64_t tile_rows,
                                                                 int64_t rows, int64_t row_shift,
                                                                 const T* __restrict__ x,
                                                                 T* __restrict__ y, int beta) {
    typedef typename Acc<T>::type A;
    constexpr int VEC = 16 / sizeof(T);
    typedef T P __attribute__((ext_vector_type(VEC)));
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (r >= rows)
        return;
    const int64_t ti = (r + row_shift) / tile_rows;
    const int64_t lr = r + row_shift - ti * tile_rows;
    A total = 0;
    for (int tj = 0; tj < ncol_tiles; ++tj) {
        const ColTile ct = tiles[ti * ncol_tiles + tj];
        const T* row = (const T*)ct.base + lr * ct.ld;
        const T* xv = x + ct.xoff;
        A acc[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            acc[u] = 0;
        int64_t c = 0;
        if (VEC16) {
            const int64_t step = 64 * VEC;
            for (; c + kUnroll * step <= ct.ncols; c += kUnroll * step) {
                P av[kUnroll], xs[kUnroll];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                    av[u] = __builtin_nontemporal_load(reinterpret_cast<const P*>(row + c + u * step + lane * VEC));
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                    xs[u] = *reinterpret_cast<const P*>(xv + c + u * step + lane * VEC);
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        acc[u] += (A)av[u][e] * (A)xs[u][e];
            }
            for (; c + step <= ct.ncols; c += step) {
                P av = *reinterpret_cast<const P*>(row + c + lane * VEC);
                P xs = *reinterpret_cast<const P*>(xv + c + lane * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    acc[0] += (A)av[e] * (A)xs[e];
            }
        }
        for (int64_t j = c + lane; j < ct.ncols; j += 64)
            acc[1] += (A)row[j] * (A)xv[j];
        A part = 0;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            part += acc[u];
        part = wave_sum<A>(part);
        total = tj == 0 ? part : total + part; // column tiles added in index order
    }
    if (lane == 0)
        y[r] = beta ? (T)((A)y[r] + total) : (T)total;
}

// The same matvec with x staged in LDS. In gemv_rows every wavefront reads all of x for its one row
// (from L2: as many bytes again as the matrix, and half of all load instructions); here a workgroup
// of kWaves wavefronts owns kWaves * kRows rows, copies the x of one column tile into LDS (64 KB)
// and every wavefront streams its rows' parts of that tile against it, column tiles in index
// order. Per lane the same elements meet in the same order as in gemv_rows, so the results are the
// same bits. Needs: 128-bit alignment, every column tile at most 64 KB of x wide, and the column
// tiles cut alike in every tile row.
constexpr int kXldsBytes = 65536;

// What a fused launch does besides the product (fp64 only): the vector formed on the way as
// xa + (S / den) * xb, S the sum of `num_count` values in a fixed order (x then receives the vector,
// every element written by exactly one workgroup), and the partial sums of w . y per workgroup.
struct GemvFuse {
    const double* xa;
    const double* xb;
    const double* num;
    int64_t num_count;
    const double* den;
    double* num_folded;
    const double* w;
    double* dot_partials;
    double* x_out;          // where the formed vector is stored (the launch's x)
    double* quotient_out;   // receives S / den when not null
};

template <typename T, int kWaves, int kRows, int kUnroll, bool FUSED = false>
__global__ __launch_bounds__(kWaves * 64) void gemv_rows_xlds(const ColTile* __restrict__ tiles, int ncol_tiles,
                                                              int64_t tile_rows, int64_t rows, int64_t row_shift,
                                                              const T* x, T* __restrict__ y,
                                                              int beta, GemvFuse f = GemvFuse()) {
    typedef typename Acc<T>::type A;
    constexpr int VEC = 16 / sizeof(T);
    typedef T P __attribute__((ext_vector_type(VEC)));
    __shared__ __attribute__((aligned(16))) T xs[kXldsBytes / sizeof(T)];
    __shared__ double fuse_lds[kWaves + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t r0 = ((int64_t)blockIdx.x * kWaves + wave) * kRows;
    A total[kRows];
#pragma unroll
    for (int q = 0; q < kRows; ++q)
        total[q] = 0;
    double factor = 0.0;
    if (FUSED && f.xa != nullptr) {
        // S: lane l of the first wavefront adds num[l], num[l + 64], ... in that order, then the
        // fixed lane tree; every workgroup forms the same bits
        if (wave == 0) {
            double sacc = 0.0;
            for (int64_t i = lane; i < f.num_count; i += 64)
                sacc += f.num[i];
            sacc = wave_sum<double>(sacc);
            if (lane == 0) {
                fuse_lds[kWaves] = sacc;
                if (blockIdx.x == 0 && f.num_folded != nullptr)
                    *f.num_folded = sacc;
            }
        }
        __syncthreads();
        factor = fuse_lds[kWaves] / f.den[0];
        if (blockIdx.x == 0 && threadIdx.x == 0 && f.quotient_out != nullptr)
            *f.quotient_out = factor;
    }
    // The elements of the vector this workgroup stores when it forms the vector itself: those with
    // the indices of its own rows (the matrix is square), which are also the only elements of w it
    // reads for the dot at the end, so w may be the vector being formed.
    const int64_t own_lo = (int64_t)blockIdx.x * kWaves * kRows, own_hi = own_lo + kWaves * kRows;
    for (int tj = 0; tj < ncol_tiles; ++tj) {
        const int64_t ncols = tiles[tj].ncols, xoff = tiles[tj].xoff;
        if (tj > 0)
            __syncthreads();       // everybody is done with the previous tile's x
        if (FUSED && f.xa != nullptr) {
            // x = xa + factor * xb, one rounding per operation (no contraction), kept in LDS and,
            // for this workgroup's own share, stored
#pragma clang fp contract(off)
            for (int64_t i = (int64_t)threadIdx.x * 2; i + 2 <= ncols; i += (int64_t)kWaves * 64 * 2) {
                const double2 a = *reinterpret_cast<const double2*>(f.xa + xoff + i);
                const double2 b = *reinterpret_cast<const double2*>(f.xb + xoff + i);
                double2 v;
                v.x = a.x + factor * b.x;
                v.y = a.y + factor * b.y;
                *reinterpret_cast<double2*>(reinterpret_cast<double*>(xs) + i) = v;
                const int64_t g = xoff + i;
                if (g >= own_lo && g < own_hi)
                    f.x_out[g] = v.x;
                if (g + 1 >= own_lo && g + 1 < own_hi)
                    f.x_out[g + 1] = v.y;
            }
            if ((ncols & 1) && threadIdx.x == 0) {
                const int64_t i = ncols - 1, g = xoff + i;
                const double v = f.xa[g] + factor * f.xb[g];
                reinterpret_cast<double*>(xs)[i] = v;
                if (g >= own_lo && g < own_hi)
                    f.x_out[g] = v;
            }
        } else {
        for (int64_t i = (int64_t)threadIdx.x * VEC; i + VEC <= ncols; i += (int64_t)kWaves * 64 * VEC)
            *reinterpret_cast<P*>(xs + i) = *reinterpret_cast<const P*>(x + xoff + i);
        for (int64_t i = ncols / VEC * VEC + threadIdx.x; i < ncols; i += kWaves * 64)
            xs[i] = x[xoff + i];
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kRows; ++q) {
            const int64_t r = r0 + q;
            if (r >= rows)
                continue;
            const int64_t ti = (r + row_shift) / tile_rows;
            const int64_t lr = r + row_shift - ti * tile_rows;
            const ColTile ct = tiles[ti * ncol_tiles + tj];
            const T* row = (const T*)ct.base + lr * ct.ld;
            A acc[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                acc[u] = 0;
            int64_t c = 0;
            const int64_t step = 64 * VEC;
            for (; c + kUnroll * step <= ncols; c += kUnroll * step) {
                P av[kUnroll], xv[kUnroll];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                    av[u] = __builtin_nontemporal_load(reinterpret_cast<const P*>(row + c + u * step + lane * VEC));
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                    xv[u] = *reinterpret_cast<const P*>(xs + c + u * step + lane * VEC);
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        acc[u] += (A)av[u][e] * (A)xv[u][e];
            }
            for (; c + step <= ncols; c += step) {
                P av = *reinterpret_cast<const P*>(row + c + lane * VEC);
                P xv = *reinterpret_cast<const P*>(xs + c + lane * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    acc[0] += (A)av[e] * (A)xv[e];
            }
            for (int64_t j = c + lane; j < ncols; j += 64)
                acc[1] += (A)row[j] * (A)xs[j];
            A part = 0;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                part += acc[u];
            part = wave_sum<A>(part);
            total[q] = tj == 0 ? part : total[q] + part; // column tiles added in index order
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int q = 0; q < kRows; ++q)
            if (r0 + q < rows)
                y[r0 + q] = beta ? (T)((A)y[r0 + q] + total[q]) : (T)total[q];
    }
    if (FUSED && f.w != nullptr) {
        // w . y over this workgroup's rows: a wavefront's rows in order, then the wavefronts in order
        if (lane == 0) {
#pragma clang fp contract(off)
            double d = 0.0;
#pragma unroll
            for (int q = 0; q < kRows; ++q)
                if (r0 + q < rows)
                    d += f.w[r0 + q] * (double)total[q];
            fuse_lds[wave] = d;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            double d = fuse_lds[0];
#pragma unroll
            for (int wv = 1; wv < kWaves; ++wv)
                d += fuse_lds[wv];
            f.dot_partials[blockIdx.x] = d;
        }
    }
}

int g_gemv_xlds = 1;   // 0: always one wavefront per row reading x from cache; 1: the LDS form where it applies

template <typename T>
__global__ __launch_bounds__(256) void axpy1_kernel(int64_t n, const T* __restrict__ p,
                                                    T* __restrict__ y) {
    typedef typename Acc<T>::type A;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        y[i] = (T)((A)y[i] + (A)p[i]);
}

template <typename T>
int run_gemv(const std::vector<ColTile>& tiles, int ncol_tiles, int64_t tile_rows, int64_t rows,
             int64_t row_shift, const void* x, void* y, int beta, hipStream_t st) {
    bool vec = ((uintptr_t)x & 15) == 0;
    constexpr int VEC = 16 / sizeof(T);
    for (const ColTile& t : tiles) {
        if (((uintptr_t)t.base & 15) || (t.ld % VEC) || (t.xoff % VEC))
            vec = false;
    }
    const void* dtiles = nullptr;
    if (int rc = desc_upload(tiles.data(), tiles.size() * sizeof(ColTile), st, &dtiles))
        return rc;
    // x staged in LDS: big aligned products whose column tiles are cut alike in every tile row
    if (vec && g_gemv_xlds > 0 && rows >= 8192) {
        bool ok = true;
        const int64_t tile_rows_used = (int64_t)tiles.size() / ncol_tiles;
        for (int tj = 0; tj < ncol_tiles && ok; ++tj) {
            ok = tiles[(size_t)tj].ncols * (int64_t)sizeof(T) <= kXldsBytes;
            for (int64_t ti = 1; ti < tile_rows_used && ok; ++ti)
                ok = tiles[(size_t)(ti * ncol_tiles + tj)].ncols == tiles[(size_t)tj].ncols &&
                     tiles[(size_t)(ti * ncol_tiles + tj)].xoff == tiles[(size_t)tj].xoff;
        }
        if (ok) {
            // 8 wavefronts per workgroup; rows per wavefront so that every CU still gets a workgroup
            // (n = 16384, fp64: 8 x 8 rows 311 us, 16 x 4 317, 8 x 4 318, 16 x 8 383, one row per
            // wavefront without LDS 327-333)
            constexpr int kW = 8;
            if (rows >= 16384) {
                const int64_t nb = (rows + kW * 8 - 1) / (kW * 8);
                hipLaunchKernelGGL((gemv_rows_xlds<T, kW, 8, 4>), dim3((unsigned)nb), dim3(kW * 64), 0, st,
                                   (const ColTile*)dtiles, ncol_tiles, tile_rows, rows, row_shift, (const T*)x,
                                   (T*)y, beta);
            } else {
                const int64_t nb = (rows + kW * 4 - 1) / (kW * 4);
                hipLaunchKernelGGL((gemv_rows_xlds<T, kW, 4, 4>), dim3((unsigned)nb), dim3(kW * 64), 0, st,
                                   (const ColTile*)dtiles, ncol_tiles, tile_rows, rows, row_shift, (const T*)x,
                                   (T*)y, beta);
            }
            CNH_HIP(hipGetLastError());
            return 0;
        }
    }
    constexpr int kWavesPerBlock = kWavesPerBlockDefault;
    int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
    CNH_CHECK(blocks < (1ll << 31), -3, "matvec with %lld rows is too large for one launch",
              (long long)rows);
    if (vec)
        hipLaunchKernelGGL((gemv_rows<T, true>), dim3((unsigned)blocks), dim3(kWavesPerBlock * 64),
                           0, st, (const ColTile*)dtiles, ncol_tiles, tile_rows, rows, row_shift,
                           (const T*)x, (T*)y, beta);
    else
        hipLaunchKernelGGL((gemv_rows<T, false>), dim3((unsigned)blocks), dim3(kWavesPerBlock * 64),
                           0, st, (const ColTile*)dtiles, ncol_tiles, tile_rows, rows, row_shift,
                           (const T*)x, (T*)y, beta);
    CNH_HIP(hipGetLastError());
    return 0;
}

int dispatch_gemv(int dtype, const std::vector<ColTile>& tiles, int ncol_tiles, int64_t tile_rows,
                  int64_t rows, const void* x, void* y, int beta, hipStream_t st, int64_t row_shift = 0) {
    switch (dtype) {
    case CNH_F32: return run_gemv<float>(tiles, ncol_tiles, tile_rows, rows, row_shift, x, y, beta, st);
    case CNH_F64: return run_gemv<double>(tiles, ncol_tiles, tile_rows, rows, row_shift, x, y, beta, st);
    case CNH_I32: return run_gemv<int32_t>(tiles, ncol_tiles, tile_rows, rows, row_shift, x, y, beta, st);
    case CNH_I64: return run_gemv<int64_t>(tiles, ncol_tiles, tile_rows, rows, row_shift, x, y, beta, st);
    }
    return set_error(-2, "unknown dtype %d", dtype);
}

} // namespace

namespace cnh {
void gemv_set_xlds(int on) { g_gemv_xlds = on; }
} // namespace cnh

extern "C" {

int cnh_gemv(int dtype, int64_t rows, int64_t cols, const void* A, int64_t lda, const void* x,
             void* y, int beta, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(rows >= 0 && cols >= 0 && lda >= cols, -2, "cnh_gemv: bad shape %lld x %lld, lda %lld",
              (long long)rows, (long long)cols, (long long)lda);
    CNH_CHECK(beta == 0 || beta == 1, -2, "cnh_gemv: beta must be 0 or 1");
    if (rows == 0)
        return 0;
    CNH_CHECK(y != nullptr && (cols == 0 || (A != nullptr && x != nullptr)), -2,
              "cnh_gemv: null pointer");
    std::vector<ColTile> tiles(1);
    tiles[0] = {A, lda, cols, 0};
    return dispatch_gemv(dtype, tiles, 1, rows, rows, x, y, beta, as_stream(s));
}

int cnh_gemv_tiles(int dtype, int64_t rows, int64_t cols, int32_t tile, const void* const* tptr,
                   const void* x, void* y, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(rows > 0 && cols > 0 && tile > 0, -2, "cnh_gemv_tiles: bad shape");
    CNH_CHECK(tptr && x && y, -2, "cnh_gemv_tiles: null pointer");
    int64_t gr = (rows + tile - 1) / tile, gc = (cols + tile - 1) / tile;
    std::vector<ColTile> tiles((size_t)(gr * gc));
    for (int64_t i = 0; i < gr; ++i)
        for (int64_t j = 0; j < gc; ++j) {
            const void* p = tptr[i * gc + j];
            CNH_CHECK(p != nullptr, -2, "cnh_gemv_tiles: tile (%lld,%lld) is null", (long long)i,
                      (long long)j);
            int64_t nc = std::min<int64_t>(tile, cols - j * tile);
            tiles[(size_t)(i * gc + j)] = {p, nc, nc, j * tile};
        }
    return dispatch_gemv(dtype, tiles, (int)gc, tile, rows, x, y, 0, as_stream(s));
}

int cnh_gemv_tiles_fused(int64_t rows, int64_t cols, int32_t tile, const void* const* tptr, void* x, void* y,
                         const cnh_gemv_fusion* fu, int64_t* n_partials, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(rows > 0 && cols > 0 && tile > 0, -2, "cnh_gemv_tiles_fused: bad shape");
    CNH_CHECK(tptr && x && y && fu, -2, "cnh_gemv_tiles_fused: null pointer");
    CNH_CHECK(rows >= 16384 && (int64_t)tile * 8 <= kXldsBytes && tile % 2 == 0 && cols % 2 == 0, -3,
              "cnh_gemv_tiles_fused: needs 16384 rows or more and even column tiles of at most %d columns",
              kXldsBytes / 8);
    const bool form_x = fu->xa != nullptr;
    CNH_CHECK(!form_x || (fu->xb && fu->num && fu->num_count >= 1 && fu->den), -2,
              "cnh_gemv_tiles_fused: the vector's parts are incomplete");
    CNH_CHECK(!form_x || (rows == cols && x != fu->xa && x != fu->xb), -2,
              "cnh_gemv_tiles_fused: a vector formed on the way needs a square matrix and a buffer of its own");
    {
        // y is written while x, xa, xb and w are still being read by other workgroups
        auto overlaps = [&](const void* q, int64_t n) {
            const char *a = static_cast<const char*>(y), *b = static_cast<const char*>(q);
            return q != nullptr && a < b + n * 8 && b < a + rows * 8;
        };
        CNH_CHECK(!overlaps(x, cols) && !overlaps(fu->xa, cols) && !overlaps(fu->xb, cols) && !overlaps(fu->w, rows),
                  -2, "cnh_gemv_tiles_fused: y overlaps one of the vectors the launch reads");
    }
    CNH_CHECK(fu->w == nullptr || fu->dot_partials != nullptr, -2, "cnh_gemv_tiles_fused: no room for the partial sums");
    int64_t gr = (rows + tile - 1) / tile, gc = (cols + tile - 1) / tile;
    std::vector<ColTile> tiles((size_t)(gr * gc));
    bool aligned = (((uintptr_t)x | (uintptr_t)fu->xa | (uintptr_t)fu->xb) & 15) == 0;
    for (int64_t i = 0; i < gr; ++i)
        for (int64_t j = 0; j < gc; ++j) {
            const void* p = tptr[i * gc + j];
            CNH_CHECK(p != nullptr, -2, "cnh_gemv_tiles_fused: tile (%lld,%lld) is null", (long long)i, (long long)j);
            int64_t nc = std::min<int64_t>(tile, cols - j * tile);
            tiles[(size_t)(i * gc + j)] = {p, nc, nc, j * tile};
            aligned = aligned && ((uintptr_t)p & 15) == 0 && nc % 2 == 0;
        }
    CNH_CHECK(aligned, -3, "cnh_gemv_tiles_fused: operands must be 16-byte aligned");
    constexpr int kW = 8, kR = 8;
    const int64_t nb = (rows + kW * kR - 1) / (kW * kR);
    CNH_CHECK(fu->w == nullptr || fu->dot_capacity >= nb, -3,
              "cnh_gemv_tiles_fused: %lld partial sums, room for %lld", (long long)nb, (long long)fu->dot_capacity);
    if (n_partials)
        *n_partials = nb;
    hipStream_t st = as_stream(s);
    const void* dtiles = nullptr;
    if (int rc = desc_upload(tiles.data(), tiles.size() * sizeof(ColTile), st, &dtiles))
        return rc;
    GemvFuse f;
    f.xa = (const double*)fu->xa;
    f.xb = (const double*)fu->xb;
    f.num = (const double*)fu->num;
    f.num_count = fu->num_count;
    f.den = (const double*)fu->den;
    f.num_folded = (double*)fu->num_folded;
    f.w = (const double*)fu->w;
    f.dot_partials = (double*)fu->dot_partials;
    f.x_out = (double*)x;
    f.quotient_out = form_x ? (double*)fu->quotient_out : nullptr;
    hipLaunchKernelGGL((gemv_rows_xlds<double, kW, kR, 4, true>), dim3((unsigned)nb), dim3(kW * 64), 0, st,
                       (const ColTile*)dtiles, (int)gc, (int64_t)tile, rows, (int64_t)0, (const double*)x,
                       (double*)y, 0, f);
    CNH_HIP(hipGetLastError());
    return 0;
}

static_assert(sizeof(cnh_gemv_panel) == sizeof(ColTile), "cnh_gemv_panel is the kernel's descriptor");

int cnh_gemv_panels(int dtype, int64_t rows, int32_t n_col_panels, int64_t tile_rows, int64_t row_shift,
                    int64_t n_panels, const cnh_gemv_panel* panels, const void* x, void* y,
                    cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(rows > 0 && n_col_panels > 0 && tile_rows > 0 && row_shift >= 0 && row_shift < tile_rows,
              -2, "cnh_gemv_panels: bad shape");
    CNH_CHECK(panels && x && y, -2, "cnh_gemv_panels: null pointer");
    const int64_t panel_rows = (rows + row_shift + tile_rows - 1) / tile_rows;
    CNH_CHECK(n_panels == panel_rows * n_col_panels, -2,
              "cnh_gemv_panels: %lld panels given, %lld x %d needed", (long long)n_panels,
              (long long)panel_rows, n_col_panels);
    std::vector<ColTile> tiles((size_t)n_panels);
    for (int64_t i = 0; i < n_panels; ++i) {
        CNH_CHECK(panels[i].base != nullptr && panels[i].ncols > 0 && panels[i].ld >= panels[i].ncols &&
                      panels[i].xoff >= 0,
                  -2, "cnh_gemv_panels: bad panel %lld", (long long)i);
        tiles[(size_t)i] = {panels[i].base, panels[i].ld, panels[i].ncols, panels[i].xoff};
    }
    return dispatch_gemv(dtype, tiles, n_col_panels, tile_rows, rows, x, y, 0, as_stream(s), row_shift);
}

int cnh_axpy1(int dtype, int64_t n, const void* partial, void* y, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(n >= 0, -2, "cnh_axpy1: negative length");
    if (n == 0)
        return 0;
    CNH_CHECK(partial && y, -2, "cnh_axpy1: null pointer");
    unsigned blocks = (unsigned)((n + 255) / 256);
    hipStream_t st = as_stream(s);
    switch (dtype) {
    case CNH_F32:
        hipLaunchKernelGGL(axpy1_kernel<float>, dim3(blocks), dim3(256), 0, st, n,
                           (const float*)partial, (float*)y);
        break;
    case CNH_F64:
        hipLaunchKernelGGL(axpy1_kernel<double>, dim3(blocks), dim3(256), 0, st, n,
                           (const double*)partial, (double*)y);
        break;
    case CNH_I32:
        hipLaunchKernelGGL(axpy1_kernel<int32_t>, dim3(blocks), dim3(256), 0, st, n,
                           (const int32_t*)partial, (int32_t*)y);
        break;
    case CNH_I64:
        hipLaunchKernelGGL(axpy1_kernel<int64_t>, dim3(blocks), dim3(256), 0, st, n,
                           (const int64_t*)partial, (int64_t*)y);
        break;
    default: return set_error(-2, "unknown dtype %d", dtype);
    }
    CNH_HIP(hipGetLastError());
    return 0;
}

} // extern "C"
