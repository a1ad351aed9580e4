// Synthetic inputs generated on the device with a counter-based SplitMix64: element k of a
// stream depends only on (seed, stream, k), so any partition can fill its own tile and the
// values match a host generator bit for bit. Upstream has no generator and no bulk upload
// (charmnumeric/random.py:4-5, charmnumeric/charmnumeric.py:863-878).
#include "common.h"

using namespace cnh;

namespace {

__device__ __forceinline__ unsigned long long splitmix(unsigned long long seed,
                                                       unsigned long long stream,
                                                       unsigned long long i) {
    unsigned long long s = seed * 0x9E3779B97F4A7C15ull + stream * 0xD1B54A32D192ED03ull + i;
    unsigned long long z = s + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ double u01(unsigned long long seed, unsigned long long stream,
                                      unsigned long long i) {
    return (double)(splitmix(seed, stream, i) >> 11) * 0x1.0p-53;
}

__global__ __launch_bounds__(256) void fill_uniform_kernel(double* __restrict__ out, int64_t n,
                                                           unsigned long long seed,
                                                           unsigned long long stream,
                                                           unsigned long long first, double lo,
                                                           double w) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < n; i += stride) {
        // one multiply and one add, separately rounded (no fused multiply-add)
        double prod = __dmul_rn(w, u01(seed, stream, first + (unsigned long long)i));
        out[i] = __dadd_rn(lo, prod);
    }
}

__global__ __launch_bounds__(256) void fill_cg_kernel(double* __restrict__ out, int64_t n,
                                                      int64_t row0, int64_t nrows, int64_t col0,
                                                      int64_t ncols, int64_t ld,
                                                      unsigned long long seed) {
    int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t i = blockIdx.y;
    if (j >= ncols || i >= nrows)
        return;
    int64_t gi = row0 + i, gj = col0 + j;
    double v;
    if (gi == gj) {
        v = 2.0;
    } else {
        double s = __dadd_rn(u01(seed, 0, (unsigned long long)(gi * n + gj)),
                             u01(seed, 0, (unsigned long long)(gj * n + gi)));
        v = s / (2.0 * (double)n);
    }
    out[i * ld + j] = v;
}

struct TileFill {
    int64_t ext[3], origin[3], gshape[3];
};

// One tile of a row-major global array: the counter of an element is its global flat index.
__global__ __launch_bounds__(256) void fill_tile_kernel(double* __restrict__ out, TileFill t,
                                                        unsigned long long seed,
                                                        unsigned long long stream, double lo,
                                                        double w) {
    const int64_t total = t.ext[0] * t.ext[1] * t.ext[2];
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < total; i += stride) {
        const int64_t l2 = i % t.ext[2];
        const int64_t l1 = (i / t.ext[2]) % t.ext[1];
        const int64_t l0 = i / (t.ext[2] * t.ext[1]);
        const int64_t g = ((t.origin[0] + l0) * t.gshape[1] + (t.origin[1] + l1)) * t.gshape[2] +
                          (t.origin[2] + l2);
        double prod = __dmul_rn(w, u01(seed, stream, (unsigned long long)g));
        out[i] = __dadd_rn(lo, prod);
    }
}

} // namespace

extern "C" {

int cnh_fill_uniform_tile(double* out, int ndims, const int64_t* ext, const int64_t* origin,
                          const int64_t* global_shape, uint64_t seed, uint64_t stream_id, double lo,
                          double hi, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(ndims >= 1 && ndims <= CNH_MAX_ND, -2, "cnh_fill_uniform_tile: ndims %d", ndims);
    CNH_CHECK(out && ext && origin && global_shape, -2, "cnh_fill_uniform_tile: null pointer");
    TileFill t;
    const int pad = CNH_MAX_ND - ndims;
    for (int d = 0; d < 3; ++d) {
        t.ext[d] = 1;
        t.origin[d] = 0;
        t.gshape[d] = 1;
    }
    int64_t total = 1;
    for (int d = 0; d < ndims; ++d) {
        CNH_CHECK(ext[d] >= 0 && origin[d] >= 0 && origin[d] + ext[d] <= global_shape[d], -2,
                  "cnh_fill_uniform_tile: tile leaves the array in dim %d", d);
        t.ext[pad + d] = ext[d];
        t.origin[pad + d] = origin[d];
        t.gshape[pad + d] = global_shape[d];
        total *= ext[d];
    }
    if (total == 0)
        return 0;
    int64_t want = (total + 255) / 256;
    unsigned blocks = (unsigned)(want > 65536 ? 65536 : want);
    hipLaunchKernelGGL(fill_tile_kernel, dim3(blocks), dim3(256), 0, as_stream(s), out, t,
                       (unsigned long long)seed, (unsigned long long)stream_id, lo, hi - lo);
    CNH_HIP(hipGetLastError());
    return 0;
}


int cnh_fill_uniform(double* out, int64_t n, uint64_t seed, uint64_t stream_id, uint64_t first,
                     double lo, double hi, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(n >= 0, -2, "cnh_fill_uniform: negative length");
    if (n == 0)
        return 0;
    CNH_CHECK(out != nullptr, -2, "cnh_fill_uniform: null pointer");
    int64_t want = (n + 255) / 256;
    unsigned blocks = (unsigned)(want > 65536 ? 65536 : want);
    hipLaunchKernelGGL(fill_uniform_kernel, dim3(blocks), dim3(256), 0, as_stream(s), out, n,
                       (unsigned long long)seed, (unsigned long long)stream_id,
                       (unsigned long long)first, lo, hi - lo);
    CNH_HIP(hipGetLastError());
    return 0;
}

int cnh_fill_cg_matrix(double* out, int64_t n, int64_t row0, int64_t nrows, int64_t col0,
                       int64_t ncols, int64_t ld, uint64_t seed, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(n > 0 && nrows >= 0 && ncols >= 0 && ld >= ncols, -2, "cnh_fill_cg_matrix: bad shape");
    if (nrows == 0 || ncols == 0)
        return 0;
    CNH_CHECK(out != nullptr, -2, "cnh_fill_cg_matrix: null pointer");
    CNH_CHECK(nrows <= 65535 * 1ll * 65535, -3, "too many rows");
    // grid.y is limited to 65535 rows per launch
    for (int64_t r = 0; r < nrows; r += 65535) {
        int64_t nr = nrows - r < 65535 ? nrows - r : 65535;
        dim3 grid((unsigned)((ncols + 255) / 256), (unsigned)nr);
        hipLaunchKernelGGL(fill_cg_kernel, grid, dim3(256), 0, as_stream(s), out + r * ld, n,
                           row0 + r, nr, col0, ncols, ld, (unsigned long long)seed);
        CNH_HIP(hipGetLastError());
    }
    return 0;
}

} // extern "C"
