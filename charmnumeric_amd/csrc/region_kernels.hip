// Strided N-D fill and copy kernels: SET_REGION scalar fill / region copy, halo pack/unpack.
// Upstream these are element-at-a-time odometer loops (src/executor_ast_visitor.cpp:149-207,
// :268-311) or one-thread-per-element Kokkos loops (src/executor_core.cpp:71-81); here one
// workgroup covers a run of the innermost dimension so that unit-stride rows coalesce.
#include "common.h"

#include <cstring>

using namespace cnh;

namespace {

struct RegionArgs {
    int64_t dstride[CNH_MAX_ND], dstart[CNH_MAX_ND], dstep[CNH_MAX_ND];
    int64_t sstride[CNH_MAX_ND], sstart[CNH_MAX_ND], sstep[CNH_MAX_ND];
    int64_t counts[CNH_MAX_ND]; // normalised to 3 dims, leading dims = 1
    int64_t nchunks;
};

constexpr int kBlock = 256;
constexpr int kPerThread = 4;

template <typename W, bool FILL>
__global__ __launch_bounds__(kBlock) void region_kernel(W* __restrict__ dst,
                                                        const W* __restrict__ src, W value,
                                                        RegionArgs a) {
    int64_t bid = blockIdx.x;
    int64_t outer = bid / a.nchunks;
    int64_t chunk = bid - outer * a.nchunks;
    int64_t i1 = outer % a.counts[1];
    int64_t i0 = outer / a.counts[1];
    int64_t dbase = (a.dstart[0] + i0 * a.dstep[0]) * a.dstride[0] +
                    (a.dstart[1] + i1 * a.dstep[1]) * a.dstride[1];
    int64_t sbase = 0;
    if (!FILL)
        sbase = (a.sstart[0] + i0 * a.sstep[0]) * a.sstride[0] +
                (a.sstart[1] + i1 * a.sstep[1]) * a.sstride[1];
    int64_t x0 = chunk * (kBlock * kPerThread) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
        int64_t x = x0 + (int64_t)k * kBlock;
        if (x < a.counts[2]) {
            int64_t d = dbase + (a.dstart[2] + x * a.dstep[2]) * a.dstride[2];
            if (FILL) {
                dst[d] = value;
            } else {
                int64_t s = sbase + (a.sstart[2] + x * a.sstep[2]) * a.sstride[2];
                dst[d] = src[s];
            }
        }
    }
}

// The strided copy with a change of element type on the way: dst = (D)src, C conversion rules
// (round to nearest even into floating point, truncation towards zero into integers).
template <typename S, typename D>
__global__ __launch_bounds__(kBlock) void convert_kernel(D* __restrict__ dst, const S* __restrict__ src,
                                                         RegionArgs a) {
    int64_t bid = blockIdx.x;
    int64_t outer = bid / a.nchunks;
    int64_t chunk = bid - outer * a.nchunks;
    int64_t i1 = outer % a.counts[1];
    int64_t i0 = outer / a.counts[1];
    int64_t dbase = (a.dstart[0] + i0 * a.dstep[0]) * a.dstride[0] +
                    (a.dstart[1] + i1 * a.dstep[1]) * a.dstride[1];
    int64_t sbase = (a.sstart[0] + i0 * a.sstep[0]) * a.sstride[0] +
                    (a.sstart[1] + i1 * a.sstep[1]) * a.sstride[1];
    int64_t x0 = chunk * (kBlock * kPerThread) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
        int64_t x = x0 + (int64_t)k * kBlock;
        if (x < a.counts[2])
            dst[dbase + (a.dstart[2] + x * a.dstep[2]) * a.dstride[2]] =
                (D)src[sbase + (a.sstart[2] + x * a.sstep[2]) * a.sstride[2]];
    }
}

template <typename S>
int launch_convert(int dst_dtype, void* dst, const void* src, const RegionArgs& a, unsigned blocks,
                   hipStream_t st) {
    switch (dst_dtype) {
    case CNH_F32:
        hipLaunchKernelGGL((convert_kernel<S, float>), dim3(blocks), dim3(kBlock), 0, st, (float*)dst, (const S*)src, a);
        break;
    case CNH_F64:
        hipLaunchKernelGGL((convert_kernel<S, double>), dim3(blocks), dim3(kBlock), 0, st, (double*)dst, (const S*)src, a);
        break;
    case CNH_I32:
        hipLaunchKernelGGL((convert_kernel<S, int32_t>), dim3(blocks), dim3(kBlock), 0, st, (int32_t*)dst, (const S*)src, a);
        break;
    case CNH_I64:
        hipLaunchKernelGGL((convert_kernel<S, int64_t>), dim3(blocks), dim3(kBlock), 0, st, (int64_t*)dst, (const S*)src, a);
        break;
    default: return set_error(-2, "cnh_convert_region: unknown destination dtype %d", dst_dtype);
    }
    CNH_HIP(hipGetLastError());
    return 0;
}

__global__ __launch_bounds__(256) void zero_kernel(uint4* __restrict__ p, size_t n16,
                                                   unsigned char* __restrict__ tail_base,
                                                   size_t tail) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < n16; k += stride)
        p[k] = make_uint4(0, 0, 0, 0);
    if (i < tail)
        tail_base[i] = 0;
}

int pack_args(int nd, const int64_t* dstr, const int64_t* dsta, const int64_t* dste,
              const int64_t* sstr, const int64_t* ssta, const int64_t* sste, const int64_t* counts,
              RegionArgs& a) {
    int pad = CNH_MAX_ND - nd;
    for (int d = 0; d < CNH_MAX_ND; ++d) {
        a.dstride[d] = a.sstride[d] = 0;
        a.dstart[d] = a.sstart[d] = 0;
        a.dstep[d] = a.sstep[d] = 1;
        a.counts[d] = 1;
    }
    for (int d = 0; d < nd; ++d) {
        a.dstride[pad + d] = dstr[d];
        a.dstart[pad + d] = dsta[d];
        a.dstep[pad + d] = dste[d];
        if (sstr) {
            a.sstride[pad + d] = sstr[d];
            a.sstart[pad + d] = ssta[d];
            a.sstep[pad + d] = sste[d];
        }
        a.counts[pad + d] = counts[d];
    }
    a.nchunks = (a.counts[2] + kBlock * kPerThread - 1) / (kBlock * kPerThread);
    return 0;
}

} // namespace

extern "C" {

int cnh_memset0(void* dptr, size_t bytes, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    if (bytes == 0)
        return 0;
    CNH_CHECK(((uintptr_t)dptr & 15) == 0, -2, "cnh_memset0: pointer must be 16-byte aligned");
    size_t n16 = bytes / 16, tail = bytes % 16;
    size_t want = (n16 + 255) / 256;
    unsigned blocks = (unsigned)(want < 1 ? 1 : (want > 16384 ? 16384 : want));
    hipLaunchKernelGGL(zero_kernel, dim3(blocks), dim3(256), 0, as_stream(s), (uint4*)dptr, n16,
                       (unsigned char*)dptr + n16 * 16, tail);
    CNH_HIP(hipGetLastError());
    return 0;
}

int cnh_fill_region(int nd, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const int64_t* counts,
                    const void* scalar8, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(nd >= 1 && nd <= CNH_MAX_ND, -2, "cnh_fill_region: ndims %d not in 1..3", nd);
    CNH_CHECK(esz == 4 || esz == 8, -2, "cnh_fill_region: element size %d not in {4,8}", esz);
    CNH_CHECK(dst && scalar8, -2, "cnh_fill_region: null pointer");
    for (int d = 0; d < nd; ++d) {
        CNH_CHECK(dst_step[d] >= 1, -2, "cnh_fill_region: step must be >= 1");
        if (counts[d] <= 0)
            return 0;
    }
    RegionArgs a;
    pack_args(nd, dst_strides, dst_start, dst_step, nullptr, nullptr, nullptr, counts, a);
    int64_t blocks = a.counts[0] * a.counts[1] * a.nchunks;
    CNH_CHECK(blocks < (1ll << 31), -3, "cnh_fill_region: region too large for one launch");
    if (esz == 8) {
        uint64_t v;
        std::memcpy(&v, scalar8, 8);
        hipLaunchKernelGGL((region_kernel<uint64_t, true>), dim3((unsigned)blocks), dim3(kBlock), 0,
                           as_stream(s), (uint64_t*)dst, (const uint64_t*)nullptr, v, a);
    } else {
        uint32_t v;
        std::memcpy(&v, scalar8, 4);
        hipLaunchKernelGGL((region_kernel<uint32_t, true>), dim3((unsigned)blocks), dim3(kBlock), 0,
                           as_stream(s), (uint32_t*)dst, (const uint32_t*)nullptr, v, a);
    }
    CNH_HIP(hipGetLastError());
    return 0;
}

int cnh_copy_region(int nd, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const void* src,
                    const int64_t* src_strides, const int64_t* src_start, const int64_t* src_step,
                    const int64_t* counts, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(nd >= 1 && nd <= CNH_MAX_ND, -2, "cnh_copy_region: ndims %d not in 1..3", nd);
    CNH_CHECK(esz == 4 || esz == 8, -2, "cnh_copy_region: element size %d not in {4,8}", esz);
    CNH_CHECK(dst && src, -2, "cnh_copy_region: null pointer");
    for (int d = 0; d < nd; ++d) {
        CNH_CHECK(dst_step[d] >= 1 && src_step[d] >= 0, -2,
                  "cnh_copy_region: destination steps must be >= 1, source steps >= 0");
        if (counts[d] <= 0)
            return 0;
    }
    RegionArgs a;
    pack_args(nd, dst_strides, dst_start, dst_step, src_strides, src_start, src_step, counts, a);
    int64_t blocks = a.counts[0] * a.counts[1] * a.nchunks;
    CNH_CHECK(blocks < (1ll << 31), -3, "cnh_copy_region: region too large for one launch");
    if (esz == 8)
        hipLaunchKernelGGL((region_kernel<uint64_t, false>), dim3((unsigned)blocks), dim3(kBlock),
                           0, as_stream(s), (uint64_t*)dst, (const uint64_t*)src, (uint64_t)0, a);
    else
        hipLaunchKernelGGL((region_kernel<uint32_t, false>), dim3((unsigned)blocks), dim3(kBlock),
                           0, as_stream(s), (uint32_t*)dst, (const uint32_t*)src, (uint32_t)0, a);
    CNH_HIP(hipGetLastError());
    return 0;
}

int cnh_convert_region(int nd, int dst_dtype, void* dst, const int64_t* dst_strides,
                       const int64_t* dst_start, const int64_t* dst_step, int src_dtype, const void* src,
                       const int64_t* src_strides, const int64_t* src_start, const int64_t* src_step,
                       const int64_t* counts, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(nd >= 1 && nd <= CNH_MAX_ND, -2, "cnh_convert_region: ndims %d not in 1..3", nd);
    CNH_CHECK(dst && src, -2, "cnh_convert_region: null pointer");
    CNH_CHECK(dtype_size(dst_dtype) && dtype_size(src_dtype), -2, "cnh_convert_region: unknown dtype %d -> %d",
              src_dtype, dst_dtype);
    for (int d = 0; d < nd; ++d) {
        CNH_CHECK(dst_step[d] >= 1 && src_step[d] >= 0, -2,
                  "cnh_convert_region: destination steps must be >= 1, source steps >= 0");
        if (counts[d] <= 0)
            return 0;
    }
    RegionArgs a;
    pack_args(nd, dst_strides, dst_start, dst_step, src_strides, src_start, src_step, counts, a);
    int64_t blocks = a.counts[0] * a.counts[1] * a.nchunks;
    CNH_CHECK(blocks < (1ll << 31), -3, "cnh_convert_region: region too large for one launch");
    hipStream_t st = as_stream(s);
    switch (src_dtype) {
    case CNH_F32: return launch_convert<float>(dst_dtype, dst, src, a, (unsigned)blocks, st);
    case CNH_F64: return launch_convert<double>(dst_dtype, dst, src, a, (unsigned)blocks, st);
    case CNH_I32: return launch_convert<int32_t>(dst_dtype, dst, src, a, (unsigned)blocks, st);
    default: return launch_convert<int64_t>(dst_dtype, dst, src, a, (unsigned)blocks, st);
    }
}

} // extern "C"
