// Shared internals of libcnhip (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/cnhip.h"
#include "../../include/cnbench.h"

namespace cnh {

// Thread-local error text behind cnh_last_error().
int set_error(int code, const char* fmt, ...);
std::string& error_slot();

#define CNH_HIP(expr)                                                                            \
    do {                                                                                         \
        hipError_t _e = (expr);                                                                  \
        if (_e != hipSuccess)                                                                    \
            return cnh::set_error(-100, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),   \
                                  __FILE__, __LINE__);                                           \
    } while (0)

#define CNH_CHECK(cond, code, ...)                                                               \
    do {                                                                                         \
        if (!(cond))                                                                             \
            return cnh::set_error(code, __VA_ARGS__);                                            \
    } while (0)

inline int dtype_size(int dt) {
    switch (dt) {
    case CNH_F32:
    case CNH_I32: return 4;
    case CNH_F64:
    case CNH_I64: return 8;
    }
    return 0;
}

inline hipStream_t as_stream(cnh_stream s) { return reinterpret_cast<hipStream_t>(s); }

// Lazily selects the device on first use of any entry point.
int ensure_init();
// The device cnh_init selected, -1 before the first call.
int current_device();
// Resolves the address of the no-allocation dot's scratch array on `device` (which is current).
int reduce_scratch_init(int device);

// Device scratch for reduction partials, one region per stream handle so that calls on
// different streams never share slots. Returns a device pointer to `bytes` bytes.
int reduce_workspace(hipStream_t s, size_t bytes, void** out);

// Folds the per-wavefront partials a reducing stencil launch left behind (sum, or maximum of
// non-negative values) into *out, in index order, on the same stream.
// The buffer behind `slots` holds n + kFoldRuns doubles: the fold keeps its run sums behind them.
constexpr int64_t kFoldRuns = 1024;
constexpr int kFoldMaxVectors = 4;
int reduce_slots_f64_many(int nvec, const int* maximum, double* const* vecs, int64_t n, double* const* outs,
                          hipStream_t st);
void gemv_set_xlds(int on);
void gemm_set_buffer_loads(int on);
void gemm_set_ksplit(int on);
// Which form of the matrix-core kernel a single overwriting fp64 product of this shape takes with
// buffer loads (0: none of them — extents no multiples of the 64 x 64 x 16 tile, unaligned or too
// widely strided operands): 1 = two sets of eight wavefronts per workgroup sharing the K steps (at
// most one workgroup per CU, K a multiple of 32), 2 = eight wavefronts of 16 x 32, 3 = four of
// 32 x 32 (1024 tiles and more). The kernel with a group's statements in its epilogue is built in
// the same form, so it adds its sums in the same order.
int gemm_form(int64_t M, int64_t N, int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb);
int reduce_slots_f64(bool maximum, double* slots, int64_t n, double* out, hipStream_t st);

// Option "product_statements": may a product's launch evaluate the statements that follow it?
bool product_statements_on();

// Descriptor tables (per-partition pointers/shapes) live on the device. Identical tables are
// uploaded once and found again by content hash, so steady-state launches issue no copy.
int desc_upload(const void* host, size_t bytes, hipStream_t s, const void** dev_out);

} // namespace cnh
