/*
 * cnbench.h — benchmark fixtures exported by libcnhip. Not part of the drop-in boundary: nothing
 * here stands in for an upstream function, and an integration of the library does not call them.
 * They exist so that the benchmark and the full-size tests can build their inputs on the device
 * and set a measured ceiling beside the matmatmul figure.
 */
#ifndef CNBENCH_H
#define CNBENCH_H

#include "cnexec.h"
#include "cnhip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Block [row0, row0+nrows) x [col0, col0+ncols) of the dense conjugate-gradient test matrix of
 * order n, written row-major with row stride ld: A[i][j] = (u01(seed, 0, i*n+j) + u01(seed, 0,
 * j*n+i)) / (2n) off the diagonal, 2.0 on it (symmetric, diagonally dominant). */
int cnh_fill_cg_matrix(double* out, int64_t n, int64_t row0, int64_t nrows, int64_t col0,
                       int64_t ncols, int64_t ld, uint64_t seed, cnh_stream s);
/* The same matrix into the square fp64 array `name` of a host executor, tile by tile. */
int cnx_fill_cg_matrix(cnx_executor* ex, int name, uint64_t seed);
/* The rate at which this device issues the fp64 matrix instruction (v_mfma_f64_16x16x4) from
 * registers, 8 wavefronts per CU with four accumulators each, `iters` rounds. Synchronous. */
int cnh_probe_mfma_f64(int iters, double* tflops);

#ifdef __cplusplus
}
#endif
#endif
