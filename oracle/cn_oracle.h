/*
 * cn_oracle.h — CPU restatement of charmnumeric's per-partition array execution path.
 *
 * THIS IS TEST INFRASTRUCTURE. It exists to check the HIP path and to time a CPU baseline.
 * Nothing in the product (the charmnumeric_amd package, libcnhip) may include, link or call it.
 *
 * Every function cites the reference file:line (under the upstream charmnumeric tree) whose
 * behaviour it restates. Plain data only crosses this interface (C ABI, no C++ types).
 *
 * Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):
 *   region algebra ............ reference-held vectors (tests/test_jit.cpp:244-326, comments in
 *                               src/array_region.hpp:481-485,840-843) + brute-force lattice sets
 *   tile rule ................. reference-held vectors (tests/test_compute_decompositions.cpp)
 *   fused group evaluation .... NumPy in the same operand order (IEEE-754 closed form),
 *                               reference tests (tests/test_backend_integration.py) known answers
 *   exp/tanh .................. host libm (the symbols the reference JIT resolves)
 *   fill/copy region .......... NumPy slicing assignment, bit-exact
 *   dot/gemv/gemm ............. closed forms from the reference examples + math.fsum / long double;
 *                               the summation ORDER inside Eigen is "parity unpinned" (only 1e-12 bar)
 *   integer division by zero and INT_MIN / -1: undefined in the reference (arith.divsi);
 *                               defined here as 0 and wrap — "parity unpinned" for those two inputs
 */
#ifndef CN_ORACLE_H
#define CN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_MAX_ND 3

/* Opcode numbering: src/opcodes.hpp:3-20 (mirrors charmnumeric/charmnumeric.py:139-150). */
enum {
    ORC_OP_COPY = -5, ORC_OP_SET_REGION = -4, ORC_OP_GET_REGION = -3, ORC_OP_CREATE = -2,
    ORC_OP_NOOP = -1, ORC_OP_ADD = 0, ORC_OP_SUB = 1, ORC_OP_MUL = 2, ORC_OP_DIV = 3,
    ORC_OP_MATMUL = 4, ORC_OP_TANH = 5, ORC_OP_EXP = 6, ORC_OP_TILE = 7, ORC_OP_REDUCE = 8,
    ORC_OP_MATMATMUL = 9, ORC_OP_DIAG = 10
};
/* DType wire values: charmnumeric/charmnumeric.py:34-40. */
enum { ORC_F32 = 0, ORC_F64 = 1, ORC_I32 = 2, ORC_I64 = 3 };

/* ArrayRegion<N> (src/array_region.hpp:21-33) with N carried at run time (N <= 3). */
typedef struct orc_region {
    int32_t is_global;
    int32_t ndims;
    int32_t start[ORC_MAX_ND];
    int32_t stop[ORC_MAX_ND];
    int32_t step[ORC_MAX_ND];
} orc_region;

/* ArrayDecomp<N> (src/array_region.hpp:293-387). */
typedef struct orc_decomp {
    int32_t ndims;
    int32_t offset[ORC_MAX_ND];
    int32_t global_shape[ORC_MAX_ND];
    int32_t tile;
} orc_decomp;

/* The ASTNode field set as the backend consumes it (tests/test_jit.cpp:35-46,
 * src/jit.cpp:223-263, src/execute_node_regions.cpp:56-107). Operands are indices into the
 * flat node array; leaves are NOOP/CREATE nodes. */
typedef struct orc_ast_node {
    int32_t result_name;
    int32_t opcode;
    int32_t is_temp;
    int32_t is_scalar;
    int32_t is_broadcast;
    int32_t ndims;
    int32_t dtype;
    int32_t n_operands;
    int32_t operands[2];
    int32_t has_operand_region[2];
    double scalar;
    orc_region operand_regions[2];
    orc_region region;
} orc_ast_node;

/* AST{roots[]}: flat list, temporaries first (src/jit.cpp:120-122). */
typedef struct orc_ast {
    int32_t n_nodes;
    int32_t n_roots;
    const orc_ast_node* nodes;
    const int32_t* roots;
} orc_ast;

/* MemRef<N,T> (src/array_region.hpp:404-415): sizes/strides/offset in ELEMENTS. */
typedef struct orc_memref {
    void* allocated;
    void* aligned;
    int64_t offset;
    int64_t sizes[ORC_MAX_ND];
    int64_t strides[ORC_MAX_ND];
} orc_memref;

/* ---- region algebra (src/array_region.hpp) ---- */
int orc_first_aligned_point(int start_a, int step_a, int start_b, int step_b, int lo, int hi,
                            int* aligned, int* aligned_step);              /* :75-108 */
int orc_region_size_dim(const orc_region* r, int d);                       /* :111 */
int orc_region_size(const orc_region* r);                                  /* :114-119 */
int orc_region_overlaps(const orc_region* a, const orc_region* b);         /* :137-158 */
int orc_region_covers(const orc_region* a, const orc_region* b);           /* :160-187 */
int orc_region_intersect(const orc_region* a, const orc_region* b, orc_region* out); /* :189-225 */
int orc_region_subtract(const orc_region* r1, const orc_region* r2, orc_region* out /*cap 2N+1*/); /* :471-519 */
void orc_region_map(const orc_region* r1, const orc_region* parent1, const orc_region* parent2,
                    orc_region* out);                                      /* :524-545 */
int orc_decomp_num_chares(const orc_decomp* d, int dim);                   /* :350-354 */
void orc_decomp_chare_region_global(const orc_decomp* d, const int32_t* ci, orc_region* out); /* :360-368 */
/* decompose (:822-866): returns count; chare indices (count*ndims ints) and sub-regions are
 * emitted in lexicographic chare-index order (the reference's unordered_map has no order). */
int orc_decompose(const orc_region* region, const orc_decomp* decomp, int cap, int32_t* chare_idx,
                  orc_region* out);
/* local_inputs (:553-604): my_inputs[n_inputs] (full mapped input regions) + expected_msgs. */
int orc_local_inputs(const orc_region* r_out, int n_inputs, const orc_region* inputs,
                     const int32_t* nd_idx, const orc_decomp* out_decomp,
                     const orc_decomp* in_decomps, orc_region* my_inputs, int* expected_msgs);
/* send_remote_inputs (:625-663): emits (target chare idx[ndims], region, input_index). */
int orc_send_remote_inputs(const orc_region* r_out, int n_inputs, const orc_region* inputs,
                           const int32_t* nd_idx, const orc_decomp* out_decomp,
                           const orc_decomp* in_decomps, int cap, int32_t* targets,
                           orc_region* regions, int32_t* input_index);
/* align_fragments (:675-818). Fragments of input k are frags[frag_begin[k] .. frag_begin[k+1]).
 * data offsets are expressed in elements relative to each fragment's own base, so no pointers
 * cross the interface: out_offsets[k*M+m] is the element offset into fragment out_frag[k*M+m].
 * Returns M (cells per input) or <0 on error. */
typedef struct orc_fragment {
    orc_region region;
    int64_t src_strides[ORC_MAX_ND]; /* all 0 = packed */
} orc_fragment;
int orc_align_fragments(int ndims, int K, const int32_t* frag_begin, const orc_fragment* frags,
                        const orc_region* parents, int cap, int32_t* out_frag, int64_t* out_offsets,
                        int64_t* out_sizes /*M*K*3*/, int64_t* out_strides /*M*K*3*/,
                        orc_region* out_cells /*M*K*/);

/* ---- tile rule (src/decomposition_solver.hpp:100-122, src/backend_internal.hpp:137-160) ---- */
int orc_next_pow2(int v);
int orc_tile_rule(int ndims, const int32_t* shape, int odf, int num_pes, int min_tile);

/* ---- fused group: numerical definition per src/jit.cpp:28-150,223-459 ---- */
/* Argument layout the compiled kernel expects (src/jit.cpp:78-87): one memref per leaf USE,
 * one scalar per unique broadcast leaf, one memref per non-temp root. */
int orc_group_signature(const orc_ast* ast, int cap, int32_t* leaf_node /*node index per leaf use*/,
                        int32_t* leaf_root, int32_t* leaf_operand, int* n_leaves,
                        int32_t* bcast_node, int* n_bcast, int32_t* out_root, int* n_out);
/* Element dtype of a group: first root dtype != F32, else F32 (src/jit.cpp:50-69). */
int orc_group_dtype(const orc_ast* ast);
/* Evaluate the group elementwise, roots in AST order, no FMA contraction, no re-association.
 * scalars[i] points at ONE element of the group dtype. Returns 0, or <0 for an AST the
 * reference JIT cannot compile (tanh/exp on ints, unary op on a scalar, unknown opcode). */
int orc_eval_group(const orc_ast* ast, int dtype, int ndims, int n_in, const orc_memref* in,
                   int n_scalar, const void* const* scalars, int n_out, const orc_memref* out);

/* One fused SET_REGION group over one tiled array (offset 0, `tile` edge, tiles in row-major grid
 * order, each row-major over its own extent), executed chare by chare as the reference's fragment
 * path does: halo pack + message per remote fragment, local + received fragments per operand,
 * align_fragments, one kernel per aligned cell into a packed result buffer, SET_REGION copy
 * (src/executor_core.cpp:8-143,684-747, src/execute_node.cpp:1376-1585,
 * src/executor_ast_visitor.cpp:268-311). Every leaf must be the assigned array. `threads` chares
 * run side by side in the compute phase. stats: [0] messages, [1] bytes packed, [2] kernel calls,
 * [3] largest cell count of a chare. */
int orc_world_group(const orc_ast* ast, int dtype, int ndims, const int32_t* shape, int tile,
                    void* const* tiles, int threads, int64_t* stats);

/* ---- SET_REGION fill / strided copy (src/executor_ast_visitor.cpp:112-313) ---- */
/* Element i along dim d sits at (start[d] + i*step[d]) * strides[d]; byte-wise, bit-exact. */
int orc_fill_region(int ndims, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const int64_t* counts,
                    const void* scalar);
int orc_copy_region(int ndims, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const void* src,
                    const int64_t* src_strides, const int64_t* src_start, const int64_t* src_step,
                    const int64_t* counts);
/* Scalar conversion to the target dtype: (T)double (src/executor_ast_visitor.cpp:112-147). */
int orc_scalar_to_dtype(int dtype, double s, void* out8);

/* ---- reductions / matvec / matmatmul ---- */
/* eigen_dot (src/backend_internal.hpp:88-93): restated as a left-to-right sum. */
int orc_dot(int dtype, int64_t n, const void* a, const void* b, void* out);
/* reduce_dot_sum (src/executor_reducer.cpp:11-57): sequential a += b over the contributions. */
int orc_reduce_partials(int dtype, int n, const void* partials, void* out);
/* eigen_gemv_sub (src/backend_internal.hpp:28-41): res[i] = sum_j mat[(row_off+i)*full_cols+col_off+j]*vec[j]. */
int orc_gemv_sub(int dtype, const void* mat, int64_t full_local_cols, int64_t row_off,
                 int64_t col_off, int64_t sub_rows, int64_t sub_cols, const void* vec, void* res);
/* 1-D partial accumulate, res += partial (src/execute_node.cpp:563-577). */
int orc_axpy1(int dtype, int64_t n, const void* partial, void* res);
/* C += A*B, row-major with row strides (src/executor_incremental.cpp:120-132). */
int orc_gemm_acc(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                 const void* B, int64_t ldb, void* C, int64_t ldc);
/* Same contraction split over `threads` row blocks (one std::thread per emulated PE). */
int orc_gemm_acc_mt(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                    const void* B, int64_t ldb, void* C, int64_t ldc, int threads);
int orc_gemv_sub_mt(int dtype, const void* mat, int64_t full_local_cols, int64_t row_off,
                    int64_t col_off, int64_t sub_rows, int64_t sub_cols, const void* vec,
                    void* res, int threads);

/* Extensions the workloads need that the reference lacks (no counterpart; closed-form pinned). */
int orc_sum(int dtype, int64_t n, const void* a, void* out);
int orc_sumsq_diff(int64_t n, const double* a, const double* b, double* out);  /* sum (a-b)^2 */
int orc_maxabs_diff(int64_t n, const double* a, const double* b, double* out); /* max |a-b| */

/* ---- synthetic input generator (counter-based SplitMix64) ---- */
uint64_t orc_splitmix(uint64_t seed, uint64_t stream, uint64_t i);
double orc_u01(uint64_t seed, uint64_t stream, uint64_t i);
/* out[k] = lo + (hi-lo)*u01(seed, stream, first+k), one mul + one add, no FMA. */
void orc_fill_uniform(double* out, int64_t n, uint64_t seed, uint64_t stream, uint64_t first,
                      double lo, double hi);
/* Rows [row0,row0+nrows) x cols [col0,col0+ncols) of the dense CG matrix of order n:
 * A[i][j] = (u01(seed,0,i*n+j) + u01(seed,0,j*n+i)) / (2n) for i != j, A[i][i] = 2.0;
 * written row-major with row stride ld. */
void orc_fill_cg_matrix(double* out, int64_t n, int64_t row0, int64_t nrows, int64_t col0,
                        int64_t ncols, int64_t ld, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif
