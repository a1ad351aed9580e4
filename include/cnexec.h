/*
 * cnexec.h — the host executor of libcnhip: plays upstream's ArrayDAGGroup + PartitionImpl for all
 * partitions of every array on one device, without Charm++.
 *
 * The entry points mirror the entry methods of src/backend.ci:10-18 (what the CCS handlers of the
 * server call): a serialized DAG comes in through cnx_receive_dag, array contents leave through
 * cnx_get. Everything between (shape pass, tile rule, array creation, kernel compilation and cache,
 * per-node routing) happens inside, on top of the cnh_* calls of cnhip.h.
 *
 * Conventions as in cnhip.h: 0 on success, < 0 on error with cnh_last_error(); one thread per
 * executor at a time.
 *
 * ---- DAG message (little endian) ----
 * The upstream byte format is defined by charmtyles (DAG::deserialize, called from
 * src/dag_group_receive.cpp:191-192) and is not part of the charmnumeric tree; this format carries
 * the same information: the fields of DAGNode/ASTNode the backend reads
 * (src/dag_group_compile.cpp:45-51, src/jit.cpp:223-385, src/execute_node_regions.cpp:56-107) and
 * regions in upstream's own region encoding (charmnumeric.py:194-207).
 *
 *   message  := int32 magic (CNX_DAG_MAGIC), int32 version (1), int32 n_dag_nodes, dag_node*
 *   dag_node := int32 id, int32 fusible, int32 n_ast_nodes, int32 n_roots, ast_node*, int32 roots[n_roots]
 *   ast_node := int32 result_name, int32 opcode, int32 is_temp, int32 is_scalar, int32 is_broadcast,
 *               int32 ndims, int32 dtype, int32 n_operands (<= 2), int32 operands[n_operands],
 *               float64 scalar, region operand_regions[n_operands], region node_region
 *   region   := int32 is_global, then if not global: int32 ndims, (int32 start, stop, step)[ndims]
 *
 * DAG nodes are listed in execution (program) order. operands[] index the ast_node list of the same
 * DAG node. Opcodes are upstream's (src/opcodes.hpp:3-20) plus the extension opcodes below.
 * Leaves are NOOP nodes naming an existing array (is_broadcast = 1 for a size-1 array used as a
 * scalar), or is_scalar nodes carrying a literal.
 *
 * Root kinds and what they do:
 *   CREATE      node_region = [0:shape) of a new zero-filled array `result_name`
 *               (src/dag_group_receive.cpp:227-250, src/partition_lifecycle.cpp:43-88)
 *   elementwise group of ADD/SUB/MUL/DIV/TANH/EXP temporaries ending in one non-temp root, or in a
 *               SET_REGION root (operands: target leaf, value) — src/execute_node.cpp:1195-1585
 *   SET_REGION  with a scalar value: fill (src/executor_ast_visitor.cpp:112-147)
 *   REDUCE      dot of two 1-D arrays -> size-1 array (src/executor_reduce.cpp:8-119)
 *   MATMUL      2-D array times 1-D array -> 1-D array (src/executor_matmul.cpp:150-498)
 *   MATMATMUL   2-D times 2-D -> 2-D (src/executor_matmatmul.cpp:105-484)
 *   CNX_OP_DELETE  drop array `result_name`; its buffer goes to the free list
 *               (src/backend.hpp:366-545)
 */
#ifndef CNEXEC_H
#define CNEXEC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CNX_DAG_MAGIC 0x47444e43 /* "CNDG" */

/* Extension opcodes (no upstream counterpart; upstream has no N-D reduction, no random numbers and
 * no bulk upload: src/executor_reduce.cpp:9-12, charmnumeric/random.py:4-5, charmnumeric.py:863-878).
 * Operand layout: SUM(a); SUMSQ_DIFF(a, b); MAXABS_DIFF(a, b) -> size-1 fp64 array `result_name`,
 * over whole arrays of any rank; DELETE names the array in result_name; ASTYPE(a) -> a new array
 * `result_name` of a's shape holding a's values converted to the node's dtype (C conversion rules;
 * upstream's astype raises, charmnumeric/charmnumeric.py:738-744, and its mixed-dtype operations
 * only label the result, :369-373). */
enum {
    CNX_OP_DELETE = 100,
    CNX_OP_SUM = 101,
    CNX_OP_SUMSQ_DIFF = 102,
    CNX_OP_MAXABS_DIFF = 103,
    CNX_OP_ASTYPE = 104
};

typedef struct cnx_executor cnx_executor;

/* Start-up: what `charmrun +p<num_pes> server` plus the client's connect(ip, port, odf) fix
 * (charmnumeric/interface.py:70-92): odf * num_pes caps the number of tiles per array
 * (src/decomposition_solver.hpp:107-111). device is passed to cnh_init. */
int cnx_create(int device, int num_pes, int odf, cnx_executor** out);
int cnx_destroy(cnx_executor* ex);
/* Overrides CT_MIN_TILE_1D/2D/3D (src/backend.hpp:10-18; the upstream tests build with 64). */
int cnx_set_min_tile(cnx_executor* ex, int ndims, int min_tile);

/* Decomposition planning, off by default. Off: every array gets the tile rule and offset 0 (on
 * one device kernels read neighbouring tiles in place, so lining tiles up saves no traffic).
 * On: each DAG message is planned as a whole before it runs, as upstream does
 * (src/dag_group_receive.cpp:222-399 -> cnx_solve_decompositions below), and the arrays it
 * produces are laid out with the planned tile edge and offset; values do not depend on it.
 * Statements over arrays whose tiles line up run per tile; all others go through the general
 * gather; a product or paired reduction whose operand's tile grid does not start at element 0
 * works on a copy that does. */
int cnx_set_solver(cnx_executor* ex, int on);
/* Storage of rank-3 arrays created from now on. flat_rank3 != 0 (default): one row-major block
 * over the whole array, its partitions (src/backend.hpp:112-200 keeps one buffer per chare) being
 * views into it with the array's row and plane pitches; stencil sweeps then run on the block as a
 * whole. 0: one contiguous buffer per partition, as for the other ranks. Values never depend on it. */
int cnx_set_layout(cnx_executor* ex, int flat_rank3);
/* Launch fusion across the nodes of a DAG message, on by default. (1) A run of assignments
 * `target[box] = f(operand boxes)` of one extent (at most 2^22 elements each), every box one
 * strided block of device memory, goes out as ONE group with an output root per statement through
 * the memref launch (cnh_launch_group); a statement that reads the very box an earlier one of the
 * run assigned takes it from registers, and boxes of one array that are neither identical nor
 * disjoint end the run, so results are those of the statements run one by one. (2) MATMATMUL into a
 * temporary followed by `target[box] = temporary` and the temporary's deletion writes the fp64
 * product straight into the box. (3) Statements that make new arrays of one shape from whole arrays
 * laid out alike, the statements on one-element arrays between them (alpha = rr / pAp) and the
 * reductions of the new arrays go out as one group: scalar statements are formed in registers and
 * stored once (CNH_OP_SCALAR_OF), reductions leave partial sums that the next launch to read them
 * as a kernel scalar adds up itself (cnh_launch_group_sums) — anything else that needs the value
 * gets a fold first (cnh_fold_sums). (4) `beta = a / b; p = xa + beta * xb; y = A @ p; d = p @ y` on a
 * matrix of 16384 rows or more is one launch of cnh_gemv_tiles_fused. (5) Two SET_REGION statements
 * on lattices of step 2 of one array that neither read what the other assigns (the two halves of a
 * red-black colour) are one sweep in place; arrays cut into tiles are stored as one block first.
 * Off: every node is executed on its own, as upstream does.
 * Stored results of element-wise statements are the same bits either way. Reductions, and values
 * computed from them, agree to the order of summation: fused and unfused forms add different partial
 * sums, and (for a statement held back at the end of a message) which form runs can depend on where
 * the caller's flushes fall. fp64 products: see "gemm_ksplit" in cnhip.h for the one other place
 * where the order of additions depends on the launch's shape. */
int cnx_set_fusion(cnx_executor* ex, int on);

/* ArrayDAGGroup::receive_dag(int epoch, int size, char msg[size]) (src/backend.ci:15,
 * src/dag_group_receive.cpp:190-575) followed by the partitions' run(): executes every node of the
 * DAG in order. Returns when all work is queued on the executor's stream (not when it finished). */
int cnx_receive_dag(cnx_executor* ex, int epoch, int64_t size, const char* msg);
/* Asynchronous mode (off by default). When on, cnx_receive_dag copies the message, queues it for a
 * thread that belongs to the executor and returns; the messages run in the order received, as
 * upstream's frontend hands messages to its server and goes on recording
 * (charmnumeric/interface.py upstream). Every other call on the executor first waits for the
 * queue. A queued message that fails makes the executor drop what is queued behind it, and its
 * error code and text are returned by the next call on the executor, whichever it is. */
int cnx_set_async(cnx_executor* ex, int on);

/* The statement log: the frontend's recording, shipped raw. Upstream's frontend groups what it
 * recorded into DAG nodes itself (charmtyles, outside the charmnumeric tree) and sends the result to
 * receive_dag; with this entry point the grouping (which element-wise operations fuse, which
 * results never become arrays, which deletions have nothing to delete) runs inside the executor, on
 * its own thread in asynchronous mode, and the nodes it makes run exactly as if they had arrived
 * through cnx_receive_dag. Records (little endian, int32 words unless noted):
 *   delete      := 5, name
 *   create      := head, shape                                   kind 1
 *   op          := head, shape, operand * n_operands             kind 2, element-wise, <= 2 operands
 *   set         := head, shape, region, operand                  kind 3, target[region] = operand
 *   nonfusible  := head, shape, operand * n_operands             kind 4: reductions, products, ...
 *   head        := kind, name, opcode, dtype, n_operands, aux    aux: rank of the target (set), else 0
 *   shape       := ndims, extent[3]                              of the result / the assigned region
 *   region      := ndims, start[3], stop[3], step[3]
 *   operand     := 0, 0, float64 value
 *                | 1, name, base_ndims, dtype, broadcast, has_region, start[3], stop[3], step[3]
 * hold_back_window < 0: everything recorded so far is planned and run. >= 0 (an automatic flush in
 * the middle of a program): statements from the one that produced a still-live result within the
 * last `window` records onwards stay unplanned in the executor, so that a result whose handle is
 * about to go away is not turned into an array just because the flush fell there. They are planned
 * with the next cnx_receive_log, and to their end by whatever needs the arrays' state first:
 * cnx_get, cnx_put, cnx_fill_*, cnx_sync, cnx_array_info and cnx_receive_dag (a DAG message runs
 * behind every statement logged before it). */
int cnx_receive_log(cnx_executor* ex, int64_t size, const char* log, int hold_back_window);
/* Forgets the part of the log an automatic flush held back (the frontend's reset()). */
int cnx_discard_log(cnx_executor* ex);
/* Test hook: with capture on, every DAG message planned from the log is also kept as bytes, each
 * preceded by its int64 length; cnx_captured copies them out as cnx_trace does and clears them. */
int cnx_set_capture(cnx_executor* ex, int on);
int64_t cnx_captured(cnx_executor* ex, char* buf, size_t cap);

/* receive_get_request(int ndims, int epoch, int name, int size, int dtype) + gather + reply
 * (src/backend.ci:16-17, src/partition_get.cpp:4-67, src/dag_group_runtime.cpp:55-118): copies
 * array `name` into host_out as one global row-major array of `size` elements. Blocks. */
int cnx_get(cnx_executor* ex, int ndims, int epoch, int name, int64_t size, int dtype, void* host_out);

/* Extensions without upstream counterpart. */
/* Bulk upload of a whole row-major host array into existing array `name`. Blocks. */
int cnx_put(cnx_executor* ex, int name, int64_t size, int dtype, const void* host_in);
/* array[i] = lo + (hi-lo)*u01(seed, stream_id, i), i = global row-major index; fp64 arrays. */
int cnx_fill_uniform(cnx_executor* ex, int name, uint64_t seed, uint64_t stream_id, double lo, double hi);
/* Waits for everything queued so far. */
int cnx_sync(cnx_executor* ex);

/* Introspection (tests, logs). */
/* ndims, dtype, tile edge, shape[3], offset[3] of array `name`; < 0 if unknown. */
int cnx_array_info(cnx_executor* ex, int name, int* ndims, int* dtype, int* tile, int32_t* shape3,
                   int32_t* offset3);
/* Measurement (no upstream counterpart). With timing on, every matvec launch of the executor is
 * bracketed by a pair of events on its stream; cnx_matvec_times waits for the stream, writes the
 * elapsed milliseconds of the launches timed so far (oldest first, at most `cap`) to `ms`, forgets
 * them and returns how many it wrote. Switching timing on or off also forgets them. */
int cnx_set_matvec_timing(cnx_executor* ex, int on);
int64_t cnx_matvec_times(cnx_executor* ex, float* ms, int64_t cap);
/* Counters since creation: [0] kernels compiled (upstream num_compile, src/backend.hpp:241),
 * [1] compile-cache hits, [2] DAG nodes executed, [3] device allocations, [4] free-list reuses,
 * [5] fused-group launches, [6] live arrays, [7] bytes held (live + free list). */
int cnx_stats(cnx_executor* ex, int64_t out[8]);
/* Decision log: one text line per array creation, launch choice (dense / tiles, ping-pong or in
 * place), reduction, product. cnx_trace copies the NUL-terminated log into buf when it fits, clears
 * it, and returns the size needed. With device < 0 in cnx_create the executor takes every decision
 * and logs it but allocates and launches nothing (host-logic tests on machines without a GPU). */
int cnx_set_trace(cnx_executor* ex, int on);
int64_t cnx_trace(cnx_executor* ex, char* buf, size_t cap);

/* ArrayDAGGroup::compute_decompositions (src/dag_group_runtime.cpp:42-44 over
 * src/decomposition_solver.hpp:94-1714): tile edge and offset of every array a DAG message
 * produces. arrays[] is ArrayMetadata (src/backend.hpp:264-288) for the arrays the message names:
 * existing ones with final = 1 (their tile and offset are kept), results with final = 0 and their
 * shape filled in (tile 0 = the rank's minimum). On return every entry carries its tile and
 * absolute offset and final = 1. min_tile = CT_MIN_TILE_1D/2D/3D. msg is a DAG message as above
 * (size 0: tile rule only); a leaf may name a temporary root of the same DAG node
 * (is_temp = 1), which stands for that root's expression. Pure host code: no device is touched.
 * Upstream iterates hash maps; where its answer depends on their order (which of several
 * already-placed arrays a component is rooted at) this function takes ascending array names. */
typedef struct cnx_decomp {
    int32_t name;
    int32_t ndims;
    int32_t shape[3];
    int32_t offset[3];
    int32_t tile;
    int32_t final;
} cnx_decomp;
int cnx_solve_decompositions(int odf, int num_pes, const int32_t min_tile[3], int n_arrays,
                             cnx_decomp* arrays, int64_t size, const char* msg);

#ifdef __cplusplus
}
#endif
#endif
