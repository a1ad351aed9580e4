/*
 * cnhip.h — C ABI of libcnhip: the MI355X (gfx950) executor back end for charmnumeric's
 * per-partition array execution path.
 *
 * Each entry point replaces one seam of the upstream C++ backend; the comment on every
 * declaration names the upstream function (file:line in the charmnumeric tree) it stands in for.
 *
 * Conventions
 *   - return 0 on success, < 0 on error; cnh_last_error() returns the message of the last error
 *     raised on the calling thread. Nothing throws or aborts across this boundary.
 *   - the library never frees caller memory and never keeps a host pointer past return.
 *   - sizes, strides and offsets are in ELEMENTS (int64), as in the upstream MemRef descriptor.
 *   - dtype codes are the wire values F32=0, F64=1, I32=2, I64=3 (charmnumeric.py:34-40).
 *   - a cnh_stream of NULL is the device's default stream. Work on one stream is ordered.
 *   - one thread per handle at a time (the upstream scheduler runs entry methods to completion).
 */
#ifndef CNHIP_H
#define CNHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CNH_MAX_ND 3

/* Opcode numbering: src/opcodes.hpp:3-20. */
enum {
    CNH_OP_COPY = -5, CNH_OP_SET_REGION = -4, CNH_OP_GET_REGION = -3, CNH_OP_CREATE = -2,
    CNH_OP_NOOP = -1, CNH_OP_ADD = 0, CNH_OP_SUB = 1, CNH_OP_MUL = 2, CNH_OP_DIV = 3,
    CNH_OP_MATMUL = 4, CNH_OP_TANH = 5, CNH_OP_EXP = 6, CNH_OP_TILE = 7, CNH_OP_REDUCE = 8,
    CNH_OP_MATMATMUL = 9, CNH_OP_DIAG = 10,
    /* Extension, no upstream counterpart: a group root that reduces its operand over every
     * element of the launch instead of storing it (sum, or the largest absolute value). Upstream
     * runs a reduction as a pass of its own over the stored array (src/executor_reduce.cpp:8-119);
     * as a root of the group that produces the values it costs no second read. */
    CNH_OP_SUM_OF = 20, CNH_OP_MAXABS_OF = 21,
    /* Extension, no upstream counterpart: an output root whose operand is formed from the launch's
     * scalars alone (alpha = r.r / p.Ap next to the updates that use it). Upstream runs such a
     * statement as a group of its own over one-element arrays (src/jit.cpp:329-333,
     * src/executor_core.cpp:390-605); here the first lane of the launch stores the value once, at
     * element 0 of the output's memref. Dense launches only. */
    CNH_OP_SCALAR_OF = 22
};
enum { CNH_F32 = 0, CNH_F64 = 1, CNH_I32 = 2, CNH_I64 = 3 };

typedef void* cnh_stream;
typedef void* cnh_event;

/* ArrayRegion<N> (src/array_region.hpp:21-33); N <= 3 carried at run time. */
typedef struct cnh_region {
    int32_t is_global;
    int32_t ndims;
    int32_t start[CNH_MAX_ND];
    int32_t stop[CNH_MAX_ND];
    int32_t step[CNH_MAX_ND];
} cnh_region;

/* One AST node, with the fields the upstream backend reads from charmtyles' ASTNode
 * (src/jit.cpp:223-385, src/execute_node_regions.cpp:56-107, tests/test_jit.cpp:35-46).
 * operands[] index into the flat node array; leaves are NOOP/CREATE nodes. */
typedef struct cnh_ast_node {
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
    cnh_region operand_regions[2];
    cnh_region region;
} cnh_ast_node;

/* AST{roots[]}: flat, temporaries first (src/jit.cpp:120-122). */
typedef struct cnh_ast {
    int32_t n_nodes;
    int32_t n_roots;
    const cnh_ast_node* nodes;
    const int32_t* roots;
} cnh_ast;

/* MemRef<N,T> {allocated, aligned, offset, sizes[N], strides[N]} (src/array_region.hpp:404-415). */
typedef struct cnh_memref {
    void* allocated;
    void* aligned;
    int64_t offset;
    int64_t sizes[CNH_MAX_ND];
    int64_t strides[CNH_MAX_ND];
} cnh_memref;

/* ---- library state ---- */
int cnh_init(int device);               /* selects the device; idempotent */
const char* cnh_last_error(void);
int cnh_device_name(char* buf, size_t cap);
int cnh_version(void);
/* Tuning switches (defaults are what measured best on MI355X; 0 restores a default geometry).
 *   "stencil_mode"   kernel cnh_launch_group_tiles uses for same-array unit-step stencils:
 *                    2 (default) register window, 1 LDS sliding window, 0 general gather
 *   "direct_tx/ry/rz"  register window: lanes along x per workgroup row, rows and planes per lane
 *   "direct_lean"    wavefront-level lean kernel with lane exchange: 1 on, 0 off, -1 (default) on
 *   "direct_group"   workgroup order for rank 3: 0 (default) tile by tile, 1 groups of G^3 tiles,
 *                    2 rows of tiles along x
 *   "direct_stagger" concurrent groups start at different places of their tiles (default 0)
 *   "direct_merge"   lean part and the rest in one launch (default 1) or two
 *   "direct_flat"    arrays whose tiles are views into one row-major block take the whole-array
 *                    register-window kernel (default 1)
 *   "flat_nt_mib", "stencil_nt_mib"  a dense launch / a sweep whose arrays add up to this many MiB or
 *                    more streams past the caches with non-temporal accesses (default 272: what the
 *                    256 MiB last-level cache keeps from one launch of a loop to the next)
 *   "flat_tail"      that kernel gives one or two unassigned columns beyond a multiple of 128 (the
 *                    boundary of a 2^k + 1 grid) to the wavefront before them (default 1)
 *   "flat_obz/oby/obx"  extents in elements of the blocks that kernel's workgroups are ordered by
 *                    (default 256^3 for rank 3, bands of whole rows for rank 2)
 *   "tiles_rows"     general gather: rows shorter than 1024 elements share a workgroup (default 1)
 *   "tiles_block"    general gather: a launch whose arrays are one row-major block each (or single
 *                    tiles) addresses them without tile tables (default 1)
 *   "block_pairs"    ... and statements with unit steps along the rows move pairs of elements as one
 *                    access each (default 1). Same bits.
 *   "gemv_xlds"      matvecs of 8192 rows or more whose column tiles are at most 64 KB of x wide
 *                    stage x in LDS, 32 or 64 rows per workgroup (default 1); 0: one wavefront per
 *                    row reading x through the caches. Same bits either way.
 *   "gemm_buffer_loads"  aligned fp64 products fetch A and B with buffer loads (default 1). Same bits.
 *   "gemm_ksplit"        fp64 products on grids of at most one workgroup per CU, every K a multiple of
 *                        32: two sets of wavefronts per workgroup, each taking every other K step,
 *                        their sums added first + second (default 1). One fixed order, another than
 *                        with 0; whether a product qualifies depends on the device's CU count, so two
 *                        devices with different CU counts may differ in the last bits of a product
 *                        (0 gives the single-set order everywhere).
 *   "product_statements"  cnh_launch_product_group takes the shapes it can (default 1); 0: it answers
 *                        -17 for every shape, so callers issue the product and the group separately.
 *                        Same bits.
 *   "slide_bx/ry/zc/pd", "slide2d_march"  geometry of the sliding-window kernel */
int cnh_set_option(const char* name, int value);

/* ---- storage: Array<N,T> ctor zero-fill / data_ptr / copyToHost / copyToDevice / dtor
 *      (src/backend.hpp:112-200) ---- */
int cnh_alloc(size_t bytes, int zero, void** dptr);   /* zero: returns after the fill has landed */
/* The same with the zero-fill queued on `s`: ordered with what the caller queues there next, and the
 * host does not wait (an Array constructor on the scheduler thread of a PE should not block it;
 * work on other streams must order itself with `s` before it touches the block). */
int cnh_alloc_on(size_t bytes, int zero, cnh_stream s, void** dptr);
int cnh_free(void* dptr);
/* How many device or pinned-host allocations and descriptor-table copies the library has made so
 * far in this process: a caller that must not allocate (cnh_dot_partial_noalloc) can check that a
 * call left it unchanged. */
int64_t cnh_allocation_count(void);
int cnh_memset0(void* dptr, size_t bytes, cnh_stream s);
int cnh_h2d(void* dst_dev, const void* src_host, size_t bytes, cnh_stream s); /* returns after the copy */
int cnh_d2h(void* dst_host, const void* src_dev, size_t bytes, cnh_stream s); /* returns after the copy */
int cnh_d2d(void* dst_dev, const void* src_dev, size_t bytes, cnh_stream s);  /* asynchronous */
/* Strided device -> host gather of one tile into a global row-major host buffer; replaces the
 * one-message-per-innermost-row gather of src/partition_get.cpp:42-65 +
 * src/dag_group_runtime.cpp:99-118. counts/strides/starts in elements. */
int cnh_d2h_region(int ndims, int esz, void* dst_host, const int64_t* dst_strides,
                   const int64_t* dst_start, const void* src_dev, const int64_t* src_strides,
                   const int64_t* src_start, const int64_t* counts, cnh_stream s);

/* ---- completion: CT_KOKKOS_FENCE / hapiAddCallback (src/executor_core.cpp:618-627,761-774,
 *      src/dispatch.hpp:40-53) ---- */
int cnh_stream_create(cnh_stream* out);
int cnh_stream_destroy(cnh_stream s);
int cnh_stream_sync(cnh_stream s);
int cnh_stream_callback(cnh_stream s, void (*fn)(void*), void* arg);
int cnh_device_sync(void);
int cnh_event_create(cnh_event* out);
int cnh_event_destroy(cnh_event e);
int cnh_event_record(cnh_event e, cnh_stream s);
int cnh_event_sync(cnh_event e);
int cnh_event_elapsed_ms(cnh_event start, cnh_event stop, float* ms);

/* ---- SET_REGION scalar fill and strided copy; halo pack/unpack
 *      (src/executor_ast_visitor.cpp:112-313, src/executor_core.cpp:8-143,
 *       src/execute_node.cpp:1001-1181). Element i of dim d is at
 *      (start[d] + i*step[d]) * strides[d]. Byte-wise, bit-exact; esz in {4, 8}. A source step of
 *      0 repeats the source along that dimension (TILE of an extent-1 dimension). ---- */
int cnh_fill_region(int ndims, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const int64_t* counts,
                    const void* scalar8, cnh_stream s);
int cnh_copy_region(int ndims, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const void* src,
                    const int64_t* src_strides, const int64_t* src_start, const int64_t* src_step,
                    const int64_t* counts, cnh_stream s);
/* The strided copy with a change of element type, dst = (dst type)src with C's conversion rules
 * (to floating point: round to nearest even; to an integer type: truncation towards zero; a
 * floating-point value outside the integer type's range, or NaN, gives an unspecified integer).
 * What NumPy's astype computes. Upstream labels the result of an operation between arrays of two
 * element types with np.result_type (charmnumeric/charmnumeric.py:369-373) but its kernels read
 * every operand in one element type (src/jit.cpp:47-69) and astype raises
 * (charmnumeric.py:738-744): this is the conversion those lines leave open. */
int cnh_convert_region(int ndims, int dst_dtype, void* dst, const int64_t* dst_strides,
                       const int64_t* dst_start, const int64_t* dst_step, int src_dtype, const void* src,
                       const int64_t* src_strides, const int64_t* src_start, const int64_t* src_step,
                       const int64_t* counts, cnh_stream s);
/* Scalar -> dtype conversion used by the fill ((T)double, src/executor_ast_visitor.cpp:112-147). */
int cnh_scalar_to_dtype(int dtype, double s, void* out8);

/* ---- fused groups: ArrayDAGGroup::compile_node (src/dag_group_compile.cpp:6-56) and
 *      dispatch_kernel<N,T> (src/dispatch.hpp:137-265) ---- */
typedef struct cnh_kernel cnh_kernel;
/* Generates HIP source for the group and registers it under `key` (the upstream cache key is
 * node->identifier). Non-zero return = "could not compile": the caller falls back, as upstream
 * does on a null compile result (src/execute_node.cpp:102-112). Code objects are built with
 * hipRTC on first launch of each kernel variant. */
int cnh_compile_group(const cnh_ast* ast, int dtype, int ndims, uint64_t key, cnh_kernel** out);
/* Drops one reference; the kernel object goes with its last holder (a later compile with the same
 * key builds it again). Code objects are shared between kernels with identical generated text
 * and stay loaded. */
/* 1 when `k` was compiled from exactly this AST, element type and rank (a cache keyed by a hash of
 * the AST asks before it reuses a kernel), else 0. */
int cnh_kernel_matches(const cnh_kernel* k, const cnh_ast* ast, int dtype, int ndims);
int cnh_kernel_release(cnh_kernel* k);
/* Argument counts in the upstream order: memref per leaf use, scalar per unique broadcast leaf,
 * memref per non-temp root (src/jit.cpp:78-87). */
int cnh_kernel_signature(const cnh_kernel* k, int* n_in, int* n_scalar, int* n_out);
/* Which array each argument stands for, so a caller can bind buffers by name: input i is leaf
 * use i (array name + the region attached to that use, has_region = 0 when it is the whole
 * array); scalar i is the size-1 array `name`; output i is root `result_name`, which for a
 * SET_REGION root assigns `region` of array `target_name`. */
int cnh_kernel_input(const cnh_kernel* k, int i, int* name, int* has_region, cnh_region* region);
int cnh_kernel_scalar(const cnh_kernel* k, int i, int* name);
int cnh_kernel_output(const cnh_kernel* k, int i, int* result_name, int* target_name,
                      int* is_set_region, cnh_region* region);
/* Generated source of one variant ("flat", "nd", "tiles"), NUL-terminated; returns needed size. */
int64_t cnh_kernel_source(cnh_kernel* k, const char* variant, char* buf, size_t cap);
/* Builds the code object of one variant for gfx950 without loading it (works without a GPU). */
int cnh_kernel_build(cnh_kernel* k, const char* variant);
/* Can the group run as a register-window sweep over a lattice (cnh_launch_group_tiles on arrays
 * stored as one block)? Every region of it then has the same step, 1 or 2, per dimension, its one or
 * two SET_REGION roots assign lattices of one array that share no point (two: the halves of one
 * colour of a red-black sweep, examples/gauss_seidel.py upstream), and operands are read at constant
 * offsets from their root's lattice. 0: no; 1: yes, into a second buffer (dst != cur); 2: yes, also
 * in place (no shifted read of the assigned array can meet an assigned point). */
int cnh_kernel_lattice(const cnh_kernel* k);
/* How many variants whose name starts with `prefix` ("flat", "nd", "tiles", "slide", "direct")
 * have a code object, i.e. were built or launched: tells a test which kernel a launch took. */
int cnh_kernel_variants_loaded(const cnh_kernel* k, const char* prefix);
/* How many distinct code objects this process has compiled so far. Kernels whose generated text is
 * the same share one: groups that differ only in literal scalars other than small multiples of a
 * quarter do (such literals travel with the launch), so a loop whose coefficient changes every
 * step compiles once. Upstream writes every scalar leaf into the module as a constant
 * (src/jit.cpp:108-116). */
int64_t cnh_code_objects(void);
/* With the environment variable CHARMNUMERIC_KERNEL_CACHE naming a directory, code objects are also
 * kept there, one file each (named by the hash of the generated text, which the file repeats in
 * full and which is compared before the code is used), and a later process loads them instead of
 * compiling: how many of the code objects above came from there. Off when the variable is unset.
 * Upstream compiles every group anew in every run (src/dag_group_compile.cpp:6-56). */
int64_t cnh_code_objects_from_disk(void);
/* One fragment / one tile. scalars[i] points at one element of the group dtype; with
 * scalars_on_device != 0 they are device pointers and are read by the kernel itself (no host
 * round trip for dot results feeding later groups). */
int cnh_launch_group(cnh_kernel* k, int ndims, int n_in, const cnh_memref* in, int n_scalar,
                     const void* const* scalars, int scalars_on_device, int n_out,
                     const cnh_memref* out, cnh_stream s);
/* All partitions (or all aligned cells) of a node in ONE launch: in[p*n_in + i], out[p*n_out + o]. */
int cnh_launch_group_batched(cnh_kernel* k, int ndims, int n_parts, int n_in, const cnh_memref* in,
                             int n_scalar, const void* const* scalars, int scalars_on_device,
                             int n_out, const cnh_memref* out, cnh_stream s);
/* Outputs that are CNH_OP_SUM_OF / CNH_OP_MAXABS_OF roots (fp64, dense operands): the memref of such
 * an output names ONE element, which receives the result over all partitions of the launch, or more
 * than one, in which case the launch leaves its partial results there (one per workgroup of 256
 * lanes, i.e. per 512 fp64 elements of a partition; it needs room for all of them) and folds nothing: a later
 * launch takes them through cnh_launch_group_sums. Elements past the last partial are not written,
 * so a buffer that starts out as zeros can be summed over its whole length.
 *
 * cnh_launch_group with run-time scalars that are sums of partial results (no upstream counterpart:
 * upstream finishes every reduction in a pass and a contribute of its own,
 * src/executor_reduce.cpp:60-110). Scalar i is the sum of `count` fp64 values at device address
 * `ptr` (count 1: the value itself), formed by every workgroup in the same fixed order, and stored at
 * `folded` too when that is not null. One partition, dense operands. */
typedef struct cnh_scalar_sum {
    const void* ptr;
    int64_t count;
    void* folded;
} cnh_scalar_sum;
int cnh_launch_group_sums(cnh_kernel* k, int ndims, int n_in, const cnh_memref* in, int n_scalar,
                          const cnh_scalar_sum* scalars, int n_out, const cnh_memref* out, cnh_stream s);
/* *out (device, fp64) = the sum of `count` partial results at `partials`, added in exactly the order a
 * launch uses that takes them as a summed scalar: for the caller that needs the value with no such
 * launch at hand. 1 <= count <= 2^20. */
int cnh_fold_sums(const void* partials, int64_t count, void* out, cnh_stream s);

/* Shifted-slice groups over tiles that all live on this device: replaces send_remote_input +
 * receive_data + align_fragments + M kernel calls + the SET_REGION copy
 * (src/executor_core.cpp:8-143,684-747, src/partition_comm.cpp:26-61,
 *  src/execute_node.cpp:1338-1585, src/executor_ast_visitor.cpp:268-311) by one launch that
 * reads neighbour tiles directly and writes every tile of the target.
 * A tiled array is described by its decomposition (tile edge, per-dim offset and shape,
 * src/array_region.hpp:293-387) and a table of tile base pointers in row-major tile-grid order;
 * every tile is row-major over its own local extent (src/backend.hpp:112-200), contiguous unless
 * pitches are given. */
typedef struct cnh_tiled {
    int32_t ndims;
    int32_t tile;
    int32_t offset[CNH_MAX_ND];
    int32_t shape[CNH_MAX_ND];
    int32_t grid_lo[CNH_MAX_ND];   /* first tile index per dim: offset / tile */
    int32_t grid[CNH_MAX_ND];      /* tiles per dim */
    void* const* tiles;            /* host array of device pointers, prod(grid) entries */
    /* Elements between consecutive indices of each dimension inside a tile. All zero: every tile
     * is contiguous over its own extents (what a partition's buffer is upstream). Non-zero: the
     * tiles are views into one larger row-major block and share these pitches (pitch of the last
     * dimension 1); an executor that holds every partition of an array on one device may store
     * it that way. */
    int64_t pitch[CNH_MAX_ND];
} cnh_tiled;
/* in[i] describes the array behind leaf use i (regions come from the AST); dst is where the
 * SET_REGION target's new contents are written (all elements of every tile: computed inside the
 * assigned region, copied from `cur` outside it); cur is the target's current contents. dst may
 * equal cur only when no input aliases the target with a different region. */
int cnh_launch_group_tiles(cnh_kernel* k, int n_in, const cnh_tiled* in, int n_scalar,
                           const void* const* scalars, int scalars_on_device,
                           const cnh_tiled* cur, const cnh_tiled* dst, cnh_stream s);

/* The same launch, which also reduces what it changes (no upstream counterpart: upstream has no
 * reduction over 2-D or 3-D arrays, src/executor_reduce.cpp:9-12, and its examples fetch the array
 * and use NumPy, examples/multigrid2d.py:659-666). *out (device, fp64) = sum over all elements of
 * (new - old)^2 for mode 0, max |new - old| for mode 1; fp64 groups with cur != dst (the old
 * contents must survive the launch). The whole-array register-window kernel accumulates per
 * wavefront while it sweeps and a second small launch adds the partials in index order, so the
 * residual costs no second pass over the data; every other kernel path is followed by
 * cnh_sumsq_diff_tiles / cnh_maxabs_diff_tiles over (dst, cur). Results never depend on scheduling. */
int cnh_launch_group_tiles_residual(cnh_kernel* k, int n_in, const cnh_tiled* in, int n_scalar,
                                    const void* const* scalars, int scalars_on_device,
                                    const cnh_tiled* cur, const cnh_tiled* dst, int mode, void* out,
                                    cnh_stream s);

/* ---- REDUCE: eigen_dot + contribute + reduce_dot_sum + reduce_result
 *      (src/backend_internal.hpp:88-93, src/executor_reduce.cpp:8-119,
 *       src/executor_reducer.cpp:11-57, src/partition_comm.cpp:69-111) ---- */
/* dot of one 1-D tile -> *partial_slot (device). Fixed grid and fixed-order tree: the result
 * depends only on (n, data), never on scheduling. */
int cnh_dot_partial(int dtype, int64_t n, const void* a, const void* b, void* partial_slot,
                    cnh_stream s);
/* Sequential sum of the per-tile partials in index order -> *out (device). */
int cnh_reduce_final(int dtype, int n_partials, const void* partials, void* out, cnh_stream s);
/* All tiles in one launch + the final pass: out = sum_t dot(a[t], b[t]), tiles in index order. */
int cnh_dot_tiles(int dtype, int n_tiles, const void* const* a, const void* const* b,
                  const int64_t* n, void* out, cnh_stream s);
/* cnh_dot_partial for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). No counterpart upstream. Same kernels, same slicing and
 * the same bits as cnh_dot_partial, but the stage-1 partials go to a 256 KiB array that is part of
 * the library's code object on every device instead of a workspace the library allocates, and the
 * call allocates and frees nothing. n is limited to 2^28 elements (-3 beyond that). All calls on
 * one device share the array: calls that overlap in time on one device (different streams) race;
 * calls on one stream are ordered. Nothing in the array needs clearing between calls: stage 1
 * writes every slot stage 2 reads. */
int cnh_dot_partial_noalloc(int dtype, int64_t n, const void* a, const void* b, void* out,
                            cnh_stream s);
/* Extensions with no upstream counterpart (upstream REDUCE is 1-D dot only,
 * src/executor_reduce.cpp:9-12): sum of elements, sum of squared differences, max |a-b|,
 * over lists of contiguous chunks. fp64 only for the last two. */
int cnh_sum_tiles(int dtype, int n_tiles, const void* const* a, const int64_t* n, void* out,
                  cnh_stream s);
int cnh_sumsq_diff_tiles(int n_tiles, const void* const* a, const void* const* b, const int64_t* n,
                         void* out, cnh_stream s);
int cnh_maxabs_diff_tiles(int n_tiles, const void* const* a, const void* const* b,
                          const int64_t* n, void* out, cnh_stream s);

/* ---- MATMUL (matvec): eigen_gemv_sub + 1-D partial accumulate
 *      (src/backend_internal.hpp:28-41, src/execute_node.cpp:226-229,563-577) ---- */
/* y[i] = beta*y[i] + sum_j A[i*lda + j] * x[j], beta in {0,1}; row-major. */
int cnh_gemv(int dtype, int64_t rows, int64_t cols, const void* A, int64_t lda, const void* x,
             void* y, int beta, cnh_stream s);
/* y += partial (src/execute_node.cpp:572-576). */
int cnh_axpy1(int dtype, int64_t n, const void* partial, void* y, cnh_stream s);
/* The whole tiled matvec in one launch: A is a grid_r x grid_c grid of row-major tiles
 * (tile (i,j) holds rows [i*tile, ..) x cols [j*tile, ..) of a rows x cols matrix, row stride =
 * its own column count); y[r] = sum over column tiles j = 0,1,.. in that order. */
int cnh_gemv_tiles(int dtype, int64_t rows, int64_t cols, int32_t tile, const void* const* tiles,
                   const void* x, void* y, cnh_stream s);

/* cnh_gemv_tiles (fp64) with the vector work around the product of a Krylov iteration taken along
 * (no upstream counterpart: upstream runs MATMUL, REDUCE and the vector update as nodes of their
 * own, examples/cg.py:40-52, src/execute_node.cpp:116-273, src/executor_reduce.cpp:8-119):
 *  - xa != NULL: the vector is formed on the way, x[j] = xa[j] + (S / den[0]) * xb[j] (one rounding
 *    per operation), S = the sum of the num_count values at num in a fixed order; x receives the
 *    vector (a buffer of its own, every element stored once) and *num_folded receives S if not
 *    null. CG: p = r + (r.r_new / r.r_old) p with r.r_new left as partial sums by the launch that
 *    updated r. Needs a square matrix.
 *    *quotient_out receives S / den if not null (CG: beta).
 *  - w != NULL: dot_partials[b] = sum of w[r] * y[r] over the rows of workgroup b (64 rows each, in
 *    row order), b < *n_partials <= dot_capacity; their sum in index order is w . y (CG: p . Ap),
 *    which cnh_launch_group_sums hands to the next launch. w may be x, also when x is formed on the
 *    way: a workgroup reads w at the indices of its own rows only, and those are the elements of x it
 *    stores itself.
 * y must not overlap x, xa, xb or w (-2).
 * Applies to products of 16384 rows or more with even column tiles of at most 8192 columns and
 * 16-byte aligned operands (-3 otherwise: use cnh_gemv_tiles and the separate calls). y has the
 * bits cnh_gemv_tiles gives for the same x. */
typedef struct cnh_gemv_fusion {
    const void* xa;
    const void* xb;
    const void* num;
    int64_t num_count;
    const void* den;
    void* num_folded;
    const void* w;
    void* dot_partials;
    int64_t dot_capacity;
    void* quotient_out;
} cnh_gemv_fusion;
int cnh_gemv_tiles_fused(int64_t rows, int64_t cols, int32_t tile, const void* const* tiles, void* x, void* y,
                         const cnh_gemv_fusion* fusion, int64_t* n_partials, cnh_stream s);

/* The same over a window of a tiled matrix (a sliced or dimension-dropped operand,
 * charmnumeric.py:536-578, src/executor_matmul.cpp:150-498): row r of the window lies in panel row
 * p = (r + row_shift) / tile_rows at local row (r + row_shift) % tile_rows; panels[p * n_col_panels
 * + j] describes the part of tile (p, j) the window covers: base = the element at that tile's
 * local row 0 and the window's first column inside it, ld = the tile's row stride, ncols = columns
 * covered, xoff = index in x of the first of them. y[r] = sum over j = 0,1,.. in that order. */
typedef struct cnh_gemv_panel {
    const void* base;
    int64_t ld;
    int64_t ncols;
    int64_t xoff;
} cnh_gemv_panel;
int cnh_gemv_panels(int dtype, int64_t rows, int32_t n_col_panels, int64_t tile_rows, int64_t row_shift,
                    int64_t n_panels, const cnh_gemv_panel* panels, const void* x, void* y,
                    cnh_stream s);

/* ---- MATMATMUL: C += A_panel * B_panel, row-major with row strides
 *      (src/backend_internal.hpp:113-133, src/executor_incremental.cpp:97-132) ---- */
int cnh_gemm_acc(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                 const void* B, int64_t ldb, void* C, int64_t ldc, cnh_stream s);
/* A list of such products in one launch, with the result of calling cnh_gemm_acc on each job in
 * list order: jobs naming the same C block (same C, M, N, ldc) accumulate into it in that order
 * (the panel pairs of one C partition, src/executor_matmatmul.cpp:105-484); C blocks of
 * different chains must not overlap. */
typedef struct cnh_gemm_job {
    int64_t M, N, K;
    const void* A;
    int64_t lda;
    const void* B;
    int64_t ldb;
    void* C;
    int64_t ldc;
} cnh_gemm_job;
int cnh_gemm_acc_batch(int dtype, int njobs, const cnh_gemm_job* jobs, cnh_stream s);
/* The same with a choice of what happens to C. overwrite = 0: C += the products of its chain
 * (cnh_gemm_acc_batch). overwrite = 1 (fp64 only): C = the products of its chain; what C held is
 * neither read nor kept, so a freshly allocated result needs no zero-fill
 * (upstream zero-fills result_data and accumulates, src/executor_matmatmul.cpp:105-160). */
int cnh_gemm_batch(int dtype, int njobs, const cnh_gemm_job* jobs, int overwrite, cnh_stream s);

/* One overwriting fp64 product C = A @ B and, in the same launch, the statements of a compiled
 * group evaluated on its result (no upstream counterpart: upstream runs the panel products,
 * src/executor_incremental.cpp:97-132, and the groups that read their result,
 * src/dispatch.hpp:137-265, as separate tasks; examples/lstm_forward.py:40-49 is the
 * program this is for: the gate statements of a step behind its product). The product's N columns
 * are n_blocks (1, 2 or 4) column blocks of equal width; the group's memrefs all have the extents
 * (1, ..., M, N / n_blocks), and input i with in_block[i] >= 0 is column block in_block[i] of the
 * product (its memref is not read: the values come from the workgroup's tile of sums), the others
 * are read through their memrefs. C receives the product as cnh_gemm_batch(overwrite = 1) would
 * leave it, bit for bit, and the outputs what cnh_launch_group would store when launched behind
 * it. The statements of an element run as soon as its workgroup's sums are complete, while other
 * workgroups still multiply: no output may overlap A, B or C, and no input other than the
 * product's blocks may overlap C or an output at a different element.
 * Returns -17 without launching anything for shapes the fused kernel does not take: it is built
 * in the three forms cnh_gemm_batch runs aligned products in (by tile count and K), so M and N must
 * be multiples of 64, K of 16, lda and ldb even and A and B 16-byte aligned; the caller then issues
 * cnh_gemm_batch and cnh_launch_group. */
int cnh_launch_product_group(cnh_kernel* k, const cnh_gemm_job* job, int n_blocks, int ndims, int n_in,
                             const cnh_memref* in, const int32_t* in_block, int n_scalar,
                             const void* const* scalars, int scalars_on_device, int n_out,
                             const cnh_memref* out, cnh_stream s);

/* ---- synthetic inputs generated on the device (no upstream counterpart: upstream has no RNG,
 *      charmnumeric/random.py:4-5, and no bulk upload, charmnumeric.py:863-878) ---- */
/* out[k] = lo + (hi-lo)*u01(seed, stream_id, first+k); counter-based SplitMix64, fp64. */
int cnh_fill_uniform(double* out, int64_t n, uint64_t seed, uint64_t stream_id, uint64_t first,
                     double lo, double hi, cnh_stream s);
/* One tile of a row-major global array: the counter of an element is its global flat index, so
 * the tiles of an array together hold exactly what one global fill would produce. */
int cnh_fill_uniform_tile(double* out, int ndims, const int64_t* ext, const int64_t* origin,
                          const int64_t* global_shape, uint64_t seed, uint64_t stream_id, double lo,
                          double hi, cnh_stream s);

#ifdef __cplusplus
}
#endif
#endif
