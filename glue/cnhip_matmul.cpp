// MATMUL (matrix times vector) on libcnhip: the tile product of a 2-D chare and the accumulation
// of the partial rows on the 1-D owner.
// Replaces, inside the interpreter branch of execute_node_nd, the tile product
// (src/execute_node.cpp:116-273 upstream: eigen_gemv_sub / KokkosBlas::gemv at :226-229 and the
// reassembly of the vector from its fragments at :159-190) and the accumulate on the 1-D chare
// (src/execute_node.cpp:489-583: `eigen_res += eigen_partial` at :563-577). What selects the
// overlapping rows and columns (:128-157), creates the result array (:196-205) and ships the
// partial rows (:234-266) is upstream's and is only called from here.
// Not compiled in this repository (needs charm++.h and charmtyles).
#include "backend_internal.hpp"

#include <algorithm>

#include "cnhip.h"
#include "cnhip_array.hpp"

// The slice of the vector this tile multiplies with, as ONE device buffer. A single fragment is
// used where it lies; several are laid end to end in ascending order of their start (upstream
// sorts and memcpy's on the host, :168-187; here the pieces are device buffers and the copies are
// queued on the partition's stream).
template <int N, typename T>
static const T* gather_vector(PartitionImpl<N>* partition, std::vector<RemoteBuffer<N>>& pieces,
                              int* length, T** owned) {
    *owned = nullptr;
    *length = 0;
    if (pieces.empty())
        return nullptr;
    if (pieces.size() == 1) {
        *length = (int)(pieces[0].byte_size / sizeof(T));
        return reinterpret_cast<const T*>(pieces[0].data);
    }
    std::sort(pieces.begin(), pieces.end(), [](const RemoteBuffer<N>& x, const RemoteBuffer<N>& y) {
        return x.region.start[0] < y.region.start[0];
    });
    size_t bytes = 0;
    for (const auto& p : pieces)
        bytes += (size_t)p.byte_size;
    CNH_OR_ABORT(cnh_alloc(bytes, 0, (void**)owned));
    size_t at = 0;
    for (const auto& p : pieces) {
        CNH_OR_ABORT(cnh_d2d(reinterpret_cast<char*>(*owned) + at, p.data, (size_t)p.byte_size,
                             partition->compute_stream));
        at += (size_t)p.byte_size;
    }
    *length = (int)(bytes / sizeof(T));
    return *owned;
}

// 2-D chare: result[0:sub_rows] = mat[row_offset:+sub_rows, col_offset:+cols] * vec[0:cols].
// `mat` is the local tile (row stride local_cols); the window (row_offset, col_offset, sub_rows,
// sub_cols) is what upstream computes at :139-157 from the operand region and the decomposition.
template <typename T>
static void tile_matvec(PartitionImpl<2>* partition, Array<2, T>* mat, int local_cols, int row_offset,
                        int col_offset, int sub_rows, int sub_cols,
                        std::vector<RemoteBuffer<2>>& vector_pieces, Array<2, T>* result) {
    int vec_len = 0;
    T* owned = nullptr;
    const T* vec = gather_vector<2, T>(partition, vector_pieces, &vec_len, &owned);
    const int cols = std::min(sub_cols, vec_len);
    if (vec != nullptr && sub_rows > 0 && cols > 0) {
        const T* window = static_cast<const T*>(mat->device_data_ptr()) +
                          (int64_t)row_offset * local_cols + col_offset;
        CNH_OR_ABORT(cnh_gemv(static_cast<int>(dtype_of<T>()), sub_rows, cols, window, local_cols, vec,
                              result->device_data_ptr(), /*beta=*/0, partition->compute_stream));
    }
    if (owned != nullptr) {
        // the product is queued behind the copies on the same stream; free after it has run
        CNH_OR_ABORT(cnh_stream_sync(partition->compute_stream));
        cnh_free(owned);
    }
}

// 1-D owner: every received partial covers rows [partial_start, +len) of the result and is added
// in arrival order into the zero-initialised result tile (same order as upstream's loop, :556-577).
template <typename T>
static void accumulate_partials(PartitionImpl<1>* partition, CTArrayBase<1>* result, int my_result_start,
                                const std::vector<RemoteBuffer<1>>& partials) {
    T* res = static_cast<T*>(result->device_data_ptr());
    for (const auto& rb : partials) {
        const int64_t len = rb.byte_size / (int64_t)sizeof(T);
        const int64_t at = rb.region.start[0] - my_result_start;
        CNH_OR_ABORT(cnh_axpy1(static_cast<int>(dtype_of<T>()), len, rb.data, res + at,
                               partition->compute_stream));
    }
}

// Where every tile of the matrix lives in this process (+p1, one GPU), the whole node is one
// launch issued by the group instead of one product per chare plus messages: rows summed over the
// column tiles in index order.
template <typename T>
static void matvec_all_tiles_local(ArrayDAGGroup* dag_group, int mat_name, int vec_name, int result_name,
                                   cnh_stream stream) {
    const ArrayMeta& meta = dag_group->array_meta[mat_name];
    std::vector<const void*> tiles;                        // row-major over the chare grid
    dag_group->collect_local_tiles_2d(mat_name, tiles);
    CNH_OR_ABORT(cnh_gemv_tiles(static_cast<int>(dtype_of<T>()), meta.global_shape[0], meta.global_shape[1],
                                meta.tile, tiles.data(), dag_group->device_ptr_1d(vec_name),
                                dag_group->device_ptr_1d(result_name), stream));
}
