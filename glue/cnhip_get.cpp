// get / gather on libcnhip: a chare hands its tile to PE 0 as ONE contiguous message of the
// tile's bytes plus the tile's place in the global array, instead of one message per innermost
// row read from a host mirror.
// Replaces PartitionImpl<N>::process_get (src/partition_get.cpp:4-67 upstream: copyToHost at :24
// and the row loop at :42-65). The receiving side, ArrayDAGGroup::gather
// (src/dag_group_runtime.cpp:99-118), copies rows of the tile into the global row-major buffer
// with the strides sent along; where PE 0 holds every chare itself (+p1) it skips the messages
// and calls cnh_d2h_region per tile straight into the reply buffer.
// Not compiled in this repository (needs charm++.h and charmtyles).
#include "backend_internal.hpp"

#include <vector>

#include "cnhip.h"
#include "cnhip_array.hpp"

template <int N>
void PartitionImpl<N>::process_get(int epoch) {
    auto* req = executor->group->get_get_request(N, epoch);
    if (req == nullptr)
        CkAbort("No get request found for epoch %d", epoch);
    auto found = arrays.find(req->name);
    if (found == arrays.end())
        return;                      // this chare holds no part of the array
    CTArrayBase<N>* arr = found->second;
    const auto where = arr->decomp.chare_region_global(this->nd_index());
    const int esz = arr->elem_size();

    int64_t tile_strides[N], global_strides[N], starts[N], zero[N], counts[N];
    int64_t run_t = 1, run_g = 1;
    for (int d = N - 1; d >= 0; --d) {
        tile_strides[d] = run_t;
        global_strides[d] = run_g;
        run_t *= arr->region.size(d);
        run_g *= arr->global_shape[d];
        starts[d] = where.start[d] - arr->decomp.offset[d];   // position in the array itself
        zero[d] = 0;
        counts[d] = arr->region.size(d);
    }

    auto* dag_group = static_cast<ArrayDAGGroup*>(dag_proxy.ckLocalBranch());
    if (char* reply = dag_group->local_get_buffer(epoch)) {
        // PE 0 assembles the reply itself: strided device -> host copy, one 2-D copy per plane
        CNH_OR_ABORT(cnh_d2h_region(N, esz, reply, global_strides, starts, arr->device_data_ptr(),
                                    tile_strides, zero, counts, compute_stream));
        dag_group->tile_gathered(epoch, req->name);
        return;
    }
    // other PEs: the tile in one message (a pinned staging block would make the copy asynchronous;
    // a get is a synchronisation point of the program anyway)
    std::vector<char> tile((size_t)run_t * esz);
    CNH_OR_ABORT(cnh_d2h(tile.data(), arr->device_data_ptr(), tile.size(), compute_stream));
    dag_proxy[0].gather_tile(epoch, req->name, N, starts, counts, (int64_t)tile.size(), tile.data());
}

template void PartitionImpl<1>::process_get(int);
template void PartitionImpl<2>::process_get(int);
template void PartitionImpl<3>::process_get(int);
