// dispatch_kernel<N,T> on libcnhip: the packed-argument call of a JIT function becomes one
// cnh_launch_group with the same three argument classes in the same order — a memref per leaf use,
// a pointer per broadcast scalar, a memref per non-temporary root.
// Replaces src/dispatch.hpp:137-265 upstream (all four back ends of it). The callers keep their
// shape: the fast path of execute_node_nd (src/execute_node.cpp:1263-1336) calls it once per chare,
// the fragment path (:1338-1585) once per aligned cell.
// Not compiled in this repository (needs charm++.h and charmtyles).
#pragma once

#include <vector>

#include "cnhip.h"
#include "cnhip_array.hpp"   // CNH_OR_ABORT

// MemRef<N,T> {allocated, aligned, offset, sizes[N], strides[N]} (src/array_region.hpp:404-415) and
// cnh_memref carry the same fields; entries beyond N stay zero.
template <int N, typename T>
static inline cnh_memref as_cnh_memref(const MemRef<N, T>& m) {
    cnh_memref out = {};
    out.allocated = m.allocated;
    out.aligned = m.aligned;
    out.offset = m.offset;
    for (int d = 0; d < N; ++d) {
        out.sizes[d] = m.sizes[d];
        out.strides[d] = m.strides[d];
    }
    return out;
}

/// @param func_ptr         what ArrayDAGGroup::compile_node returned (a cnh_kernel*)
/// @param descs            inputs first (n_input_memrefs of them), then outputs
/// @param scalar_args      device addresses of the size-1 arrays behind the broadcast leaves: the
///                         kernel reads them itself, so the copyToHost of the broadcast path
///                         (src/executor_core.cpp:390-605) is not needed before the call
/// @param stream           the partition's compute stream; the call returns once the launch is queued
template <int N, typename T = float>
static void dispatch_kernel(void* func_ptr, int n_memrefs, std::vector<MemRef<N, T>>& descs,
                            int n_input_memrefs = -1, const std::vector<void*>& scalar_args = {},
                            cnh_stream stream = nullptr) {
    if (n_input_memrefs < 0)
        n_input_memrefs = n_memrefs;
    std::vector<cnh_memref> refs;
    refs.reserve((size_t)n_memrefs);
    for (int i = 0; i < n_memrefs; ++i)
        refs.push_back(as_cnh_memref<N, T>(descs[(size_t)i]));
    const int n_outputs = n_memrefs - n_input_memrefs;
    CNH_OR_ABORT(cnh_launch_group(static_cast<cnh_kernel*>(func_ptr), N, n_input_memrefs, refs.data(),
                                  (int)scalar_args.size(), scalar_args.data(), /*scalars_on_device=*/1,
                                  n_outputs, refs.data() + n_input_memrefs, stream));
}

/// All chares of a PE (or all aligned cells of a chare) in one launch: parts[p] holds the memrefs
/// of partition p in the order dispatch_kernel takes them. A PE that owns several chares collects
/// their descriptors while it walks them and calls this once per node.
template <int N, typename T = float>
static void dispatch_kernel_batched(void* func_ptr, const std::vector<std::vector<MemRef<N, T>>>& parts,
                                    int n_input_memrefs, const std::vector<void*>& scalar_args,
                                    cnh_stream stream) {
    if (parts.empty())
        return;
    const int per_part = (int)parts.front().size(), n_outputs = per_part - n_input_memrefs;
    std::vector<cnh_memref> ins, outs;
    for (const auto& part : parts) {
        for (int i = 0; i < n_input_memrefs; ++i)
            ins.push_back(as_cnh_memref<N, T>(part[(size_t)i]));
        for (int i = n_input_memrefs; i < per_part; ++i)
            outs.push_back(as_cnh_memref<N, T>(part[(size_t)i]));
    }
    CNH_OR_ABORT(cnh_launch_group_batched(static_cast<cnh_kernel*>(func_ptr), N, (int)parts.size(),
                                          n_input_memrefs, ins.data(), (int)scalar_args.size(),
                                          scalar_args.data(), 1, n_outputs, outs.data(), stream));
}

/// Completion without stalling the scheduler: replaces CT_KOKKOS_FENCE(); node_finished(id)
/// (src/executor_core.cpp:618-627,761-774) and the hapiAddCallback form (src/dispatch.hpp:40-53).
template <int N>
struct NodeDone {
    PartitionImpl<N>* partition;
    int node_id;
};
template <int N>
static void node_done_trampoline(void* arg) {
    auto* done = static_cast<NodeDone<N>*>(arg);
    // back onto the chare's own scheduler: an entry method, not a direct call from the HIP thread
    done->partition->thisProxy[done->partition->thisIndex].comm_done(done->node_id);
    delete done;
}
template <int N>
static void finish_node_from_stream(PartitionImpl<N>* partition, int node_id, cnh_stream stream) {
    CNH_OR_ABORT(cnh_stream_callback(stream, node_done_trampoline<N>, new NodeDone<N>{partition, node_id}));
}
