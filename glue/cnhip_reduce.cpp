// REDUCE (1-D dot) on libcnhip. Two forms:
//  (a) the upstream message flow kept as it is — every chare contributes its partial through the
//      custom reducer — with the per-chare Eigen/KokkosBlas dot replaced by cnh_dot_partial; the
//      partial is computed on the device and only its 8 bytes come to the host for the message;
//  (b) all chares of the array in this process (+p1, one GPU): one cnh_dot_tiles launch writes the
//      result straight into the size-1 result array, tiles added in index order, no message.
// Replaces ArrayDAGExecutorND<N>::execute_reduce_node (src/executor_reduce.cpp:8-119 upstream) and
// the store in PartitionImpl<N>::reduce_result (src/partition_comm.cpp:69-111). The reducer
// reduce_dot_sum (src/executor_reducer.cpp:11-57) is unchanged.
// Not compiled in this repository (needs charm++.h and charmtyles).
#include "backend_internal.hpp"

#include "cnhip.h"
#include "cnhip_array.hpp"

namespace {
ASTNode* find_root(DAGNode* node, Opcode wanted) {
    for (ASTNode* root : node->ast->roots)
        if (static_cast<Opcode>(root->opcode) == wanted)
            return root;
    return nullptr;
}
} // namespace

template <int N>
void ArrayDAGExecutorND<N>::execute_reduce_node(DAGNode* node) {
    if constexpr (N != 1) {
        CkAbort("REDUCE only supported for 1D partitions (N=%d)", N);
    } else {
        ASTNode* root = find_root(node, Opcode::REDUCE);
        const int lhs = root->operands[0]->result_name, rhs = root->operands[1]->result_name;
        const DType dt = determine_dtype<1>(node, partition->arrays);
        auto* dag_group = static_cast<ArrayDAGGroup*>(group);

        auto a = partition->arrays.find(lhs), b = partition->arrays.find(rhs);
        const bool have = a != partition->arrays.end() && b != partition->arrays.end();
        const int64_t n = have ? std::min(a->second->local_size(), b->second->local_size()) : 0;

        if (dag_group->all_chares_local_1d()) {
            // (b) chare 0 launches for everybody: pointers and lengths of all tiles, in chare order
            if (partition->nd_index()[0] == 0) {
                std::vector<const void*> pa, pb;
                std::vector<int64_t> len;
                dag_group->collect_local_tiles_1d(lhs, rhs, pa, pb, len);
                CTArrayBase<1>* out = partition->ensure_scalar_result(root->result_name, dt);
                CNH_OR_ABORT(cnh_dot_tiles(static_cast<int>(dt), (int)len.size(), pa.data(), pb.data(),
                                           len.data(), out->device_data_ptr(), partition->compute_stream));
                finish_node_from_stream<1>(partition, node->id, partition->compute_stream);
            } else {
                node_finished(node->id);
            }
            return;
        }

        // (a) one partial per chare, summed by the reducer in the order Charm++ delivers them
        ReduceContrib contrib = {};
        contrib.node_id = node->id;
        contrib.result_name = root->result_name;
        contrib.dtype_int = static_cast<int>(dt);
        if (have && n > 0) {
            void* slot = partition->scratch_scalar();       // 8 bytes of device memory per partition
            CNH_OR_ABORT(cnh_dot_partial(static_cast<int>(dt), n, a->second->device_data_ptr(),
                                         b->second->device_data_ptr(), slot, partition->compute_stream));
            CNH_OR_ABORT(cnh_d2h(contrib.value, slot, (size_t)dtype_size(dt), partition->compute_stream));
        }
        ChareIndex<1> first;
        first.idx[0] = 0;
        CkCallback cb(CkIndex_Partition1D::reduce_result(nullptr),
                      proxy_at<1>(dag_group->partition_proxy_1, first));
        partition->contribute(sizeof(ReduceContrib), &contrib, reduce_dot_sum_type, cb);
        if (partition->nd_index()[0] != 0)
            node_finished(node->id);                         // chare 0 finishes in reduce_result
    }
}

// The part of PartitionImpl<N>::reduce_result that stores the value (src/partition_comm.cpp:92-104):
// the summed scalar goes into the device buffer of the size-1 result array.
template <int N>
void PartitionImpl<N>::store_reduce_result(int result_name, DType dt, const char* value) {
    CNH_OR_ABORT(cnh_h2d(arrays[result_name]->device_data_ptr(), value, (size_t)dtype_size(dt),
                         compute_stream));
}

template void ArrayDAGExecutorND<1>::execute_reduce_node(DAGNode*);
template void ArrayDAGExecutorND<2>::execute_reduce_node(DAGNode*);
template void ArrayDAGExecutorND<3>::execute_reduce_node(DAGNode*);
