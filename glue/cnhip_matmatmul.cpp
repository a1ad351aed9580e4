// MATMATMUL on libcnhip: a panel that has just arrived is multiplied with every panel of the other
// operand it shares a k range with, and the product is added into this chare's tile of C.
// Replaces the arithmetic of ArrayDAGExecutorND<N>::on_matmatmul_receive
// (src/executor_incremental.cpp:10-159 upstream: the Eigen map product at :120-132 and the
// KokkosBlas::gemm at :97-118). Panel bookkeeping (which buffers exist, their regions) is upstream's.
// Panels are packed row-major: A panels (rows of C) x (k range), B panels (k range) x (columns of C);
// region.start/stop[0] is the k range, [1] the rows of C (A) or the columns of C (B).
// Not compiled in this repository (needs charm++.h and charmtyles).
#include "backend_internal.hpp"

#include <algorithm>

#include "cnhip.h"
#include "cnhip_array.hpp"

template <int N>
void ArrayDAGExecutorND<N>::on_matmatmul_receive(int node_id, int input_index) {
    if constexpr (N == 2) {
        auto pending_it = pending.find(node_id);
        if (pending_it == pending.end())
            return;
        PendingComm<N>& comm = pending_it->second;
        auto& mine = comm.remote_buffers[input_index];
        auto others = comm.remote_buffers.find(1 - input_index);
        if (mine.empty() || others == comm.remote_buffers.end() || others->second.empty())
            return;
        const RemoteBuffer<N>& fresh = mine.back();

        ASTNode* root = nullptr;
        for (ASTNode* r : comm.node->ast->roots)
            if (static_cast<Opcode>(r->opcode) == Opcode::MATMATMUL)
                root = r;
        if (root == nullptr)
            return;
        auto c_it = partition->arrays.find(root->result_name);
        if (c_it == partition->arrays.end())
            return;
        CTArrayBase<N>* c = c_it->second;
        const auto idx = partition->nd_index();
        const int c_row0 = c->decomp.chare_start_global(0, idx[0]);
        const int c_col0 = c->decomp.chare_start_global(1, idx[1]);
        const int64_t ldc = c->region.size(1);
        const int esz = c->elem_size();

        // all pairs of this arrival in one launch; jobs on one C block accumulate in list order
        std::vector<cnh_gemm_job> jobs;
        for (const RemoteBuffer<N>& other : others->second) {
            const RemoteBuffer<N>& a = input_index == 0 ? fresh : other;
            const RemoteBuffer<N>& b = input_index == 0 ? other : fresh;
            const int k_lo = std::max(a.region.start[0], b.region.start[0]);
            const int k_hi = std::min(a.region.stop[0], b.region.stop[0]);
            if (k_lo >= k_hi)
                continue;
            const int64_t a_k = a.region.stop[0] - a.region.start[0];      // row stride of the A panel
            const int64_t b_cols = b.region.stop[1] - b.region.start[1];   // row stride of the B panel
            cnh_gemm_job job;
            job.M = a.region.stop[1] - a.region.start[1];
            job.N = b_cols;
            job.K = k_hi - k_lo;
            job.A = static_cast<const char*>(a.data) + (int64_t)(k_lo - a.region.start[0]) * esz;
            job.lda = a_k;
            job.B = static_cast<const char*>(b.data) + (int64_t)(k_lo - b.region.start[0]) * b_cols * esz;
            job.ldb = b_cols;
            job.C = static_cast<char*>(c->device_data_ptr()) +
                    ((int64_t)(a.region.start[1] - c_row0) * ldc + (b.region.start[1] - c_col0)) * esz;
            job.ldc = ldc;
            jobs.push_back(job);
        }
        if (!jobs.empty())
            CNH_OR_ABORT(cnh_gemm_acc_batch(static_cast<int>(c->dtype), (int)jobs.size(), jobs.data(),
                                            partition->compute_stream));
    }
}

template void ArrayDAGExecutorND<1>::on_matmatmul_receive(int, int);
template void ArrayDAGExecutorND<2>::on_matmatmul_receive(int, int);
template void ArrayDAGExecutorND<3>::on_matmatmul_receive(int, int);
