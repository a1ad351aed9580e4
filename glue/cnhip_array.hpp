// Array<N,T> on libcnhip: one zero-filled device buffer per chare tile, no host mirror.
// Replaces the storage members and bodies of Array<N,T> in src/backend.hpp:112-200 upstream
// (constructor zero-fill :122-144, non-owning wrapper :147-160, destructor :162-168, data_ptr /
// device_data_ptr :170-184, copyToHost / copyToDevice :188-199). CTArrayBase<N> (:92-110) is
// unchanged. Not compiled in this repository (needs charm++.h and charmtyles).
#pragma once

#include <vector>

#include "cnhip.h"

#define CNH_OR_ABORT(call)                                                                        \
    do {                                                                                          \
        if ((call) != 0)                                                                          \
            CkAbort("libcnhip: %s", cnh_last_error());                                            \
    } while (0)

template <int N, typename T = float>
class Array : public CTArrayBase<N> {
    T* dev_ = nullptr;            // the tile, row-major over the local region
    std::vector<T> staging_;      // host copy, filled only by copyToHost() (gather / debugging)

    void describe(int name_, DType dt) {
        this->name = name_;
        this->dtype = dt;
    }

  public:
    // Owning tile of `region_` (src/backend.hpp:122-144): zero-filled on the device. The fill is
    // queued on the partition's compute stream (the stream every kernel on this tile is launched
    // on, src/backend.hpp:549-554), so the entry method that creates the array returns without
    // waiting for it; a caller with no such stream passes nullptr and cnh_alloc's blocking form
    // applies instead.
    Array(ArrayRegion<N> region_, std::array<int, N> global_shape_, int name_, ArrayDecomp<N> decomp_,
          cnh_stream compute_stream = nullptr) {
        describe(name_, dtype_of<T>());
        this->region = region_;
        this->global_shape = global_shape_;
        this->decomp = decomp_;
        this->owner = true;
        this->global_size = 1;
        for (int extent : global_shape_)
            this->global_size *= extent;
        const size_t bytes = sizeof(T) * (size_t)this->region.size();
        if (compute_stream != nullptr)
            CNH_OR_ABORT(cnh_alloc_on(bytes, /*zero=*/1, compute_stream, (void**)&dev_));
        else
            CNH_OR_ABORT(cnh_alloc(bytes, /*zero=*/1, (void**)&dev_));
    }

    // Wrapper around a device buffer somebody else owns (src/backend.hpp:147-160 zeroes it too).
    Array(T* device_data, int name_, int size_) {
        describe(name_, dtype_of<T>());
        this->owner = false;
        this->global_size = size_;
        dev_ = device_data;
        CNH_OR_ABORT(cnh_memset0(dev_, sizeof(T) * (size_t)size_, nullptr));
        CNH_OR_ABORT(cnh_stream_sync(nullptr));
    }

    ~Array() override {
        if (this->owner)
            cnh_free(dev_);
    }

    // Free-list reuse (src/backend.hpp:490-497 zeroes a recycled buffer): on the partition's stream,
    // ordered before whatever writes the array next.
    void zero(cnh_stream stream) {
        CNH_OR_ABORT(cnh_memset0(dev_, sizeof(T) * (size_t)this->local_size(), stream));
    }

    void* device_data_ptr() override { return dev_; }

    // The host view exists only after copyToHost(); kernels never read it.
    void* data_ptr() override {
        if (staging_.empty())
            staging_.resize((size_t)this->local_size());
        return staging_.data();
    }

    int elem_size() const override { return sizeof(T); }

    void copyToHost() override {
        staging_.resize((size_t)this->local_size());
        CNH_OR_ABORT(cnh_d2h(staging_.data(), dev_, sizeof(T) * staging_.size(), nullptr));
    }

    void copyToDevice() override {
        if (!staging_.empty())
            CNH_OR_ABORT(cnh_h2d(dev_, staging_.data(), sizeof(T) * staging_.size(), nullptr));
    }
};
