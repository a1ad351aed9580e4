// libcnhip runtime: device selection, storage, copies, streams/events, descriptor cache.
// Stands in for Array<N,T> storage (src/backend.hpp:112-200 upstream), the row-wise gather of
// src/partition_get.cpp:42-65 and the fence/callback completion of src/dispatch.hpp:40-53.
#include "common.h"

#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace cnh {

std::string& error_slot() {
    static thread_local std::string msg;
    return msg;
}

int set_error(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    error_slot() = buf;
    return code;
}

namespace {
std::mutex g_mu;
bool g_inited = false;
int g_device = 0;
constexpr int kMaxDevices = 64;

struct Workspace {
    void* ptr = nullptr;
    size_t bytes = 0;
    std::vector<void*> retired; // outgrown blocks, possibly still read by kernels in flight
};

struct DescEntry {
    size_t off, bytes;
    hipStream_t stream; // where the copy was queued
    bool visible;       // known complete for every stream
};

// Everything the library keeps in device memory belongs to one device.
const size_t kSlabBytes = 16u << 20;
struct DeviceState {
    std::unordered_map<hipStream_t, Workspace> ws;
    // Descriptor slab: device memory + pinned host mirror, bump-allocated.
    char* slab_dev = nullptr;
    char* slab_host = nullptr;
    size_t slab_used = 0;
    std::unordered_map<uint64_t, std::vector<DescEntry>> desc;
    hipStream_t fill_stream = nullptr; // zero-fills of fresh allocations
};
DeviceState g_dev[kMaxDevices];

DeviceState& dev_state() { return g_dev[g_device]; }

// Content hash of a descriptor table, eight bytes a step: tables of a few thousand tile pointers are
// hashed on every launch that names them.
uint64_t table_hash(const void* p, size_t n) {
    const unsigned char* b = static_cast<const unsigned char*>(p);
    uint64_t h = 0x9E3779B97F4A7C15ull ^ n;
    for (; n >= 8; n -= 8, b += 8) {
        uint64_t w;
        std::memcpy(&w, b, 8);
        h = (h ^ w) * 0xD6E8FEB86659FD93ull;
        h ^= h >> 32;
    }
    for (; n > 0; --n, ++b) {
        h = (h ^ *b) * 0x100000001B3ull;
        h ^= h >> 29;
    }
    return h;
}

// Blocks a workspace outgrew are freed once the stream that used them has drained.
int release_retired(Workspace& w) {
    for (void* p : w.retired)
        CNH_HIP(hipFree(p));
    w.retired.clear();
    return 0;
}
} // namespace

// Device and pinned-host allocations and descriptor-table copies the library has made: what a
// caller that must not allocate (a stream under graph capture) can watch.
std::atomic<int64_t> g_allocations{0};

int ensure_init() {
    if (g_inited)
        return 0;
    return cnh_init(0);
}

int current_device() { return g_inited ? g_device : -1; }

int reduce_workspace(hipStream_t s, size_t bytes, void** out) {
    std::lock_guard<std::mutex> lk(g_mu);
    Workspace& w = dev_state().ws[s];
    if (w.bytes < bytes) {
        size_t want = bytes < (1u << 20) ? (1u << 20) : bytes;
        void* p = nullptr;
        CNH_HIP(hipMalloc(&p, want));
        g_allocations++;
        // The old block may still be read by kernels in flight on `s`: it waits in `retired` for
        // the next synchronisation of that stream.
        if (w.ptr)
            w.retired.push_back(w.ptr);
        w.ptr = p;
        w.bytes = want;
    }
    *out = w.ptr;
    return 0;
}

// Descriptor tables are content-addressed: a table seen before is reused. A new one is written to
// the pinned mirror of the slab and copied on the consumer's own stream, ahead of the kernel that
// reads it, so the host does not wait for the copy. A slot of the mirror is written once per pass
// over the slab, and the slab is recycled only after the device has drained.
int desc_upload(const void* host, size_t bytes, hipStream_t st, const void** dev_out) {
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceState& D = dev_state();
    if (!D.slab_dev) {
        CNH_HIP(hipMalloc((void**)&D.slab_dev, kSlabBytes));
        CNH_HIP(hipHostMalloc((void**)&D.slab_host, kSlabBytes, hipHostMallocDefault));
        g_allocations += 2;
    }
    CNH_CHECK(bytes <= kSlabBytes / 4, -3, "descriptor table of %zu bytes is too large", bytes);
    uint64_t h = table_hash(host, bytes);
    auto it = D.desc.find(h);
    if (it != D.desc.end())
        for (DescEntry& e : it->second)
            if (e.bytes == bytes && std::memcmp(D.slab_host + e.off, host, bytes) == 0) {
                if (!e.visible && e.stream != st) {
                    // uploaded on another stream: its copy must have landed before this one reads
                    CNH_HIP(hipStreamSynchronize(e.stream));
                    e.visible = true;
                }
                *dev_out = D.slab_dev + e.off;
                return 0;
            }
    size_t need = (bytes + 255) & ~size_t(255);
    if (D.slab_used + need > kSlabBytes) {
        // Tables handed out earlier may still be in use by queued kernels: drain, then recycle.
        CNH_HIP(hipDeviceSynchronize());
        D.desc.clear();
        D.slab_used = 0;
    }
    size_t off = D.slab_used;
    D.slab_used += need;
    std::memcpy(D.slab_host + off, host, bytes);
    CNH_HIP(hipMemcpyAsync(D.slab_dev + off, D.slab_host + off, bytes, hipMemcpyHostToDevice, st));
    g_allocations++;
    D.desc[h].push_back({off, bytes, st, false});
    *dev_out = D.slab_dev + off;
    return 0;
}

} // namespace cnh

using namespace cnh;

extern "C" {

int cnh_version(void) { return 100; }

const char* cnh_last_error(void) { return error_slot().c_str(); }

int cnh_init(int device) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_inited && device == g_device)
        return 0;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return set_error(-101, "no HIP device available (%s)",
                         e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    CNH_CHECK(device >= 0 && device < count && device < kMaxDevices, -2,
              "device %d out of range (have %d)", device, count);
    CNH_HIP(hipSetDevice(device));
    // Descriptor tables, reduction workspaces and the scratch array are kept per device, so a
    // later call with another device finds its own (or none yet) and never one of this device.
    if (int rc = reduce_scratch_init(device))
        return rc;
    g_device = device;
    g_inited = true;
    return 0;
}

int cnh_device_name(char* buf, size_t cap) {
    if (int rc = ensure_init())
        return rc;
    hipDeviceProp_t prop;
    CNH_HIP(hipGetDeviceProperties(&prop, g_device));
    // some driver stacks leave the marketing name empty
    snprintf(buf, cap, "%s (%s, %d CUs)", prop.name[0] ? prop.name : "AMD GPU", prop.gcnArchName,
             prop.multiProcessorCount);
    return 0;
}

int cnh_alloc(size_t bytes, int zero, void** dptr) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(dptr != nullptr, -2, "cnh_alloc: null output pointer");
    void* p = nullptr;
    CNH_HIP(hipMalloc(&p, bytes ? bytes : 1));
    g_allocations++;
    if (zero && bytes) {
        // The caller may first write the block on any stream, and no stream waits for another's
        // fill by itself: the fill runs on a stream of the library's own and the host waits for
        // that stream alone, so work queued elsewhere keeps running meanwhile.
        hipStream_t fs;
        {
            std::lock_guard<std::mutex> lk(g_mu);
            DeviceState& D = dev_state();
            if (!D.fill_stream)
                CNH_HIP(hipStreamCreateWithFlags(&D.fill_stream, hipStreamNonBlocking));
            fs = D.fill_stream;
        }
        CNH_HIP(hipMemsetAsync(p, 0, bytes, fs));
        CNH_HIP(hipStreamSynchronize(fs));
    }
    *dptr = p;
    return 0;
}

int cnh_alloc_on(size_t bytes, int zero, cnh_stream s, void** dptr) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(dptr != nullptr, -2, "cnh_alloc_on: null output pointer");
    void* p = nullptr;
    CNH_HIP(hipMalloc(&p, bytes ? bytes : 1));
    g_allocations++;
    // the fill is ordered with whatever the caller queues on `s` next; the host does not wait
    if (zero && bytes)
        CNH_HIP(hipMemsetAsync(p, 0, bytes, as_stream(s)));
    *dptr = p;
    return 0;
}

int64_t cnh_allocation_count(void) { return g_allocations.load(); }

int cnh_free(void* dptr) {
    if (!dptr)
        return 0;
    CNH_HIP(hipFree(dptr));
    return 0;
}

int cnh_h2d(void* dst, const void* src, size_t bytes, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    if (bytes == 0)
        return 0;
    CNH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(s)));
    CNH_HIP(hipStreamSynchronize(as_stream(s)));
    return 0;
}

int cnh_d2h(void* dst, const void* src, size_t bytes, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    if (bytes == 0)
        return 0;
    CNH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(s)));
    CNH_HIP(hipStreamSynchronize(as_stream(s)));
    return 0;
}

int cnh_d2d(void* dst, const void* src, size_t bytes, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    if (bytes == 0)
        return 0;
    CNH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(s)));
    return 0;
}

int cnh_d2h_region(int nd, int esz, void* dst_host, const int64_t* dst_strides,
                   const int64_t* dst_start, const void* src_dev, const int64_t* src_strides,
                   const int64_t* src_start, const int64_t* counts, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(nd >= 1 && nd <= CNH_MAX_ND, -2, "cnh_d2h_region: ndims %d not in 1..3", nd);
    CNH_CHECK(esz == 4 || esz == 8, -2, "cnh_d2h_region: element size %d not in {4,8}", esz);
    CNH_CHECK(dst_strides[nd - 1] == 1 && src_strides[nd - 1] == 1, -2,
              "cnh_d2h_region: innermost stride must be 1");
    for (int d = 0; d < nd; ++d)
        if (counts[d] <= 0)
            return 0;
    int64_t doff = 0, soff = 0;
    for (int d = 0; d < nd; ++d) {
        doff += dst_start[d] * dst_strides[d];
        soff += src_start[d] * src_strides[d];
    }
    char* dbase = static_cast<char*>(dst_host) + doff * esz;
    const char* sbase = static_cast<const char*>(src_dev) + soff * esz;
    hipStream_t st = as_stream(s);
    if (nd == 1) {
        CNH_HIP(hipMemcpyAsync(dbase, sbase, (size_t)counts[0] * esz, hipMemcpyDeviceToHost, st));
    } else {
        // One 2-D copy per outermost index (a single one for ndims == 2).
        int64_t planes = nd == 3 ? counts[0] : 1;
        int rd = nd - 2; // row dimension
        for (int64_t p = 0; p < planes; ++p) {
            char* dp = dbase + (nd == 3 ? p * dst_strides[0] * esz : 0);
            const char* sp = sbase + (nd == 3 ? p * src_strides[0] * esz : 0);
            CNH_HIP(hipMemcpy2DAsync(dp, (size_t)dst_strides[rd] * esz, sp,
                                     (size_t)src_strides[rd] * esz, (size_t)counts[nd - 1] * esz,
                                     (size_t)counts[rd], hipMemcpyDeviceToHost, st));
        }
    }
    CNH_HIP(hipStreamSynchronize(st));
    return 0;
}

int cnh_stream_create(cnh_stream* out) {
    if (int rc = ensure_init())
        return rc;
    hipStream_t st;
    CNH_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *out = st;
    return 0;
}

int cnh_stream_destroy(cnh_stream s) {
    if (!s)
        return 0;
    {
        // Descriptor tables whose copies were queued on this stream outlive it in the cache: let
        // the copies land and mark them complete, so that no later call waits on a dead handle.
        std::lock_guard<std::mutex> lk(g_mu);
        CNH_HIP(hipStreamSynchronize(as_stream(s)));
        DeviceState& D = dev_state();
        for (auto& kv : D.desc)
            for (DescEntry& e : kv.second)
                if (e.stream == as_stream(s))
                    e.visible = true;
        // the stream's reduction workspace goes with it
        auto it = D.ws.find(as_stream(s));
        if (it != D.ws.end()) {
            if (int rc = release_retired(it->second))
                return rc;
            if (it->second.ptr)
                CNH_HIP(hipFree(it->second.ptr));
            D.ws.erase(it);
        }
    }
    CNH_HIP(hipStreamDestroy(as_stream(s)));
    return 0;
}

int cnh_stream_sync(cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_HIP(hipStreamSynchronize(as_stream(s)));
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = dev_state().ws.find(as_stream(s));
    if (it != dev_state().ws.end())
        return release_retired(it->second);
    return 0;
}

namespace {
struct HostCb {
    void (*fn)(void*);
    void* arg;
};
void host_cb_trampoline(void* p) {
    HostCb* cb = static_cast<HostCb*>(p);
    cb->fn(cb->arg);
    delete cb;
}
} // namespace

int cnh_stream_callback(cnh_stream s, void (*fn)(void*), void* arg) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(fn != nullptr, -2, "cnh_stream_callback: null function");
    HostCb* cb = new HostCb{fn, arg};
    hipError_t e = hipLaunchHostFunc(as_stream(s), host_cb_trampoline, cb);
    if (e != hipSuccess) {
        delete cb;
        return set_error(-100, "hipLaunchHostFunc failed: %s", hipGetErrorString(e));
    }
    return 0;
}

int cnh_device_sync(void) {
    if (int rc = ensure_init())
        return rc;
    CNH_HIP(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto& kv : dev_state().ws)
        if (int rc = release_retired(kv.second))
            return rc;
    return 0;
}

int cnh_event_create(cnh_event* out) {
    if (int rc = ensure_init())
        return rc;
    hipEvent_t e;
    CNH_HIP(hipEventCreate(&e));
    *out = e;
    return 0;
}

int cnh_event_destroy(cnh_event e) {
    if (!e)
        return 0;
    CNH_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(e)));
    return 0;
}

int cnh_event_record(cnh_event e, cnh_stream s) {
    CNH_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(e), as_stream(s)));
    return 0;
}

int cnh_event_sync(cnh_event e) {
    CNH_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(e)));
    return 0;
}

int cnh_event_elapsed_ms(cnh_event a, cnh_event b, float* ms) {
    CNH_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(a), reinterpret_cast<hipEvent_t>(b)));
    return 0;
}

int cnh_scalar_to_dtype(int dtype, double s, void* out8) {
    std::memset(out8, 0, 8);
    switch (dtype) {
    case CNH_F32: {
        float v = (float)s;
        std::memcpy(out8, &v, 4);
        return 0;
    }
    case CNH_F64:
        std::memcpy(out8, &s, 8);
        return 0;
    case CNH_I32: {
        int32_t v = (int32_t)s;
        std::memcpy(out8, &v, 4);
        return 0;
    }
    case CNH_I64: {
        int64_t v = (int64_t)s;
        std::memcpy(out8, &v, 8);
        return 0;
    }
    }
    return set_error(-2, "cnh_scalar_to_dtype: unknown dtype %d", dtype);
}

} // extern "C"
