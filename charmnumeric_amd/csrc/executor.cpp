// Host executor: one object that plays upstream's ArrayDAGGroup (shape pass, decomposition, compile
// cache: src/dag_group_receive.cpp:190-575, src/dag_group_compile.cpp:6-56) and the per-partition
// executors (routing per node: src/executor_core.cpp:195-775) for every partition of every array,
// all resident on one device. Halo messages do not exist here: kernels read neighbour tiles.
#include "../../include/cnexec.h"
#include "common.h"
#include "decomp.h"
#include "stmtlog.h"

#include <dlfcn.h>

#include <algorithm>
#include <array>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <set>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

using namespace cnh;

namespace {

constexpr int kOpDelete = CNX_OP_DELETE, kOpSum = CNX_OP_SUM, kOpSumsqDiff = CNX_OP_SUMSQ_DIFF,
              kOpMaxabsDiff = CNX_OP_MAXABS_DIFF, kOpAstype = CNX_OP_ASTYPE;

struct Reader {
    const char* p;
    const char* end;
    bool ok = true;
    template <typename T> T get() {
        T v{};
        if (!ok || (size_t)(end - p) < sizeof(T)) {
            ok = false;
            return v;
        }
        std::memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        return v;
    }
};

// Region in upstream's wire form (charmnumeric.py:194-207).
bool read_region(Reader& r, cnh_region& out) {
    std::memset(&out, 0, sizeof out);
    out.is_global = r.get<int32_t>();
    if (!r.ok)
        return false;
    if (out.is_global) {
        out.is_global = 1;
        return true;
    }
    out.ndims = r.get<int32_t>();
    if (!r.ok || out.ndims < 1 || out.ndims > CNH_MAX_ND)
        return r.ok = false;
    for (int d = 0; d < out.ndims; ++d) {
        out.start[d] = r.get<int32_t>();
        out.stop[d] = r.get<int32_t>();
        out.step[d] = r.get<int32_t>();
    }
    return r.ok;
}

int region_count(const cnh_region& r, int d) {
    if (r.step[d] <= 0 || r.stop[d] <= r.start[d])
        return 0;
    return (r.stop[d] - r.start[d] + r.step[d] - 1) / r.step[d];
}

// One distributed array: ArrayMetadata (src/backend.hpp:285-288) + the per-chare Array<N,T> buffers
// (src/backend.hpp:112-200). All tiles of an array are carved from one device allocation, tile t
// row-major over its own extent; a 1-D array is therefore contiguous as a whole.
struct XArray {
    int name = 0, ndims = 1, dtype = CNH_F64, tile = 1;
    int32_t shape[3] = {1, 1, 1}, offset[3] = {0, 0, 0}, grid[3] = {1, 1, 1};
    int64_t ntiles = 1, elems = 1;
    size_t bytes = 0;
    void* slab = nullptr;
    void* alt = nullptr; // second buffer set for sweeps that read what they assign
    std::vector<int64_t> tile_off, tile_elems;
    std::vector<void*> tiles, alt_tiles;
    // Rank-3 arrays are one row-major block over the whole array and their tiles are views into it
    // (pitch = elements between consecutive indices of each dimension): every partition of the
    // array lives on this device anyway, and sweeps over the block need no tile pointers
    // (measured on MI355X, 7-point sweep on 512^3: 382 us against 407 us tile-major).
    bool flat = false;
    int64_t pitch[3] = {0, 0, 0};

    void tile_extent(int64_t t, int32_t lo[3], int32_t ext[3]) const {
        int64_t rem = t;
        for (int d = 0; d < 3; ++d) {
            lo[d] = 0;
            ext[d] = 1;
        }
        // tile g of the grid holds the elements i with (i + offset) / tile == g
        // (src/array_region.hpp:293-387)
        for (int d = ndims - 1; d >= 0; --d) {
            int g = offset[d] / tile + (int)(rem % grid[d]);
            rem /= grid[d];
            lo[d] = std::max(g * tile, (int)offset[d]) - offset[d];
            ext[d] = std::min((g + 1) * tile, (int)(offset[d] + shape[d])) - offset[d] - lo[d];
        }
    }
    // Elements between consecutive indices of each dimension inside a tile of extents `ext`.
    void tile_strides(const int32_t ext[3], int64_t stride[3]) const {
        int64_t run = 1;
        for (int d = ndims - 1; d >= 0; --d) {
            stride[d] = flat ? pitch[d] : run;
            run *= ext[d];
        }
    }
    bool phased() const {
        for (int d = 0; d < ndims; ++d)
            if (offset[d] % tile != 0)
                return true;
        return false;
    }
    cnh_tiled tiled(bool use_alt = false) const {
        cnh_tiled t;
        std::memset(&t, 0, sizeof t);
        t.ndims = ndims;
        t.tile = tile;
        for (int d = 0; d < ndims; ++d) {
            t.offset[d] = offset[d];
            t.shape[d] = shape[d];
            t.grid_lo[d] = offset[d] / tile;
            t.grid[d] = grid[d];
        }
        t.tiles = use_alt ? alt_tiles.data() : tiles.data();
        if (flat)
            for (int d = 0; d < ndims; ++d)
                t.pitch[d] = pitch[d];
        return t;
    }
};

} // namespace

struct cnx_executor {
    bool dry = false; // no device: every decision is taken and traced, nothing is launched
    int num_pes = 1, odf = 4;
    int min_tile[4] = {0, 262144, 512, 64}; // CT_MIN_TILE_1D/2D/3D, src/backend.hpp:10-18
    bool flat3 = true;  // new rank-3 arrays are one row-major block with tiles as views into it
    bool fuse_on = true; // runs of assignments of one extent go out as one launch
    // A run of mergeable assignments that reaches the end of a message waits here for the next
    // message (where it may go on) or for the next call that needs the executor's state: what gets
    // merged then depends on the statements alone, not on where the frontend happened to cut its
    // messages, and a time loop keeps meeting the same few merged kernels.
    std::vector<DagNode> held;
    bool final_pass = false;   // running held nodes to the end: nothing may be held again
    cnh_stream stream = nullptr;
    std::map<int, XArray> arrays;
    // compile_cache (src/dag_group_compile.cpp:43-56), bounded: a time loop over slabs makes a new
    // group (same code, other regions) per step, and the oldest ones are let go
    std::unordered_map<uint64_t, cnh_kernel*> kernels;
    std::vector<uint64_t> kernel_order;
    size_t kernel_next_evict = 0;
    size_t max_kernels = 4096;
    std::map<size_t, std::vector<void*>> free_list;    // src/backend.hpp:366-545
    int64_t stats[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    bool trace_on = false;
    std::string trace;
    // Decomposition planning (off: tile rule and offset 0 for every array). When on, every DAG
    // message is planned as a whole before its first node runs and new arrays are laid out with
    // the tile and offset the plan gives them.
    bool solver_on = false;
    struct Planned {
        int ndims = 0, tile = 0;
        int32_t shape[3] = {1, 1, 1}, offset[3] = {0, 0, 0};
    };
    std::map<int, Planned> planned;
    int next_tmp = -(1 << 30); // names of relayout copies
    uintptr_t fake_ptr = 0x1000;
    // Asynchronous mode: DAG messages queue up for a thread of the executor's own, as upstream's
    // frontend hands them to a server and goes on recording. Every other entry point waits for
    // the queue first; an error of a queued message is reported by the next call on the executor.
    int device = 0;
    bool async_on = false, busy = false, stop = false;
    std::thread worker;
    std::mutex qmu;
    std::condition_variable qcv, idle_cv;
    struct Queued {
        std::vector<char> bytes;
        bool is_log = false;   // a statement log (to be planned first) rather than a DAG message
        int window = -1;
    };
    std::deque<Queued> queue;
    // Statement log: what an automatic flush held back waits here, as parsed records, for the
    // next stretch of the log. Names above every array name for the SET_REGION roots the planner
    // makes. With capture on, every planned message is also kept as bytes (tests compare them).
    std::vector<stmtlog::Instr> plog;
    int32_t next_set_name = 1 << 30;
    bool capture_on = false;
    std::vector<char> captured;
    int deferred_rc = 0;
    std::string deferred_msg;
    // One-element arrays whose value still stands as partial sums in a buffer of their own (what a
    // launch with a reducing root, or a matvec that took the dot along, left behind). The next
    // launch that reads such an array as a kernel scalar sums the partials itself and stores the
    // value; anything else that needs it gets a fold launch first (resolve_pending). They exist
    // only between the nodes of one run_nodes pass or while nodes are held.
    struct PendingSum {
        void* partials = nullptr;
        size_t bytes = 0;
        int64_t count = 0;
    };
    std::map<int, PendingSum> pending;
    // Measurement: with timing on, every matvec launch sits between two events on the stream.
    bool time_matvec = false;
    std::vector<std::pair<cnh_event, cnh_event>> matvec_events;

    void log(const std::string& s) {
        if (trace_on) {
            trace += s;
            trace += '\n';
        }
    }
};

namespace {

using Ex = cnx_executor;

std::string shape_str(const int32_t* s, int nd) {
    std::ostringstream o;
    o << "(";
    for (int d = 0; d < nd; ++d)
        o << (d ? "," : "") << s[d];
    o << ")";
    return o.str();
}

int slab_alloc(Ex* ex, size_t bytes, bool zero, void** out) {
    auto it = ex->free_list.find(bytes);
    if (it != ex->free_list.end() && !it->second.empty()) {
        *out = it->second.back();
        it->second.pop_back();
        ex->stats[4]++;
        // Reused buffers are cleared like new ones (src/backend.hpp:490-497).
        if (zero && !ex->dry)
            if (int rc = cnh_memset0(*out, bytes, ex->stream))
                return rc;
        return 0;
    }
    ex->stats[3]++;
    ex->stats[7] += (int64_t)bytes;
    if (ex->dry) {
        *out = reinterpret_cast<void*>(ex->fake_ptr);
        ex->fake_ptr += (bytes + 255) & ~(size_t)255;
        return 0;
    }
    // cleared on the executor's own stream, in order with whatever writes the array next
    if (int rc = cnh_alloc(bytes, 0, out))
        return rc;
    return zero ? cnh_memset0(*out, bytes, ex->stream) : 0;
}

void slab_release(Ex* ex, size_t bytes, void* p) {
    if (p)
        ex->free_list[bytes].push_back(p);
}

// Tile edge: the minimum tile of the rank, doubled until the array has at most odf*PEs tiles
// (src/decomposition_solver.hpp:100-122). Offsets are 0 for every array created here.
int tile_rule(const Ex* ex, int ndims, const int32_t* shape) {
    int64_t max_tiles = (int64_t)std::max(1, ex->odf) * std::max(1, ex->num_pes);
    int64_t tile = 1;
    while (tile < ex->min_tile[ndims])
        tile *= 2;
    tile = std::max<int64_t>(tile, ex->min_tile[ndims]);
    for (;;) {
        int64_t count = 1;
        for (int d = 0; d < ndims; ++d)
            count *= (shape[d] + tile - 1) / tile;
        if (count <= max_tiles || tile > (1 << 30))
            break;
        tile *= 2;
    }
    return (int)tile;
}

// Storage form of a new array. Rank 3: one row-major block whenever blocks are allowed (flat3).
// Rank 2: a buffer per tile, except where tiles would not help the kernels anyway: rows of odd
// length (128-bit accesses cannot stay inside tiles then) and ragged tile grids (a 4097 x 4097
// array cut at 4096 has tiles of one row and one column). Those are one block too, and their
// sweeps run the whole-array kernels.
bool flat_rule(const Ex* ex, int nd, const int32_t* shape, int tile, const int32_t* offset) {
    if (nd == 3)
        return ex->flat3;
    if (nd != 2 || !ex->flat3)
        return false;
    if (shape[1] % 2 != 0)
        return true;
    for (int d = 0; d < 2; ++d) {
        const int off = offset ? offset[d] : 0;
        const int glo = off / tile, ghi = (off + shape[d] + tile - 1) / tile;
        if (ghi - glo > 1 && ((off + shape[d]) % tile != 0 || off % tile != 0))
            return true;
    }
    return false;
}

int make_array(Ex* ex, int name, int ndims, int dtype, const int32_t* shape, bool zero, XArray** out) {
    CNH_CHECK(ndims >= 1 && ndims <= 3, -20, "array %d: unsupported rank %d", name, ndims);
    CNH_CHECK(dtype_size(dtype) != 0, -20, "array %d: unknown dtype %d", name, dtype);
    CNH_CHECK(ex->arrays.find(name) == ex->arrays.end(), -21, "array %d already exists", name);
    XArray a;
    a.name = name;
    a.ndims = ndims;
    a.dtype = dtype;
    a.elems = 1;
    for (int d = 0; d < ndims; ++d) {
        CNH_CHECK(shape[d] >= 1, -20, "array %d: extent %d in dim %d", name, shape[d], d);
        a.shape[d] = shape[d];
        a.elems *= shape[d];
    }
    a.tile = tile_rule(ex, ndims, shape);
    auto plan = ex->planned.find(name);
    if (plan != ex->planned.end()) {
        const auto& p = plan->second;
        bool fits = p.ndims == ndims && p.tile > 0 && (p.tile & (p.tile - 1)) == 0;
        for (int d = 0; d < ndims && fits; ++d)
            fits = p.shape[d] == shape[d] && p.offset[d] >= 0;
        if (fits) {
            a.tile = p.tile;
            for (int d = 0; d < ndims; ++d)
                a.offset[d] = p.offset[d];
        } else {
            if (ex->trace_on) ex->log("plan for " + std::to_string(name) + " does not fit the array; tile rule used");
        }
        ex->planned.erase(plan);
    }
    a.ntiles = 1;
    for (int d = 0; d < ndims; ++d) {
        a.grid[d] = (a.offset[d] + a.shape[d] + a.tile - 1) / a.tile - a.offset[d] / a.tile;
        a.ntiles *= a.grid[d];
    }
    const int esz = dtype_size(dtype);
    int64_t off = 0;
    a.flat = flat_rule(ex, ndims, a.shape, a.tile, a.offset);
    if (a.flat && ndims == 2) {
        a.pitch[1] = 1;
        a.pitch[0] = a.shape[1];
        for (int64_t t = 0; t < a.ntiles; ++t) {
            int32_t lo[3], ext[3];
            a.tile_extent(t, lo, ext);
            a.tile_off.push_back((lo[0] * a.pitch[0] + lo[1]) * esz);
            a.tile_elems.push_back((int64_t)ext[0] * ext[1]);
        }
        off = a.elems * esz;
    } else if (a.flat) {
        a.pitch[2] = 1;
        a.pitch[1] = a.shape[2];
        a.pitch[0] = (int64_t)a.shape[1] * a.shape[2];
        for (int64_t t = 0; t < a.ntiles; ++t) {
            int32_t lo[3], ext[3];
            a.tile_extent(t, lo, ext);
            a.tile_off.push_back((lo[0] * a.pitch[0] + lo[1] * a.pitch[1] + lo[2]) * esz);
            a.tile_elems.push_back((int64_t)ext[0] * ext[1] * ext[2]);
        }
        off = a.elems * esz;
    }
    for (int64_t t = 0; t < a.ntiles && !a.flat; ++t) {
        int32_t lo[3], ext[3];
        a.tile_extent(t, lo, ext);
        int64_t n = (int64_t)ext[0] * ext[1] * ext[2];
        a.tile_off.push_back(off);
        a.tile_elems.push_back(n);
        off += n * esz;
        if (ndims > 1)
            off = (off + 255) & ~(int64_t)255;
        // Equal power-of-two tiles of rank 3 back to back put the same position of every tile on
        // the same memory channels, and sweeps walk all tiles in step: measured on MI355X, 64
        // tiles of 128^3 doubles sweep 8 % faster when consecutive tiles start 2 MiB + 256 B
        // further apart (rank 2 tiles of 2048^2 are best back to back).
        if (ndims == 3 && n * esz >= (2 << 20))
            off += (2 << 20) + 256;
    }
    a.bytes = (size_t)std::max<int64_t>((off + 255) & ~(int64_t)255, 256);
    if (int rc = slab_alloc(ex, a.bytes, zero, &a.slab))
        return rc;
    for (int64_t t = 0; t < a.ntiles; ++t)
        a.tiles.push_back(static_cast<char*>(a.slab) + a.tile_off[t]);
    if (ex->trace_on) ex->log("create " + std::to_string(name) + " shape=" + shape_str(a.shape, ndims) + " dtype=" +
            std::to_string(dtype) + " tile=" + std::to_string(a.tile) + " tiles=" +
            std::to_string(a.ntiles) + (a.phased() || a.offset[0] || a.offset[1] || a.offset[2]
                                            ? " offset=" + shape_str(a.offset, ndims)
                                            : std::string()));
    auto ins = ex->arrays.emplace(name, std::move(a));
    ex->stats[6] = (int64_t)ex->arrays.size();
    if (out)
        *out = &ins.first->second;
    return 0;
}

int make_block(Ex* ex, XArray& a);

int ensure_alt(Ex* ex, XArray& a) {
    if (a.alt)
        return 0;
    if (int rc = slab_alloc(ex, a.bytes, false, &a.alt))
        return rc;
    a.alt_tiles.clear();
    for (int64_t t = 0; t < a.ntiles; ++t)
        a.alt_tiles.push_back(static_cast<char*>(a.alt) + a.tile_off[t]);
    return 0;
}

void drop_array(Ex* ex, int name) {
    auto it = ex->arrays.find(name);
    if (it == ex->arrays.end())
        return;
    auto pend = ex->pending.find(name);
    if (pend != ex->pending.end()) {            // nobody asked for the value: no fold needed
        slab_release(ex, pend->second.bytes, pend->second.partials);
        ex->pending.erase(pend);
    }
    slab_release(ex, it->second.bytes, it->second.slab);
    slab_release(ex, it->second.bytes, it->second.alt);
    ex->arrays.erase(it);
    ex->stats[6] = (int64_t)ex->arrays.size();
    if (ex->trace_on) ex->log("delete " + std::to_string(name));
}

int find_array(Ex* ex, int name, XArray** out, const char* what) {
    auto it = ex->arrays.find(name);
    CNH_CHECK(it != ex->arrays.end(), -22, "%s: array %d does not exist", what, name);
    *out = &it->second;
    return 0;
}

bool same_decomposition(const XArray& a, const XArray& b) {
    if (a.ndims != b.ndims || a.tile != b.tile || a.flat != b.flat)
        return false;
    // equal extents, tile edges and phases give the same tiles, wherever the grids start
    for (int d = 0; d < a.ndims; ++d)
        if (a.shape[d] != b.shape[d] || a.offset[d] % a.tile != b.offset[d] % b.tile)
            return false;
    return true;
}

bool region_is_whole(const cnh_region& r, const XArray& a) {
    if (r.is_global)
        return true;
    if (r.ndims != a.ndims)
        return false;
    for (int d = 0; d < a.ndims; ++d)
        if (r.start[d] != 0 || r.stop[d] != a.shape[d] || r.step[d] != 1)
            return false;
    return true;
}

bool same_region(const cnh_region& a, const cnh_region& b) {
    if (a.is_global != b.is_global)
        return false;
    if (a.is_global)
        return true;
    if (a.ndims != b.ndims)
        return false;
    for (int d = 0; d < a.ndims; ++d)
        if (a.start[d] != b.start[d] || a.stop[d] != b.stop[d] || a.step[d] != b.step[d])
            return false;
    return true;
}

// The compile cache's key: 8 bytes per step (multiply, fold the high half back), the rest byte by
// byte. A key that collides only costs a comparison of the groups themselves (compile_cached).
uint64_t mix_words(const void* data, size_t n, uint64_t h = 0x9E3779B97F4A7C15ull) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    for (; n >= 8; n -= 8, p += 8) {
        uint64_t w;
        std::memcpy(&w, p, 8);
        h = (h ^ w) * 0xD6E8FEB86659FD93ull;
        h ^= h >> 32;
    }
    for (; n > 0; --n, ++p) {
        h = (h ^ *p) * 0x100000001B3ull;
        h ^= h >> 29;
    }
    return h;
}

// ---- node kinds ----

int exec_create(Ex* ex, const cnh_ast_node& n) {
    CNH_CHECK(!n.region.is_global && n.region.ndims == n.ndims, -23,
              "CREATE %d carries no shape", n.result_name);
    int32_t shape[3] = {1, 1, 1};
    for (int d = 0; d < n.ndims; ++d)
        shape[d] = region_count(n.region, d);
    return make_array(ex, n.result_name, n.ndims, n.dtype, shape, true, nullptr);
}

// SET_REGION with a scalar value: one strided fill per tile the region touches
// (src/executor_ast_visitor.cpp:112-147).
int exec_fill(Ex* ex, XArray& a, const cnh_region& reg, double value) {
    cnh_region r = reg;
    if (r.is_global) {
        r.ndims = a.ndims;
        for (int d = 0; d < a.ndims; ++d) {
            r.start[d] = 0;
            r.stop[d] = a.shape[d];
            r.step[d] = 1;
        }
    }
    CNH_CHECK(r.ndims == a.ndims, -24, "fill of array %d: region rank %d, array rank %d", a.name,
              r.ndims, a.ndims);
    for (int d = 0; d < a.ndims; ++d)
        CNH_CHECK(r.step[d] >= 1 && r.start[d] >= 0 && r.stop[d] <= a.shape[d], -24,
                  "fill of array %d: region [%d:%d:%d] leaves extent %d in dim %d", a.name,
                  r.start[d], r.stop[d], r.step[d], a.shape[d], d);
    unsigned char s8[8];
    if (int rc = cnh_scalar_to_dtype(a.dtype, value, s8))
        return rc;
    const int esz = dtype_size(a.dtype);
    int launches = 0;
    for (int64_t t = 0; t < a.ntiles; ++t) {
        int32_t lo[3], ext[3];
        a.tile_extent(t, lo, ext);
        int64_t start[3], step[3], counts[3], strides[3];
        bool empty = false;
        a.tile_strides(ext, strides);
        for (int d = 0; d < a.ndims; ++d) {
            int64_t first = r.start[d];
            if (first < lo[d])
                first += ((lo[d] - first + r.step[d] - 1) / r.step[d]) * (int64_t)r.step[d];
            int64_t last_excl = std::min<int64_t>(r.stop[d], lo[d] + ext[d]);
            if (first >= last_excl) {
                empty = true;
                break;
            }
            start[d] = first - lo[d];
            step[d] = r.step[d];
            counts[d] = (last_excl - first + r.step[d] - 1) / r.step[d];
        }
        if (empty)
            continue;
        ++launches;
        if (!ex->dry)
            if (int rc = cnh_fill_region(a.ndims, esz, a.tiles[t], strides, start, step, counts, s8,
                                         ex->stream))
                return rc;
    }
    if (ex->trace_on) ex->log("fill " + std::to_string(a.name) + " tiles_touched=" + std::to_string(launches));
    return 0;
}

struct Group {
    std::vector<cnh_ast_node> nodes; // canonical names
    std::vector<int32_t> roots;
    std::vector<int> canon_to_actual;   // indexed by canonical name (1, 2, ...)
    int dtype = CNH_F64;
    int ndims = 1;
    uint64_t key = 0;
};

// Renames arrays, temporaries and literals by first appearance so that structurally identical
// groups (every CG iteration, every sweep) share one compiled kernel whatever their array names.
void canonicalise(const DagNode& n, Group& g) {
    g.nodes = n.nodes;
    g.roots = n.roots;
    // a group has a few dozen names at most: a flat list searched from the back (the operand
    // just produced is the likeliest match) beats a tree of allocated nodes
    g.canon_to_actual.assign(1, 0);
    g.canon_to_actual.reserve(g.nodes.size() + 1);
    for (auto& a : g.nodes) {
        int canon = 0;
        for (int c = (int)g.canon_to_actual.size() - 1; c >= 1; --c)
            if (g.canon_to_actual[(size_t)c] == a.result_name) {
                canon = c;
                break;
            }
        if (canon == 0) {
            canon = (int)g.canon_to_actual.size();
            g.canon_to_actual.push_back(a.result_name);
        }
        a.result_name = a.is_scalar ? -canon : canon;
    }
    // Element type of the kernel: the first root that is not F32 decides (src/jit.cpp:50-69).
    g.dtype = CNH_F32;
    for (int32_t r : g.roots)
        if (g.nodes[r].dtype != CNH_F32) {
            g.dtype = g.nodes[r].dtype;
            break;
        }
    g.ndims = g.nodes[g.roots.back()].ndims;
    uint64_t h = mix_words(&g.dtype, sizeof g.dtype);
    h = mix_words(&g.ndims, sizeof g.ndims, h);
    for (auto& a : g.nodes) {
        // hash field by field: the struct has padding
        int32_t head[10] = {a.result_name, a.opcode, a.is_temp, a.is_scalar, a.is_broadcast,
                            a.ndims, a.dtype, a.n_operands, a.operands[0], a.operands[1]};
        h = mix_words(head, sizeof head, h);
        h = mix_words(&a.scalar, sizeof a.scalar, h);
        h = mix_words(a.has_operand_region, sizeof a.has_operand_region, h);
        h = mix_words(&a.operand_regions[0], sizeof(cnh_region), h);
        h = mix_words(&a.operand_regions[1], sizeof(cnh_region), h);
        h = mix_words(&a.region, sizeof(cnh_region), h);
    }
    h = mix_words(g.roots.data(), g.roots.size() * sizeof(int32_t), h);
    g.key = h;
}

int compile_cached(Ex* ex, Group& g, cnh_kernel** out) {
    cnh_ast ast{(int32_t)g.nodes.size(), (int32_t)g.roots.size(), g.nodes.data(), g.roots.data()};
    // the key is a hash: a hit counts only when the kernel was compiled from this very group;
    // another group under the same key moves on to the next key of a fixed sequence
    for (auto it = ex->kernels.find(g.key); it != ex->kernels.end(); it = ex->kernels.find(g.key)) {
        if (cnh_kernel_matches(it->second, &ast, g.dtype, g.ndims)) {
            ex->stats[1]++;
            *out = it->second;
            return 0;
        }
        g.key = g.key * 6364136223846793005ull + 1442695040888963407ull;
        if (g.key == 0)
            g.key = 1;
    }
    cnh_kernel* k = nullptr;
    if (int rc = cnh_compile_group(&ast, g.dtype, g.ndims, g.key, &k))
        return rc;
    ex->stats[0]++;
    if (ex->kernel_order.size() < ex->max_kernels) {
        ex->kernel_order.push_back(g.key);
    } else { // ring: replace the oldest entry
        const uint64_t old = ex->kernel_order[ex->kernel_next_evict];
        auto victim = ex->kernels.find(old);
        if (victim != ex->kernels.end()) {
            cnh_kernel_release(victim->second);
            ex->kernels.erase(victim);
        }
        ex->kernel_order[ex->kernel_next_evict] = g.key;
        ex->kernel_next_evict = (ex->kernel_next_evict + 1) % ex->max_kernels;
    }
    ex->kernels[g.key] = k;
    *out = k;
    return 0;
}

// Shape of a new elementwise result: the root's own region when the message carries one, else the
// shape of an operand region, else the shape of a non-broadcast operand array
// (src/dag_group_receive.cpp:65-106).
int result_shape(Ex* ex, const DagNode& n, const cnh_ast_node& root, int32_t shape[3]) {
    shape[0] = shape[1] = shape[2] = 1;
    if (!root.region.is_global && root.region.ndims == root.ndims) {
        for (int d = 0; d < root.ndims; ++d)
            shape[d] = region_count(root.region, d);
        return 0;
    }
    bool found = false;
    for (const auto& a : n.nodes) {
        if (a.is_scalar || a.opcode == CNH_OP_NOOP)
            continue;
        for (int i = 0; i < a.n_operands; ++i) {
            const cnh_ast_node& op = n.nodes[a.operands[i]];
            if (op.is_scalar || op.opcode != CNH_OP_NOOP)
                continue;
            if (a.has_operand_region[i] && !a.operand_regions[i].is_global) {
                for (int d = 0; d < op.ndims; ++d)
                    shape[d] = region_count(a.operand_regions[i], d);
                return 0;
            }
            auto it = ex->arrays.find(op.result_name);
            if (it == ex->arrays.end())
                continue;
            if (!found || !op.is_broadcast) {
                for (int d = 0; d < 3; ++d)
                    shape[d] = d < it->second.ndims ? it->second.shape[d] : 1;
                found = true;
                if (!op.is_broadcast)
                    return 0;
            }
        }
    }
    CNH_CHECK(found, -25, "cannot infer the shape of result %d", root.result_name);
    return 0;
}

// True when {s0 + i*t0 < e0} and {s1 + j*t1 < e1} have no common element.
bool progressions_disjoint(int64_t s0, int64_t e0, int64_t t0, int64_t s1, int64_t e1, int64_t t1) {
    if (t0 < 1)
        t0 = 1;
    if (t1 < 1)
        t1 = 1;
    if (s0 >= e0 || s1 >= e1)
        return true;
    const int64_t last0 = s0 + (e0 - 1 - s0) / t0 * t0, last1 = s1 + (e1 - 1 - s1) / t1 * t1;
    if (last0 < s1 || last1 < s0)
        return true;
    int64_t g = t0, h = t1;
    while (h) {
        const int64_t r = g % h;
        g = h;
        h = r;
    }
    if ((s1 - s0) % g != 0)
        return true;
    // a common element exists modulo lcm; walk the progression that starts later, at most
    // t_other / g steps, and see whether one falls inside both ranges
    const int64_t hi = std::min(last0, last1);
    int64_t x = std::max(s0, s1), tx, so, to;
    if (s0 >= s1) {
        tx = t0, so = s1, to = t1;
    } else {
        tx = t1, so = s0, to = t0;
    }
    for (int64_t n = 0; n <= to / g && x <= hi; ++n, x += tx)
        if ((x - so) % to == 0)
            return false;
    return true;
}

int exec_group(Ex* ex, const DagNode& n) {
    const cnh_ast_node& root = n.nodes[n.roots.back()];
    for (size_t i = 0; i + 1 < n.roots.size(); ++i)
        CNH_CHECK(n.nodes[n.roots[i]].is_temp, -26,
                  "node %d: only the last root of a group may be a result", n.id);

    // SET_REGION with a literal: fill.
    if (root.opcode == CNH_OP_SET_REGION && root.n_operands == 2 &&
        n.nodes[root.operands[1]].is_scalar) {
        XArray* target;
        if (int rc = find_array(ex, n.nodes[root.operands[0]].result_name, &target, "SET_REGION"))
            return rc;
        return exec_fill(ex, *target, root.region, n.nodes[root.operands[1]].scalar);
    }

    Group g;
    canonicalise(n, g);
    cnh_kernel* k = nullptr;
    if (int rc = compile_cached(ex, g, &k))
        return rc;
    int n_in = 0, n_scalar = 0, n_out = 0;
    if (int rc = cnh_kernel_signature(k, &n_in, &n_scalar, &n_out))
        return rc;
    CNH_CHECK(n_out == 1, -26, "node %d: %d outputs (one expected)", n.id, n_out);

    // Bind arguments by name.
    std::vector<XArray*> in_arr(n_in);
    std::vector<cnh_region> in_reg(n_in);
    std::vector<int> in_has_reg(n_in);
    for (int i = 0; i < n_in; ++i) {
        int cname = 0;
        if (int rc = cnh_kernel_input(k, i, &cname, &in_has_reg[i], &in_reg[i]))
            return rc;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &in_arr[i], "group input"))
            return rc;
        CNH_CHECK(in_arr[i]->dtype == g.dtype, -27,
                  "node %d: input array %d has dtype %d, the group computes in dtype %d", n.id,
                  in_arr[i]->name, in_arr[i]->dtype, g.dtype);
    }
    std::vector<const void*> scalars(n_scalar ? n_scalar : 1, nullptr);
    for (int i = 0; i < n_scalar; ++i) {
        int cname = 0;
        if (int rc = cnh_kernel_scalar(k, i, &cname))
            return rc;
        XArray* s;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &s, "broadcast scalar"))
            return rc;
        CNH_CHECK(s->elems == 1, -27, "node %d: broadcast operand %d has %lld elements", n.id,
                  s->name, (long long)s->elems);
        CNH_CHECK(s->dtype == g.dtype, -27, "node %d: broadcast operand %d has dtype %d, group %d",
                  n.id, s->name, s->dtype, g.dtype);
        scalars[i] = s->tiles[0];
    }

    const bool is_set = root.opcode == CNH_OP_SET_REGION;
    XArray* target = nullptr;
    if (is_set) {
        if (int rc = find_array(ex, n.nodes[root.operands[0]].result_name, &target, "SET_REGION"))
            return rc;
        CNH_CHECK(target->dtype == g.dtype, -27, "node %d: target dtype %d, group dtype %d", n.id,
                  target->dtype, g.dtype);
    } else {
        int32_t shape[3];
        if (int rc = result_shape(ex, n, root, shape))
            return rc;
        if (int rc = make_array(ex, root.result_name, root.ndims, g.dtype, shape, false, &target))
            return rc;
        // make_array may rehash nothing (std::map), input pointers stay valid.
    }

    // Dense path: no shifted or strided operand, everything on one decomposition
    // (the no-region fast path, src/execute_node.cpp:1263-1336).
    bool dense = !is_set || region_is_whole(root.region, *target);
    for (int i = 0; i < n_in && dense; ++i) {
        if (in_has_reg[i] && !region_is_whole(in_reg[i], *in_arr[i]))
            dense = false;
        if (!same_decomposition(*in_arr[i], *target))
            dense = false;
    }
    ex->stats[5]++;
    if (dense) {
        const int nd = target->ndims;
        // an array stored as one block is a single dense run, whatever its partitions
        const int64_t parts = target->flat ? 1 : target->ntiles;
        std::vector<cnh_memref> in(std::max<size_t>(1, (size_t)parts * n_in)), out((size_t)parts);
        for (int64_t t = 0; t < parts; ++t) {
            int32_t lo[3], ext[3];
            target->tile_extent(t, lo, ext);
            if (target->flat)
                for (int d = 0; d < nd; ++d)
                    ext[d] = target->shape[d];
            auto fill = [&](cnh_memref& m, void* ptr) {
                std::memset(&m, 0, sizeof m);
                m.allocated = m.aligned = ptr;
                int64_t stride = 1;
                for (int d = nd - 1; d >= 0; --d) {
                    m.sizes[d] = ext[d];
                    m.strides[d] = stride;
                    stride *= ext[d];
                }
            };
            for (int i = 0; i < n_in; ++i)
                fill(in[(size_t)t * n_in + i], in_arr[i]->tiles[t]);
            fill(out[(size_t)t], target->tiles[t]);
        }
        if (ex->trace_on) ex->log("group node=" + std::to_string(n.id) + " path=dense parts=" + std::to_string(parts) +
                " inputs=" + std::to_string(n_in) + " scalars=" + std::to_string(n_scalar) +
                " out=" + std::to_string(target->name));
        if (ex->dry)
            return 0;
        return cnh_launch_group_batched(k, nd, (int)parts, n_in, in.data(), n_scalar, scalars.data(),
                                        1, 1, out.data(), ex->stream);
    }

    // Shifted / strided operands or mixed decompositions: one launch over the target's tiles that
    // reads whatever tiles the operand regions fall into (replaces the fragment path and its halo
    // messages, src/execute_node.cpp:1338-1585, src/executor_core.cpp:8-143).
    // Reading the target through another region is a hazard only where that region can meet the
    // assigned one. Two regions share no point when their index progressions miss each other in
    // some dimension: other slabs (C[t] = f(C[t-1])), or the other colour of a red-black update
    // (phi[1:-1:2, ...] = f(phi[0:-2:2, ...])). Those run in place.
    bool aliased = false;
    if (is_set)
        for (int i = 0; i < n_in; ++i)
            if (in_arr[i] == target) {
                cnh_region whole;
                std::memset(&whole, 0, sizeof whole);
                whole.is_global = 1;
                const cnh_region& ir = in_has_reg[i] ? in_reg[i] : whole;
                bool same = same_region(ir, root.region) ||
                            (region_is_whole(ir, *target) && region_is_whole(root.region, *target));
                if (same)
                    continue;
                bool disjoint = false;
                if (!ir.is_global && !root.region.is_global)
                    for (int d = 0; d < target->ndims; ++d)
                        if (progressions_disjoint(ir.start[d], ir.stop[d], ir.step[d], root.region.start[d],
                                                  root.region.stop[d], root.region.step[d]))
                            disjoint = true;
                if (!disjoint)
                    aliased = true;
            }
    if (aliased)
        if (int rc = ensure_alt(ex, *target))
            return rc;
    std::vector<cnh_tiled> tin(std::max(1, n_in));
    for (int i = 0; i < n_in; ++i) {
        tin[i] = in_arr[i]->tiled();
        if (in_arr[i]->ndims < target->ndims) {
            // A lower-rank operand assigned into a higher-rank region (IFOG[t] = M with M 2-D):
            // present it with extent-1 dimensions inserted where the assigned region has them.
            // A row-major tile (e0, e1) is the same memory as (1, e0, e1) or (e0, 1, e1).
            CNH_CHECK(is_set && !root.region.is_global && !in_has_reg[i], -35,
                      "node %d: operand %d has rank %d in a rank-%d group", n.id, in_arr[i]->name,
                      in_arr[i]->ndims, target->ndims);
            const XArray& a = *in_arr[i];
            cnh_tiled t;
            std::memset(&t, 0, sizeof t);
            t.ndims = target->ndims;
            t.tile = a.tile;
            t.tiles = a.tiles.data();
            int j = 0;
            int from[3] = {-1, -1, -1};          // the operand's dimension behind each of the group's
            for (int d = 0; d < target->ndims; ++d) {
                const int cnt = region_count(root.region, d);
                const int left_t = target->ndims - d, left_a = a.ndims - j;
                if (j < a.ndims && a.shape[j] == cnt && !(cnt == 1 && left_t > left_a)) {
                    t.shape[d] = a.shape[j];
                    t.grid[d] = a.grid[j];
                    t.offset[d] = a.offset[j];
                    t.grid_lo[d] = a.offset[j] / a.tile;
                    from[d] = j;
                    ++j;
                } else {
                    CNH_CHECK(cnt == 1, -35, "node %d: operand %d of shape rank %d does not fit the "
                              "assigned region", n.id, a.name, a.ndims);
                    t.shape[d] = 1;
                    t.grid[d] = 1;
                }
            }
            CNH_CHECK(j == a.ndims, -35, "node %d: operand %d does not fit the assigned region", n.id,
                      a.name);
            if (a.flat)
                // one block: an inserted dimension has one index, so any pitch that keeps the
                // pitches ordered serves; it takes the extent of what lies below it
                for (int d = target->ndims - 1; d >= 0; --d)
                    t.pitch[d] = from[d] >= 0                ? a.pitch[from[d]]
                                 : d == target->ndims - 1 ? 1
                                                          : t.pitch[d + 1] * t.shape[d + 1];
            tin[i] = t;
        } else if (in_arr[i]->ndims > target->ndims) {
            // A higher-rank operand whose extra dimensions have extent 1 (vec[:] = column with
            // column of shape (N, 1), charmnumeric.py:528-531 upstream): drop them. A row-major
            // tile (e0, 1) is the same memory as (e0).
            CNH_CHECK(!in_has_reg[i], -35, "node %d: operand %d has rank %d in a rank-%d group", n.id,
                      in_arr[i]->name, in_arr[i]->ndims, target->ndims);
            const XArray& a = *in_arr[i];
            cnh_tiled t;
            std::memset(&t, 0, sizeof t);
            t.ndims = target->ndims;
            t.tile = a.tile;
            t.tiles = a.tiles.data();
            int j = 0;
            for (int d = 0; d < a.ndims; ++d) {
                if (a.shape[d] == 1 && a.ndims - d > target->ndims - j)
                    continue; // dropped
                CNH_CHECK(j < target->ndims, -35, "node %d: operand %d of shape rank %d does not fit a "
                          "rank-%d target", n.id, a.name, a.ndims, target->ndims);
                t.shape[j] = a.shape[d];
                t.grid[j] = a.grid[d];
                t.offset[j] = a.offset[d];
                t.grid_lo[j] = a.offset[d] / a.tile;
                if (a.flat)
                    t.pitch[j] = a.pitch[d];
                ++j;
            }
            CNH_CHECK(j == target->ndims, -35, "node %d: operand %d does not reduce to rank %d", n.id,
                      a.name, target->ndims);
            // views into a block: the last kept dimension must be the one with unit pitch
            CNH_CHECK(!a.flat || t.pitch[target->ndims - 1] == 1, -35,
                      "node %d: the last dimension of operand %d is dropped", n.id, a.name);
            tin[i] = t;
        } else {
            CNH_CHECK(in_arr[i]->ndims == target->ndims, -35,
                      "node %d: operand %d has rank %d in a rank-%d group", n.id, in_arr[i]->name,
                      in_arr[i]->ndims, target->ndims);
        }
    }
    cnh_tiled cur = target->tiled(false);
    cnh_tiled dst = aliased ? target->tiled(true) : cur;
    if (!ex->dry)
        if (int rc = cnh_launch_group_tiles(k, n_in, tin.data(), n_scalar, scalars.data(), 1,
                                            is_set ? &cur : nullptr, &dst, ex->stream))
            return rc;
    // which kernels this group has used so far: the register-window or sliding-window stencil
    // kernels, or the general gather
    const char* used = ex->dry ? "" : cnh_kernel_variants_loaded(k, "direct") > 0 ? " kernel=direct"
                                  : cnh_kernel_variants_loaded(k, "slide") > 0  ? " kernel=slide"
                                                                                : " kernel=gather";
    if (ex->trace_on) ex->log("group node=" + std::to_string(n.id) + " path=tiles inputs=" + std::to_string(n_in) +
            " scalars=" + std::to_string(n_scalar) + " out=" + std::to_string(target->name) +
            (aliased ? " pingpong" : " inplace") + used);
    if (aliased) {
        std::swap(target->slab, target->alt);
        std::swap(target->tiles, target->alt_tiles);
    }
    // A statement that took the gather over tile tables (strides, two shifted arrays, anything the
    // stencil kernels refuse) runs 1.7-1.8 times faster over arrays stored as one block each
    // (restriction 8192^2 -> 4096^2: 268 against 150 us). Statements come in loops: lay the large
    // rank-2 arrays of this one out anew now, once, and its next occurrence takes that route.
    if (!ex->dry && ex->flat3 && !ex->solver_on && std::strcmp(used, " kernel=gather") == 0 && target->ndims == 2) {
        std::vector<XArray*> involved{target};
        involved.insert(involved.end(), in_arr.begin(), in_arr.begin() + n_in);
        for (XArray* a : involved)
            if (a->ndims == 2 && !a->flat && a->ntiles > 1 && !a->phased() && a->elems >= (1ll << 20))
                if (int rc = make_block(ex, *a))
                    return rc;
    }
    return 0;
}

int leaf_array(Ex* ex, const DagNode& n, const cnh_ast_node& root, int i, XArray** out,
               const char* what) {
    CNH_CHECK(root.n_operands > i, -28, "%s: operand %d missing", what, i);
    const cnh_ast_node& op = n.nodes[root.operands[i]];
    CNH_CHECK(!op.is_scalar && op.opcode == CNH_OP_NOOP, -28, "%s: operand %d is not an array", what, i);
    if (int rc = find_array(ex, op.result_name, out, what))
        return rc;
    CNH_CHECK(!root.has_operand_region[i] || region_is_whole(root.operand_regions[i], **out), -29,
              "%s on a slice of array %d is not supported", what, op.result_name);
    return 0;
}

// Operand i of a product or dot with the window it is read through (the whole array when the node
// carries no region): unit steps only, inside the array.
int leaf_window(Ex* ex, const DagNode& n, const cnh_ast_node& root, int i, XArray** out,
                cnh_region* win, const char* what) {
    CNH_CHECK(root.n_operands > i, -28, "%s: operand %d missing", what, i);
    const cnh_ast_node& op = n.nodes[root.operands[i]];
    CNH_CHECK(!op.is_scalar && op.opcode == CNH_OP_NOOP, -28, "%s: operand %d is not an array", what, i);
    if (int rc = find_array(ex, op.result_name, out, what))
        return rc;
    const XArray& a = **out;
    std::memset(win, 0, sizeof *win);
    win->ndims = a.ndims;
    const bool whole = !root.has_operand_region[i] || root.operand_regions[i].is_global;
    CNH_CHECK(whole || root.operand_regions[i].ndims == a.ndims, -29,
              "%s: region of rank %d on array %d of rank %d", what, root.operand_regions[i].ndims,
              a.name, a.ndims);
    for (int d = 0; d < a.ndims; ++d) {
        win->start[d] = whole ? 0 : root.operand_regions[i].start[d];
        win->stop[d] = whole ? a.shape[d] : root.operand_regions[i].stop[d];
        win->step[d] = whole ? 1 : root.operand_regions[i].step[d];
        CNH_CHECK(win->step[d] == 1, -29, "%s on a strided slice of array %d is not supported", what,
                  a.name);
        CNH_CHECK(win->start[d] >= 0 && win->stop[d] > win->start[d] && win->stop[d] <= a.shape[d], -29,
                  "%s: window [%d:%d] leaves extent %d of array %d in dim %d", what, win->start[d],
                  win->stop[d], a.shape[d], a.name, d);
    }
    return 0;
}

// A copy of `src` laid out with another tile edge and offset, under a name of the executor's
// own. Products and paired reductions want their operands on matching tile grids; upstream
// redistributes them by messages (src/executor_matmul.cpp:150-498, src/executor_transfer.cpp),
// here one gather launch does it. The caller drops the copy when it is done.
int relayout(Ex* ex, XArray* src, int tile, const int32_t* offset, XArray** out) {
    const int name = ex->next_tmp--;
    Ex::Planned p;
    p.ndims = src->ndims;
    p.tile = tile;
    for (int d = 0; d < src->ndims; ++d) {
        p.shape[d] = src->shape[d];
        p.offset[d] = offset ? offset[d] : 0;
    }
    ex->planned[name] = p;
    DagNode dn;
    dn.id = -1;
    dn.nodes.resize(2);
    for (auto& a : dn.nodes) {
        std::memset(&a, 0, sizeof a);
        a.ndims = src->ndims;
        a.dtype = src->dtype;
        a.region.is_global = 1;
        a.operand_regions[0].is_global = a.operand_regions[1].is_global = 1;
    }
    dn.nodes[0].result_name = src->name;
    dn.nodes[0].opcode = CNH_OP_NOOP;
    dn.nodes[1].result_name = name;
    dn.nodes[1].opcode = CNH_OP_COPY;
    dn.nodes[1].n_operands = 1;
    dn.roots = {1};
    if (ex->trace_on) ex->log("relayout " + std::to_string(src->name) + " tile=" + std::to_string(tile) + " offset=" +
            shape_str(p.offset, src->ndims));
    if (int rc = exec_group(ex, dn))
        return rc;
    return find_array(ex, name, out, "relayout");
}

// The operand itself when its tile grid starts at element 0, else a copy that does.
int unphased(Ex* ex, XArray* a, XArray** out, bool* is_copy) {
    *is_copy = a->phased();
    *out = a;
    return *is_copy ? relayout(ex, a, a->tile, nullptr, out) : 0;
}

int new_scalar_array(Ex* ex, int name, int dtype, XArray** out) {
    int32_t one[3] = {1, 1, 1};
    return make_array(ex, name, 1, dtype, one, false, out);
}

// The matvec launches of a timed stretch (cnx_set_matvec_timing) are bracketed by event pairs.
cnh_event matvec_timer_start(Ex* ex) {
    if (!ex->time_matvec || ex->dry)
        return nullptr;
    cnh_event e0 = nullptr;
    if (cnh_event_create(&e0) != 0 || cnh_event_record(e0, ex->stream) != 0)
        return nullptr;
    return e0;
}
void matvec_timer_stop(Ex* ex, cnh_event e0) {
    if (e0 == nullptr)
        return;
    cnh_event e1 = nullptr;
    if (cnh_event_create(&e1) == 0 && cnh_event_record(e1, ex->stream) == 0)
        ex->matvec_events.emplace_back(e0, e1);
}

// REDUCE: per-tile dots and their in-order sum, result = size-1 array
// (src/executor_reduce.cpp:8-119, src/executor_reducer.cpp:11-57, src/partition_comm.cpp:69-111).
int exec_reduce(Ex* ex, const DagNode& n, const cnh_ast_node& root) {
    XArray *a, *b;
    cnh_region wa, wb;
    if (int rc = leaf_window(ex, n, root, 0, &a, &wa, "REDUCE"))
        return rc;
    if (int rc = leaf_window(ex, n, root, 1, &b, &wb, "REDUCE"))
        return rc;
    CNH_CHECK(a->ndims == 1 && b->ndims == 1, -30, "REDUCE needs 1-D operands");
    const int64_t len = wa.stop[0] - wa.start[0];
    CNH_CHECK(len == wb.stop[0] - wb.start[0], -30, "REDUCE: lengths %lld and %d", (long long)len,
              wb.stop[0] - wb.start[0]);
    CNH_CHECK(a->dtype == b->dtype, -27, "REDUCE: operand dtypes %d and %d", a->dtype, b->dtype);
    XArray* out;
    if (int rc = new_scalar_array(ex, root.result_name, a->dtype, &out))
        return rc;
    // 1-D arrays are contiguous as a whole. The partial sums follow the first operand's tiles
    // (the pieces of them its window covers); the second operand is cut at the same places.
    const int esz = dtype_size(a->dtype);
    std::vector<const void*> pa, pb;
    std::vector<int64_t> cnt;
    for (int64_t t = 0; t < a->ntiles; ++t) {
        int32_t lo[3], ext[3];
        a->tile_extent(t, lo, ext);
        const int64_t first = std::max<int64_t>(lo[0], wa.start[0]);
        const int64_t last = std::min<int64_t>(lo[0] + ext[0], wa.stop[0]);
        if (last <= first)
            continue;
        pa.push_back(static_cast<const char*>(a->tiles[0]) + first * esz);
        pb.push_back(static_cast<const char*>(b->tiles[0]) + (first - wa.start[0] + wb.start[0]) * esz);
        cnt.push_back(last - first);
    }
    if (ex->trace_on) ex->log("reduce " + std::to_string(a->name) + "." + std::to_string(b->name) + " tiles=" +
            std::to_string(pa.size()) + " out=" + std::to_string(out->name));
    if (ex->dry)
        return 0;
    return cnh_dot_tiles(a->dtype, (int)pa.size(), pa.data(), pb.data(), cnt.data(), out->tiles[0],
                         ex->stream);
}

int exec_reduce_ext(Ex* ex, const DagNode& n, const cnh_ast_node& root) {
    XArray *a, *b = nullptr;
    int b_copy = 0;
    if (int rc = leaf_array(ex, n, root, 0, &a, "reduction"))
        return rc;
    if (root.opcode != kOpSum) {
        if (int rc = leaf_array(ex, n, root, 1, &b, "reduction"))
            return rc;
        bool same_shape = a->ndims == b->ndims;
        for (int d = 0; d < a->ndims && same_shape; ++d)
            same_shape = a->shape[d] == b->shape[d];
        CNH_CHECK(same_shape, -30, "reduction: operands differ in shape");
        CNH_CHECK(a->dtype == CNH_F64 && b->dtype == CNH_F64, -27, "reduction: fp64 operands needed");
        if (!same_decomposition(*a, *b)) {
            if (int rc = relayout(ex, b, a->tile, a->offset, &b))
                return rc;
            b_copy = b->name;
        }
    }
    XArray* out;
    if (int rc = new_scalar_array(ex, root.result_name, a->dtype, &out))
        return rc;
    if (ex->trace_on) ex->log("reduce_ext op=" + std::to_string(root.opcode) + " tiles=" + std::to_string(a->ntiles) +
            " out=" + std::to_string(out->name));
    int rc = 0;
    if (!ex->dry) {
        std::vector<const void*> pa(a->tiles.begin(), a->tiles.end()), pb;
        if (b)
            pb.assign(b->tiles.begin(), b->tiles.end());
        std::vector<int64_t> cnt(a->tile_elems);
        if (a->flat) {
            // one block: a single contiguous chunk (b has the same shape and so the same layout)
            pa.assign(1, a->slab);
            if (b)
                pb.assign(1, b->slab);
            cnt.assign(1, a->elems);
        }
        const int nchunks = (int)pa.size();
        if (root.opcode == kOpSum)
            rc = cnh_sum_tiles(a->dtype, nchunks, pa.data(), cnt.data(), out->tiles[0], ex->stream);
        else if (root.opcode == kOpSumsqDiff)
            rc = cnh_sumsq_diff_tiles(nchunks, pa.data(), pb.data(), cnt.data(), out->tiles[0],
                                      ex->stream);
        else
            rc = cnh_maxabs_diff_tiles(nchunks, pa.data(), pb.data(), cnt.data(), out->tiles[0],
                                       ex->stream);
    }
    if (b_copy)
        drop_array(ex, b_copy);
    return rc;
}

// ASTYPE: a new array of the operand's shape and the node's dtype. One converting strided copy per
// pair of tiles that meet (the two arrays are cut by the same rule, so unless a plan placed them
// differently that is one launch per tile, or one for a whole rank-3 block).
int exec_astype(Ex* ex, const DagNode& n, const cnh_ast_node& root) {
    XArray* in;
    if (int rc = leaf_array(ex, n, root, 0, &in, "ASTYPE"))
        return rc;
    CNH_CHECK(dtype_size(root.dtype) != 0, -27, "ASTYPE: unknown dtype %d", root.dtype);
    const int nd = in->ndims;
    int32_t shape[3] = {1, 1, 1};
    for (int d = 0; d < nd; ++d)
        shape[d] = in->shape[d];
    XArray* out;
    if (int rc = make_array(ex, root.result_name, nd, root.dtype, shape, false, &out))
        return rc;
    if (int rc = find_array(ex, n.nodes[root.operands[0]].result_name, &in, "ASTYPE"))   // the map may have moved it
        return rc;
    int launches = 0;
    const bool blocks = in->flat && out->flat;
    for (int64_t ot = 0; ot < (blocks ? 1 : out->ntiles); ++ot) {
        int32_t olo[3] = {0, 0, 0}, oext[3] = {1, 1, 1};
        if (blocks)
            for (int d = 0; d < nd; ++d)
                oext[d] = shape[d];
        else
            out->tile_extent(ot, olo, oext);
        for (int64_t it = 0; it < (blocks ? 1 : in->ntiles); ++it) {
            int32_t ilo[3] = {0, 0, 0}, iext[3] = {1, 1, 1};
            if (blocks)
                for (int d = 0; d < nd; ++d)
                    iext[d] = shape[d];
            else
                in->tile_extent(it, ilo, iext);
            int64_t dstr[3], sstr[3], dsta[3], ssta[3], one[3] = {1, 1, 1}, counts[3];
            bool empty = false;
            for (int d = 0; d < nd; ++d) {
                const int lo = std::max(olo[d], ilo[d]), hi = std::min(olo[d] + oext[d], ilo[d] + iext[d]);
                if (hi <= lo)
                    empty = true;
                dsta[d] = lo - olo[d];
                ssta[d] = lo - ilo[d];
                counts[d] = hi - lo;
            }
            if (empty)
                continue;
            out->tile_strides(oext, dstr);
            in->tile_strides(iext, sstr);
            ++launches;
            if (!ex->dry)
                if (int rc = cnh_convert_region(nd, out->dtype, blocks ? out->slab : out->tiles[ot], dstr, dsta, one,
                                                in->dtype, blocks ? in->slab : in->tiles[it], sstr, ssta, one,
                                                counts, ex->stream))
                    return rc;
        }
    }
    if (ex->trace_on) ex->log("astype in=" + std::to_string(in->name) + " out=" + std::to_string(out->name) + " dtype=" +
            std::to_string(out->dtype) + " launches=" + std::to_string(launches));
    return 0;
}

// ---- boxes: unit-step regions that are one strided block of device memory ----
struct BoxUse {
    XArray* arr = nullptr;
    cnh_region reg;        // explicit, unit steps, in the array's own rank
    int map[3] = {-1, -1, -1};   // statement dimension -> array dimension (or -1: extent 1, no such dim)
};
struct Stmt {
    const DagNode* n = nullptr;
    int nd = 0, dtype = CNH_F64;
    int32_t cnt[3] = {1, 1, 1};
    BoxUse out;
    struct Read { int root, slot; BoxUse use; };
    std::vector<Read> reads;
    // one-element arrays read as kernel scalars: the launch fetches them through a device pointer
    // before any lane has stored, so no statement of the same launch may assign them
    std::vector<const XArray*> scalars_read;
};

constexpr int64_t kFuseMaxElems = 1ll << 22;   // larger statements are bandwidth bound anyway
constexpr size_t kFuseMaxStmts = 12, kFuseMaxReads = 16;

bool boxes_identical(const BoxUse& a, const BoxUse& b) {
    return a.arr == b.arr && same_region(a.reg, b.reg);
}
bool boxes_disjoint(const BoxUse& a, const BoxUse& b) {
    if (a.arr != b.arr)
        return true;
    for (int d = 0; d < a.arr->ndims; ++d)
        if (a.reg.stop[d] <= b.reg.start[d] || b.reg.stop[d] <= a.reg.start[d])
            return true;
    return false;
}

// One strided block of device memory?
bool box_is_one_block(const XArray& a, const cnh_region& r) {
    if (a.flat || a.ntiles == 1 || a.ndims == 1)
        return true;
    if (a.phased())
        return false;
    for (int d = 0; d < a.ndims; ++d)
        if (r.start[d] / a.tile != (r.stop[d] - 1) / a.tile)
            return false;
    return true;
}

// Fills `use` for array `a` read or written through `reg` (whole array when !has) by a statement
// of extents cnt[0..nd): unit steps, inside the array, extents equal to cnt with extent-1
// dimensions inserted or dropped in order, one block of memory.
bool make_box(XArray* a, bool has, const cnh_region& reg, int nd, const int32_t* cnt, BoxUse& use) {
    use.arr = a;
    std::memset(&use.reg, 0, sizeof use.reg);
    use.reg.ndims = a->ndims;
    if (has && !reg.is_global && reg.ndims != a->ndims)
        return false;
    for (int d = 0; d < a->ndims; ++d) {
        const bool whole = !has || reg.is_global;
        use.reg.start[d] = whole ? 0 : reg.start[d];
        use.reg.stop[d] = whole ? a->shape[d] : reg.stop[d];
        use.reg.step[d] = 1;
        if (!whole && reg.step[d] != 1)
            return false;
        if (use.reg.start[d] < 0 || use.reg.stop[d] > a->shape[d] || use.reg.stop[d] <= use.reg.start[d])
            return false;
    }
    // match the box's extents with the statement's, skipping extent-1 dimensions on either side
    int ad = 0;
    for (int d = 0; d < nd; ++d) {
        use.map[d] = -1;
        while (ad < a->ndims && use.reg.stop[ad] - use.reg.start[ad] == 1 && cnt[d] != 1)
            ++ad;
        if (ad < a->ndims && use.reg.stop[ad] - use.reg.start[ad] == cnt[d]) {
            // an extent of 1 on both sides pairs up only when enough array dimensions remain
            if (cnt[d] == 1 && a->ndims - ad < nd - d)
                continue;
            use.map[d] = ad++;
        } else if (cnt[d] != 1) {
            return false;
        }
    }
    for (; ad < a->ndims; ++ad)
        if (use.reg.stop[ad] - use.reg.start[ad] != 1)
            return false;
    return box_is_one_block(*a, use.reg);
}

cnh_memref box_memref(const BoxUse& u, int nd, const int32_t* cnt) {
    const XArray& a = *u.arr;
    const int esz = dtype_size(a.dtype);
    int64_t stride[3] = {1, 1, 1};
    char* base = nullptr;
    if (a.flat || a.ndims == 1) {
        // the whole array is one row-major run
        int64_t run = 1, off = 0;
        for (int d = a.ndims - 1; d >= 0; --d) {
            stride[d] = a.flat ? a.pitch[d] : run;
            run *= a.shape[d];
            off += u.reg.start[d] * stride[d];
        }
        base = static_cast<char*>(a.tiles[0]) + off * esz;
    } else {
        int64_t t = 0;
        for (int d = 0; d < a.ndims; ++d)
            t = t * a.grid[d] + (a.ntiles == 1 ? 0 : u.reg.start[d] / a.tile);
        int32_t lo[3], ext[3];
        a.tile_extent(t, lo, ext);
        a.tile_strides(ext, stride);
        int64_t off = 0;
        for (int d = 0; d < a.ndims; ++d)
            off += (int64_t)(u.reg.start[d] - lo[d]) * stride[d];
        base = static_cast<char*>(a.tiles[(size_t)t]) + off * esz;
    }
    cnh_memref m;
    std::memset(&m, 0, sizeof m);
    m.allocated = m.aligned = base;
    for (int d = 0; d < nd; ++d) {
        m.sizes[d] = cnt[d];
        m.strides[d] = u.map[d] >= 0 ? stride[u.map[d]] : 0;
    }
    return m;
}

// A window of a 2-D array, or of a 3-D array where the window has an extent of 1 along one
// dimension (the first such is dropped), seen as a matrix in the array's own coordinates
// (the sliced and dimension-dropped operands of charmnumeric.py:510-519,536-578 upstream,
// src/executor_matmatmul.cpp:485-813). The array's tile grid starts at element 0 (unphased()).
struct MatView {
    const XArray* a = nullptr;
    int rd = 0, cd = 1, dd = -1; // row, column and dropped dimension of the array
    int r0 = 0, c0 = 0, plane = 0; // where the window starts; index along the dropped dimension
    int rows = 0, cols = 0;
    // Pointer to array element (row ar, column ac) of the plane, the row stride of the tile that
    // holds it, and that tile's bounds [rlo, rhi) x [clo, chi) in array coordinates.
    const char* at(int ar, int ac, int64_t* ld, int* rlo, int* rhi, int* clo, int* chi) const {
        int idx[3] = {0, 0, 0};
        idx[rd] = ar;
        idx[cd] = ac;
        if (dd >= 0)
            idx[dd] = plane;
        if (a->flat) {
            // one row-major block: nothing cuts a panel short, whatever the array's partitions are
            int64_t off = 0;
            for (int d = 0; d < a->ndims; ++d)
                off += (int64_t)idx[d] * a->pitch[d];
            *ld = a->pitch[rd];
            *rlo = 0;
            *rhi = a->shape[rd];
            *clo = 0;
            *chi = a->shape[cd];
            return static_cast<const char*>(a->slab) + off * dtype_size(a->dtype);
        }
        int64_t t = 0;
        for (int d = 0; d < a->ndims; ++d)
            t = t * a->grid[d] + idx[d] / a->tile;
        int32_t lo[3], ext[3];
        a->tile_extent(t, lo, ext);
        int64_t stride[3] = {1, 1, 1}, off = 0;
        a->tile_strides(ext, stride);
        for (int d = 0; d < a->ndims; ++d)
            off += (int64_t)(idx[d] - lo[d]) * stride[d];
        *ld = stride[rd];
        *rlo = lo[rd];
        *rhi = lo[rd] + ext[rd];
        *clo = lo[cd];
        *chi = lo[cd] + ext[cd];
        return static_cast<const char*>(a->tiles[(size_t)t]) + off * dtype_size(a->dtype);
    }
};

int as_matrix(const XArray& a, const cnh_region& win, MatView* m, const char* what) {
    m->a = &a;
    if (a.ndims == 2) {
        m->rd = 0;
        m->cd = 1;
        m->dd = -1;
    } else {
        CNH_CHECK(a.ndims == 3, -32, "%s needs 2-D operands (or 3-D with one extent of 1)", what);
        int dropped = -1;
        for (int d = 0; d < 3 && dropped < 0; ++d)
            if (win.stop[d] - win.start[d] == 1)
                dropped = d;
        CNH_CHECK(dropped >= 0, -32, "%s: 3-D operand %d has no extent of 1", what, a.name);
        m->dd = dropped;
        m->rd = dropped == 0 ? 1 : 0;
        m->cd = dropped == 2 ? 1 : 2;
        m->plane = win.start[dropped];
        // rows of the matrix must be contiguous in memory: nothing but extent 1 after the columns
        CNH_CHECK(m->cd == 2 || a.shape[2] == 1, -29,
                  "%s: the last dimension of array %d is dropped but has extent %d", what, a.name,
                  a.shape[2]);
    }
    m->r0 = win.start[m->rd];
    m->c0 = win.start[m->cd];
    m->rows = win.stop[m->rd] - m->r0;
    m->cols = win.stop[m->cd] - m->c0;
    return 0;
}

// MATMUL: tile GEMVs, column tiles summed in index order (src/executor_matmul.cpp:150-498,
// src/execute_node.cpp:116-273,489-583).
int exec_matmul(Ex* ex, const DagNode& n, const cnh_ast_node& root) {
    XArray *Aa, *x;
    cnh_region wA, wx;
    if (int rc = leaf_window(ex, n, root, 0, &Aa, &wA, "MATMUL"))
        return rc;
    if (int rc = leaf_window(ex, n, root, 1, &x, &wx, "MATMUL"))
        return rc;
    bool a_copy = false;
    if (int rc = unphased(ex, Aa, &Aa, &a_copy))
        return rc;
    // a 3-D matrix operand with one extent of 1 is the plane that remains
    // (charmnumeric.py:552-563, the K14 case of src/executor_matmul.cpp upstream)
    MatView A;
    if (int rc = as_matrix(*Aa, wA, &A, "MATMUL"))
        return rc;
    CNH_CHECK(x->ndims == 1, -31, "MATMUL needs a 1-D vector operand");
    CNH_CHECK(A.cols == wx.stop[0] - wx.start[0], -31, "MATMUL: %d columns, vector of %d", A.cols,
              wx.stop[0] - wx.start[0]);
    CNH_CHECK(Aa->dtype == x->dtype, -27, "MATMUL: operand dtypes %d and %d", Aa->dtype, x->dtype);
    int32_t shape[3] = {A.rows, 1, 1};
    XArray* y;
    if (int rc = make_array(ex, root.result_name, 1, Aa->dtype, shape, false, &y))
        return rc;
    if (ex->trace_on) ex->log("matmul A=" + std::to_string(Aa->name) + " tiles=" + std::to_string(Aa->ntiles) + " x=" +
            std::to_string(x->name) + " out=" + std::to_string(y->name));
    int rc = 0;
    if (!ex->dry) {
        // one panel per tile the window meets; panel rows are the array's tile rows (an array
        // stored as one block is a single panel)
        const int T = Aa->flat ? (1 << 30) : Aa->tile;
        const int pr0 = A.r0 / T, pr1 = (A.r0 + A.rows - 1) / T;
        const int pc0 = A.c0 / T, pc1 = (A.c0 + A.cols - 1) / T;
        std::vector<cnh_gemv_panel> panels;
        for (int pr = pr0; pr <= pr1; ++pr)
            for (int pc = pc0; pc <= pc1; ++pc) {
                const int ac = std::max(pc * T, A.c0);
                int64_t ld;
                int rlo, rhi, clo, chi;
                const char* p = A.at(pr * T, ac, &ld, &rlo, &rhi, &clo, &chi);
                const int cend = std::min(chi, A.c0 + A.cols);
                panels.push_back(cnh_gemv_panel{p, ld, cend - ac, ac - A.c0});
            }
        // 1-D arrays are contiguous: the vector window is a pointer into tile 0.
        const char* xp = static_cast<const char*>(x->tiles[0]) + (int64_t)wx.start[0] * dtype_size(x->dtype);
        cnh_event t0 = matvec_timer_start(ex);
        rc = cnh_gemv_panels(Aa->dtype, A.rows, pc1 - pc0 + 1, T, A.r0 - pr0 * T, (int64_t)panels.size(),
                             panels.data(), xp, y->tiles[0], ex->stream);
        matvec_timer_stop(ex, t0);
    }
    if (a_copy)
        drop_array(ex, Aa->name);
    return rc;
}

// MATMATMUL: C = sum of A_panel * B_panel over every k-overlapping pair of tiles, k ascending
// (src/executor_matmatmul.cpp:105-484, src/executor_incremental.cpp:97-132).
// `dest`: where the product goes instead of a new array (the box a following assignment names),
// null for the ordinary form.
// `plan_only`: nothing is launched, created or copied; when the product would go into the box as a
// list of panel products of operands that need no copy, the list is left there (else it stays empty),
// with the operands' arrays and windows in `operands`.
struct ProductOperands {
    XArray *A = nullptr, *B = nullptr;
    cnh_region wA, wB;
    int M = 0, N = 0, K = 0;
};
int exec_matmatmul(Ex* ex, const DagNode& n, const cnh_ast_node& root, const DagNode* dest_node = nullptr,
                   bool* dest_taken = nullptr, std::vector<cnh_gemm_job>* plan_only = nullptr,
                   ProductOperands* operands = nullptr) {
    XArray *Aa, *Ba;
    cnh_region wA, wB;
    if (int rc = leaf_window(ex, n, root, 0, &Aa, &wA, "MATMATMUL"))
        return rc;
    if (int rc = leaf_window(ex, n, root, 1, &Ba, &wB, "MATMATMUL"))
        return rc;
    if (plan_only != nullptr) {
        plan_only->clear();
        if (Aa->phased() || Ba->phased())
            return 0;
        if (operands != nullptr)
            *operands = ProductOperands{Aa, Ba, wA, wB, 0, 0, 0};
    }
    bool a_copy = false, b_copy = false;
    if (int rc = unphased(ex, Aa, &Aa, &a_copy))
        return rc;
    if (int rc = unphased(ex, Ba, &Ba, &b_copy))
        return rc;
    MatView A, B;
    if (int rc = as_matrix(*Aa, wA, &A, "MATMATMUL"))
        return rc;
    if (int rc = as_matrix(*Ba, wB, &B, "MATMATMUL"))
        return rc;
    CNH_CHECK(A.cols == B.rows, -32, "MATMATMUL: (%d,%d) @ (%d,%d)", A.rows, A.cols, B.rows, B.cols);
    CNH_CHECK(Aa->dtype == Ba->dtype, -27, "MATMATMUL: operand dtypes %d and %d", Aa->dtype, Ba->dtype);
    if (plan_only != nullptr && operands != nullptr) {
        operands->M = A.rows;
        operands->N = B.cols;
        operands->K = A.cols;
    }
    int32_t shape[3] = {A.rows, B.cols, 1};
    // fp64 products overwrite their result (every C element belongs to exactly one chain), so the
    // new array needs no zero-fill; the other types accumulate into zeros as upstream does
    const bool f64 = Aa->dtype == CNH_F64;
    // The product of `target[box] = A @ B` goes straight into the box when that is one strided
    // block with unit stride along the columns: no temporary, no copy (fp64 only: the product
    // overwrites, so what the box held does not matter).
    XArray* Cc = nullptr;
    char* dest_base = nullptr;
    int64_t dest_ld = 0;
    int dest_name = 0;
    if (dest_node != nullptr && f64) {
        const cnh_ast_node* dest_set = &dest_node->nodes[dest_node->roots.back()];
        XArray* target = nullptr;
        auto it = ex->arrays.find(dest_node->nodes[dest_set->operands[0]].result_name);
        if (it != ex->arrays.end())
            target = &it->second;
        BoxUse use;
        const int32_t cnt2[2] = {A.rows, B.cols};
        if (target != nullptr && target->dtype == Aa->dtype && target != Aa && target != Ba &&
            make_box(target, true, dest_set->region, 2, cnt2, use) && use.map[0] >= 0 &&
            use.map[1] == target->ndims - 1) {
            const cnh_memref m = box_memref(use, 2, cnt2);
            if (m.strides[1] == 1) {
                dest_base = static_cast<char*>(m.aligned);
                dest_ld = m.strides[0];
                dest_name = target->name;
            }
        }
    }
    if (dest_taken != nullptr)
        *dest_taken = dest_base != nullptr;
    if (plan_only != nullptr && dest_base == nullptr)
        return 0;
    if (dest_base == nullptr)
        if (int rc = make_array(ex, root.result_name, 2, Aa->dtype, shape, !f64, &Cc))
            return rc;
    const int esz = dtype_size(Aa->dtype);
    // panels end where an operand's tiles end; an array stored as one block has no such ends
    const int kNoCut = 1 << 30;
    const int TA = Aa->flat ? kNoCut : Aa->tile, TB = Ba->flat ? kNoCut : Ba->tile, K = A.cols;
    int calls = 0;
    std::vector<cnh_gemm_job> jobs;   // all panel products of the node go out as one launch
    const int cgrid0 = Cc ? Cc->grid[0] : 1, cgrid1 = Cc ? Cc->grid[1] : 1;
    for (int ci = 0; ci < cgrid0; ++ci)
        for (int cj = 0; cj < cgrid1; ++cj) {
            int32_t clo[3] = {0, 0, 0}, cext[3] = {A.rows, B.cols, 1};
            if (Cc)
                Cc->tile_extent((int64_t)ci * Cc->grid[1] + cj, clo, cext);
            char* const ctile = Cc ? static_cast<char*>(Cc->tiles[(size_t)ci * Cc->grid[1] + cj]) : dest_base;
            int64_t cstr[3] = {dest_ld, 1, 1};
            if (Cc)
                Cc->tile_strides(cext, cstr);   // a tile's own width, or the pitch of a block
            const int64_t cld = cstr[0];
            // rows i of this C tile are rows A.r0 + i of A's array, its columns j are columns
            // B.c0 + j of B's: cut both ranges where those arrays' tiles end
            for (int r0 = clo[0]; r0 < clo[0] + cext[0];) {
                const int r1 = std::min(clo[0] + cext[0], ((A.r0 + r0) / TA + 1) * TA - A.r0);
                for (int c0 = clo[1]; c0 < clo[1] + cext[1];) {
                    const int c1 = std::min(clo[1] + cext[1], ((B.c0 + c0) / TB + 1) * TB - B.c0);
                    // k pieces: common refinement of A's column tiles and B's row tiles
                    for (int k0 = 0; k0 < K;) {
                        const int k1 = std::min(K, std::min(((A.c0 + k0) / TA + 1) * TA - A.c0,
                                                            ((B.r0 + k0) / TB + 1) * TB - B.r0));
                        int64_t lda, ldb;
                        int t0, t1, t2, t3;
                        const char* ap = A.at(A.r0 + r0, A.c0 + k0, &lda, &t0, &t1, &t2, &t3);
                        const char* bp = B.at(B.r0 + k0, B.c0 + c0, &ldb, &t0, &t1, &t2, &t3);
                        char* cp = ctile + ((int64_t)(r0 - clo[0]) * cld + (c0 - clo[1])) * esz;
                        ++calls;
                        jobs.push_back(cnh_gemm_job{r1 - r0, c1 - c0, k1 - k0, ap, lda, bp, ldb, cp, cld});
                        k0 = k1;
                    }
                    c0 = c1;
                }
                r0 = r1;
            }
        }
    if (plan_only != nullptr) {
        plan_only->swap(jobs);
        return 0;
    }
    if (!ex->dry)
        if (int rc = cnh_gemm_batch(Aa->dtype, (int)jobs.size(), jobs.data(), f64 ? 1 : 0, ex->stream))
            return rc;
    if (ex->trace_on) ex->log("matmatmul A=" + std::to_string(Aa->name) + " B=" + std::to_string(Ba->name) + " out=" +
            std::to_string(Cc ? Cc->name : dest_name) + (Cc ? "" : " into_region") + " panel_products=" +
            std::to_string(calls));
    if (a_copy)
        drop_array(ex, Aa->name);
    if (b_copy)
        drop_array(ex, Ba->name);
    return 0;
}

// TILE: out[i0, i1, ..] = in[i0 % s0, i1 % s1, ..] with the input's shape left-padded with ones
// to the output's rank (charmnumeric/operations.py:52-72, src/dag_group_receive.cpp:353-375).
// One strided copy per (output tile, input tile, repetition) that meet; a repeated extent-1
// dimension is a copy with source step 0.
int exec_tile(Ex* ex, const DagNode& n, const cnh_ast_node& root) {
    CNH_CHECK(root.n_operands >= 1, -36, "TILE: no operand");
    const cnh_ast_node& op = n.nodes[root.operands[0]];
    XArray* in;
    if (int rc = find_array(ex, op.result_name, &in, "TILE"))
        return rc;
    CNH_CHECK(!root.region.is_global && root.region.ndims == root.ndims, -36,
              "TILE %d carries no result shape", root.result_name);
    const int nd = root.ndims, delta = nd - in->ndims;
    CNH_CHECK(delta >= 0 && nd <= 3, -36, "TILE: result rank %d below operand rank %d", nd, in->ndims);
    int32_t oshape[3] = {1, 1, 1}, ishape[3] = {1, 1, 1};
    for (int d = 0; d < nd; ++d) {
        oshape[d] = region_count(root.region, d);
        ishape[d] = d < delta ? 1 : in->shape[d - delta];
        CNH_CHECK(oshape[d] % ishape[d] == 0, -36, "TILE: extent %d is not a multiple of %d", oshape[d],
                  ishape[d]);
    }
    XArray* out;
    if (int rc = make_array(ex, root.result_name, nd, in->dtype, oshape, false, &out))
        return rc;
    const int esz = dtype_size(in->dtype);
    int copies = 0;
    for (int64_t ot = 0; ot < out->ntiles; ++ot) {
        int32_t olo[3], oext[3];
        out->tile_extent(ot, olo, oext);
        for (int64_t it = 0; it < in->ntiles; ++it) {
            int32_t ilo_a[3], iext_a[3], ilo[3] = {0, 0, 0}, iext[3] = {1, 1, 1};
            in->tile_extent(it, ilo_a, iext_a);
            for (int d = 0; d < in->ndims; ++d) {
                ilo[d + delta] = ilo_a[d];
                iext[d + delta] = iext_a[d];
            }
            // per dimension: repetitions r with [r*s + ilo, r*s + ilo + iext) meeting the output tile
            int rlo[3], rhi[3];
            bool none = false;
            for (int d = 0; d < nd; ++d) {
                const int sdim = ishape[d];
                rlo[d] = std::max(0, (olo[d] - ilo[d] - iext[d] + sdim) / sdim);
                rhi[d] = std::min(oshape[d] / sdim - 1, (olo[d] + oext[d] - 1 - ilo[d]) / sdim);
                if (ishape[d] == 1) { // extent-1 source: one copy with step 0 covers all repetitions
                    rlo[d] = 0;
                    rhi[d] = 0;
                }
                if (rhi[d] < rlo[d])
                    none = true;
            }
            if (none)
                continue;
            int r[3] = {0, 0, 0};
            for (r[0] = rlo[0]; r[0] <= (nd > 0 ? rhi[0] : 0); ++r[0])
                for (r[1] = nd > 1 ? rlo[1] : 0; r[1] <= (nd > 1 ? rhi[1] : 0); ++r[1])
                    for (r[2] = nd > 2 ? rlo[2] : 0; r[2] <= (nd > 2 ? rhi[2] : 0); ++r[2]) {
                        int64_t dstart[3], dstep[3], sstart[3], sstep[3], counts[3], dstr[3], sstr[3];
                        bool empty = false;
                        out->tile_strides(oext, dstr);
                        {
                            // the input's tile with its shape left-padded to the output's rank
                            int64_t ss = 1;
                            for (int d = nd - 1; d >= 0; --d) {
                                sstr[d] = ss;
                                ss *= iext[d];
                            }
                            if (in->flat)
                                for (int d = 0; d < in->ndims; ++d)
                                    sstr[d + delta] = in->pitch[d];
                        }
                        for (int d = 0; d < nd; ++d) {
                            if (ishape[d] == 1) {
                                dstart[d] = 0;
                                counts[d] = oext[d];
                                sstart[d] = 0;
                                sstep[d] = 0;
                            } else {
                                const int g0 = r[d] * ishape[d] + ilo[d]; // where this piece lands
                                const int lo = std::max(g0, (int)olo[d]);
                                const int hi = std::min(g0 + iext[d], olo[d] + oext[d]);
                                if (hi <= lo)
                                    empty = true;
                                dstart[d] = lo - olo[d];
                                counts[d] = hi - lo;
                                sstart[d] = lo - g0;
                                sstep[d] = 1;
                            }
                            dstep[d] = 1;
                        }
                        if (empty)
                            continue;
                        ++copies;
                        if (!ex->dry)
                            if (int rc = cnh_copy_region(nd, esz, out->tiles[ot], dstr, dstart, dstep,
                                                         in->tiles[it], sstr, sstart, sstep, counts,
                                                         ex->stream))
                                return rc;
                    }
        }
    }
    if (ex->trace_on) ex->log("tile in=" + std::to_string(in->name) + " out=" + std::to_string(out->name) + " shape=" +
            shape_str(out->shape, nd) + " copies=" + std::to_string(copies));
    return 0;
}

// DIAG with numpy.diag's meaning (charmnumeric/operations.py:125-148, src/dag_group_receive.cpp:330-347,
// src/executor_transfer.cpp:180-358, src/execute_node.cpp:600-720): a vector becomes the k-th
// diagonal of a zeroed square matrix, a matrix gives up its k-th diagonal. Vector index i pairs with
// matrix element (i + max(0,-k), i + max(0,k)). One strided copy per matrix tile the diagonal crosses:
// inside a row-major tile of width w the diagonal is a run with stride w + 1.
int exec_diag(Ex* ex, const DagNode& n, const cnh_ast_node& root) {
    XArray* in;
    if (int rc = leaf_array(ex, n, root, 0, &in, "DIAG"))
        return rc;
    int k = 0;
    if (root.n_operands >= 2) {
        const cnh_ast_node& kn = n.nodes[root.operands[1]];
        CNH_CHECK(kn.is_scalar, -37, "DIAG: the offset must be a scalar operand");
        k = (int)kn.scalar;
    }
    CNH_CHECK(in->ndims == 1 || in->ndims == 2, -37, "DIAG needs a 1-D or 2-D operand, got %d-D", in->ndims);
    const int r_off = std::max(0, -k), c_off = std::max(0, k);
    XArray *mat, *vec, *out;
    int len;
    if (in->ndims == 1) {
        len = in->shape[0];
        const int64_t side = (int64_t)len + std::abs(k);
        CNH_CHECK(side <= INT32_MAX, -37, "DIAG: result side %lld too large", (long long)side);
        int32_t shape[3] = {(int32_t)side, (int32_t)side, 1};
        if (int rc = make_array(ex, root.result_name, 2, in->dtype, shape, true, &out))
            return rc;
        mat = out;
        vec = in;
    } else {
        len = k >= 0 ? std::min(in->shape[0], in->shape[1] - k) : std::min(in->shape[0] + k, in->shape[1]);
        CNH_CHECK(len > 0, -37, "DIAG: k=%d is out of range for shape (%d, %d)", k, in->shape[0], in->shape[1]);
        int32_t shape[3] = {len, 1, 1};
        if (int rc = make_array(ex, root.result_name, 1, in->dtype, shape, false, &out))
            return rc;
        mat = in;
        vec = out;
    }
    const int esz = dtype_size(in->dtype);
    int copies = 0;
    for (int64_t t = 0; t < mat->ntiles; ++t) {
        int32_t lo[3], ext[3];
        mat->tile_extent(t, lo, ext);
        const int i0 = std::max(0, std::max(lo[0] - r_off, lo[1] - c_off));
        const int i1 = std::min(len, std::min(lo[0] + ext[0] - r_off, lo[1] + ext[1] - c_off));
        if (i1 <= i0)
            continue;
        ++copies;
        if (ex->dry)
            continue;
        int64_t tstr[3];
        mat->tile_strides(ext, tstr);           // row stride: the tile's own width, or the block's pitch
        const int64_t first = (int64_t)(i0 + r_off - lo[0]) * tstr[0] + (i0 + c_off - lo[1]);
        char* mp = static_cast<char*>(mat->tiles[(size_t)t]) + first * esz;
        char* vp = static_cast<char*>(vec->tiles[0]) + (int64_t)i0 * esz; // 1-D arrays are contiguous
        const int64_t mstr[1] = {tstr[0] + 1}, vstr[1] = {1}, zero[1] = {0}, one[1] = {1}, cnt[1] = {i1 - i0};
        const int rc = in->ndims == 1
                           ? cnh_copy_region(1, esz, mp, mstr, zero, one, vp, vstr, zero, one, cnt, ex->stream)
                           : cnh_copy_region(1, esz, vp, vstr, zero, one, mp, mstr, zero, one, cnt, ex->stream);
        if (rc)
            return rc;
    }
    if (ex->trace_on) ex->log("diag in=" + std::to_string(in->name) + " out=" + std::to_string(out->name) + " k=" +
            std::to_string(k) + " copies=" + std::to_string(copies));
    return 0;
}

int exec_node(Ex* ex, const DagNode& n) {
    CNH_CHECK(!n.roots.empty(), -33, "DAG node %d has no roots", n.id);
    const cnh_ast_node& root = n.nodes[n.roots.back()];
    ex->stats[2]++;
    switch (root.opcode) {
    case CNH_OP_CREATE: return exec_create(ex, root);
    case kOpDelete: drop_array(ex, root.result_name); return 0;
    case CNH_OP_REDUCE: return exec_reduce(ex, n, root);
    case kOpSum:
    case kOpSumsqDiff:
    case kOpMaxabsDiff: return exec_reduce_ext(ex, n, root);
    case kOpAstype: return exec_astype(ex, n, root);
    case CNH_OP_MATMUL: return exec_matmul(ex, n, root);
    case CNH_OP_MATMATMUL: return exec_matmatmul(ex, n, root);
    case CNH_OP_TILE: return exec_tile(ex, n, root);
    case CNH_OP_DIAG: return exec_diag(ex, n, root);
    case CNH_OP_ADD:
    case CNH_OP_SUB:
    case CNH_OP_MUL:
    case CNH_OP_DIV:
    case CNH_OP_TANH:
    case CNH_OP_EXP:
    case CNH_OP_COPY:
    case CNH_OP_SET_REGION: return exec_group(ex, n);
    case CNH_OP_NOOP: return 0;
    default:
        return set_error(-34, "DAG node %d: opcode %d is not supported by this executor", n.id,
                         root.opcode);
    }
}

// ---- several assignments of one extent as one launch ----
// A run of statements `target[box] = f(operands[boxes])` whose boxes all have the same extents
// (the gate statements of an LSTM step, the updates of several fields over one window) is launch
// bound when run one by one. Where every box is a single strided block of device memory — the
// array is one row-major block, or has one tile, or the box lies inside one tile — the run becomes
// one group with one output root per statement, launched through the memref interface
// (cnh_launch_group, the dispatch_kernel seam) with a memref per box. A statement that reads
// exactly the box an earlier one of the run assigned takes the value from registers; results are
// those of running the statements one after the other:
//   - a box read by a later statement and a box assigned by an earlier one of the same array are
//     either identical or share no element;
//   - a box assigned by a later statement and any box an earlier one read or assigned in the same
//     array are either identical or share no element (identical: the lane that reads or writes an
//     element is the lane that overwrites it later; an earlier identical store is dropped).

bool open_ended_allowed(const Ex* ex) { return !ex->final_pass; }

// Is node `n` an assignment this pass can take? Fills `st`.
bool analyse_statement(Ex* ex, const DagNode& n, Stmt& st) {
    if (n.roots.empty())
        return false;
    const cnh_ast_node& root = n.nodes[n.roots.back()];
    if (root.opcode != CNH_OP_SET_REGION || root.n_operands != 2 || root.region.is_global)
        return false;
    if (n.nodes[root.operands[1]].is_scalar)
        return false;                                   // a fill
    for (size_t i = 0; i + 1 < n.roots.size(); ++i)
        if (!n.nodes[n.roots[i]].is_temp)
            return false;
    st.n = &n;
    st.nd = root.region.ndims;
    int64_t elems = 1;
    for (int d = 0; d < st.nd; ++d) {
        if (root.region.step[d] != 1)
            return false;
        st.cnt[d] = root.region.stop[d] - root.region.start[d];
        if (st.cnt[d] <= 0)
            return false;
        elems *= st.cnt[d];
    }
    if (elems > kFuseMaxElems)
        return false;
    auto tgt = ex->arrays.find(n.nodes[root.operands[0]].result_name);
    if (tgt == ex->arrays.end() || tgt->second.ndims != st.nd)
        return false;
    st.dtype = tgt->second.dtype;
    if (!make_box(&tgt->second, true, root.region, st.nd, st.cnt, st.out))
        return false;
    std::set<int> internal;
    for (int32_t r : n.roots)
        internal.insert(n.nodes[r].result_name);
    st.reads.clear();
    st.scalars_read.clear();
    for (size_t ri = 0; ri < n.roots.size(); ++ri) {
        const cnh_ast_node& r = n.nodes[n.roots[ri]];
        if (r.dtype != st.dtype)
            return false;
        for (int oi = 0; oi < r.n_operands; ++oi) {
            if (r.opcode == CNH_OP_SET_REGION && oi == 0)
                continue;
            if (r.operands[oi] < 0 || r.operands[oi] >= (int)n.nodes.size())
                return false;
            const cnh_ast_node& op = n.nodes[r.operands[oi]];
            if (op.is_scalar || internal.count(op.result_name))
                continue;
            auto it = ex->arrays.find(op.result_name);
            if (it == ex->arrays.end() || it->second.dtype != st.dtype)
                return false;
            if (op.is_broadcast) {
                if (it->second.elems != 1 || &it->second == st.out.arr)
                    return false;
                st.scalars_read.push_back(&it->second);
                continue;
            }
            Stmt::Read rd;
            rd.root = (int)ri;
            rd.slot = oi;
            if (!make_box(&it->second, r.has_operand_region[oi] != 0, r.operand_regions[oi], st.nd, st.cnt,
                          rd.use))
                return false;
            // reading the assigned array elsewhere than at the assigned box: ping-pong territory
            if (rd.use.arr == st.out.arr && !boxes_identical(rd.use, st.out) && !boxes_disjoint(rd.use, st.out))
                return false;
            st.reads.push_back(rd);
        }
    }
    // one array read at several overlapping boxes is a stencil: the register-window route reads
    // each element once, this one would read it once per box
    for (size_t a = 0; a < st.reads.size(); ++a)
        for (size_t b = a + 1; b < st.reads.size(); ++b)
            if (st.reads[a].use.arr == st.reads[b].use.arr &&
                !boxes_identical(st.reads[a].use, st.reads[b].use) &&
                !boxes_disjoint(st.reads[a].use, st.reads[b].use))
                return false;
    return st.reads.size() <= kFuseMaxReads;
}

bool can_join(const std::vector<Stmt>& run, const Stmt& b) {
    const Stmt& first = run.front();
    if (b.nd != first.nd || b.dtype != first.dtype)
        return false;
    for (int d = 0; d < b.nd; ++d)
        if (b.cnt[d] != first.cnt[d])
            return false;
    size_t reads = b.reads.size();
    for (const Stmt& s : run) {
        reads += s.reads.size();
        for (const auto& rd : b.reads)
            if (!boxes_identical(rd.use, s.out) && !boxes_disjoint(rd.use, s.out))
                return false;
        if (!boxes_identical(b.out, s.out) && !boxes_disjoint(b.out, s.out))
            return false;
        for (const auto& rd : s.reads)
            if (!boxes_identical(b.out, rd.use) && !boxes_disjoint(b.out, rd.use))
                return false;
        // a kernel scalar is read once, at the start of the launch, by every lane: a statement
        // that assigns that array cannot share a launch with one that reads it as a scalar
        for (const XArray* a : b.scalars_read)
            if (a == s.out.arr)
                return false;
        for (const XArray* a : s.scalars_read)
            if (a == b.out.arr)
                return false;
    }
    return run.size() < kFuseMaxStmts && reads <= kFuseMaxReads;
}

// An assignment whose extent along one dimension is 2 to 4 times `want`'s there (the others equal)
// as that many assignments side by side, each with `want`'s extents: elementwise work may be cut
// anywhere, and the pieces can then join a run of statements of the smaller extent (an LSTM step's
// sigmoid over three gates' columns next to the statements on one gate's columns).
bool cut_statement(const Stmt& a, const int32_t* want, std::vector<Stmt>& pieces) {
    int along = -1;
    for (int d = 0; d < a.nd; ++d) {
        if (a.cnt[d] == want[d])
            continue;
        if (along >= 0 || want[d] <= 0 || a.cnt[d] % want[d] != 0)
            return false;
        along = d;
    }
    if (along < 0)
        return false;
    const int m = a.cnt[along] / want[along];
    if (m < 2 || m > 4)
        return false;
    auto narrowed = [&](const BoxUse& u, int k, BoxUse& out) {
        out = u;
        const int ad = u.map[along];
        if (ad < 0)
            return false;
        out.reg.start[ad] = u.reg.start[ad] + k * want[along];
        out.reg.stop[ad] = out.reg.start[ad] + want[along];
        return true;
    };
    pieces.clear();
    for (int k = 0; k < m; ++k) {
        Stmt p = a;
        p.cnt[along] = want[along];
        if (!narrowed(a.out, k, p.out))
            return false;
        for (size_t r = 0; r < a.reads.size(); ++r)
            if (!narrowed(a.reads[r].use, k, p.reads[r].use))
                return false;
        pieces.push_back(p);
    }
    return true;
}

// The run as one multi-root group. Boxes are numbered; the group's regions carry the numbers, not
// the coordinates (the launch hands over memrefs), so every step of a time loop finds the kernel
// of the first one in the cache.
// `site`: a product the run rides on. Reads of the product's box, column block by column block, take
// their values from the product's launch (cnh_launch_product_group); `fused` tells whether that launch
// took the shape, else the product and the run went out as two launches.
struct ProductSite {
    cnh_gemm_job job;
    XArray* target = nullptr;
    cnh_region region;         // the product's box in the target's coordinates
    int blocks = 1;            // column blocks the run reads it in
    std::string what;          // trace text of the product
    bool fused = false;
};
// Which column block of the site's box is `u` (-1: none)?
int product_block(const ProductSite& site, const BoxUse& u) {
    if (u.arr != site.target)
        return -1;
    const int last = site.target->ndims - 1;
    for (int d = 0; d < last; ++d)
        if (u.reg.start[d] != site.region.start[d] || u.reg.stop[d] != site.region.stop[d])
            return -1;
    const int width = (site.region.stop[last] - site.region.start[last]) / site.blocks;
    const int off = u.reg.start[last] - site.region.start[last];
    if (off < 0 || off % width != 0 || u.reg.stop[last] - u.reg.start[last] != width || off / width >= site.blocks)
        return -1;
    return off / width;
}

int exec_statement_run(Ex* ex, const std::vector<Stmt>& run, ProductSite* site = nullptr) {
    DagNode merged;
    merged.id = run.front().n->id;
    merged.fusible = 1;
    std::vector<BoxUse> boxes;                 // by number
    auto number_of = [&](const BoxUse& u) {
        for (size_t i = 0; i < boxes.size(); ++i)
            if (boxes_identical(boxes[i], u) && std::memcmp(boxes[i].map, u.map, sizeof u.map) == 0)
                return (int)i;
        boxes.push_back(u);
        return (int)boxes.size() - 1;
    };
    auto tag_region = [&](cnh_region& r, int number, int nd) {
        std::memset(&r, 0, sizeof r);
        r.ndims = nd;
        for (int d = 0; d < nd; ++d) {
            r.start[d] = number;
            r.stop[d] = number + 1;
            r.step[d] = 1;
        }
    };
    struct Done { int value_node; int set_root; const Stmt* st; };
    std::vector<Done> done;
    int next_literal = -1, next_temporary = 0x7e000000;
    for (const Stmt& st : run) {
        const DagNode& n = *st.n;
        const int base = (int)merged.nodes.size();
        for (const cnh_ast_node& a : n.nodes) {
            merged.nodes.push_back(a);
            cnh_ast_node& c = merged.nodes.back();
            for (int oi = 0; oi < c.n_operands; ++oi)
                if (c.operands[oi] >= 0)
                    c.operands[oi] += base;
            // literals are named per DAG node (-1, -2, ...): keep them apart across statements
            if (c.is_scalar)
                c.result_name = next_literal--;
        }
        // the pieces of a cut statement are copies of one node: their temporaries and the
        // assignment itself (a name nothing else refers to) need names of their own
        std::map<int, int> renamed;
        for (size_t ri = 0; ri + 1 < n.roots.size(); ++ri)
            renamed[n.nodes[(size_t)n.roots[ri]].result_name] = next_temporary++;
        for (size_t q = (size_t)base; q < merged.nodes.size(); ++q) {
            cnh_ast_node& c = merged.nodes[q];
            auto it = c.is_scalar ? renamed.end() : renamed.find(c.result_name);
            if (it != renamed.end())
                c.result_name = it->second;
        }
        merged.nodes[(size_t)base + n.roots.back()].result_name = next_temporary++;
        for (const auto& rd : st.reads) {
            cnh_ast_node& r = merged.nodes[(size_t)base + n.roots[(size_t)rd.root]];
            // the newest earlier statement that assigned exactly this box supplies the value
            const Done* src = nullptr;
            for (const Done& d : done)
                if (boxes_identical(d.st->out, rd.use))
                    src = &d;
            if (src != nullptr) {
                const cnh_ast_node& set = merged.nodes[(size_t)src->set_root];
                r.operands[rd.slot] = set.operands[1];
                r.has_operand_region[rd.slot] = set.has_operand_region[1];
                r.operand_regions[rd.slot] = set.operand_regions[1];
            } else {
                r.has_operand_region[rd.slot] = 1;
                tag_region(r.operand_regions[rd.slot], number_of(rd.use), st.nd);
            }
        }
        for (int32_t r : n.roots)
            merged.roots.push_back(base + r);
        const int set_root = base + n.roots.back();
        tag_region(merged.nodes[(size_t)set_root].region, number_of(st.out), st.nd);
        // an earlier store into the very same box is dead
        for (const Done& d : done)
            if (boxes_identical(d.st->out, st.out))
                merged.nodes[(size_t)d.set_root].is_temp = 1;
        done.push_back({merged.nodes[(size_t)set_root].operands[1], set_root, &st});
    }

    Group g;
    canonicalise(merged, g);
    cnh_kernel* k = nullptr;
    if (int rc = compile_cached(ex, g, &k))
        return rc;
    int n_in = 0, n_scalar = 0, n_out = 0;
    if (int rc = cnh_kernel_signature(k, &n_in, &n_scalar, &n_out))
        return rc;
    const int nd = run.front().nd;
    const int32_t* cnt = run.front().cnt;
    std::vector<cnh_memref> ins((size_t)std::max(1, n_in)), outs((size_t)std::max(1, n_out));
    std::vector<int32_t> in_block((size_t)std::max(1, n_in), -1);
    for (int i = 0; i < n_in; ++i) {
        int cname = 0, has = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_input(k, i, &cname, &has, &reg))
            return rc;
        CNH_CHECK(has && reg.start[0] >= 0 && reg.start[0] < (int)boxes.size(), -26,
                  "statement run: input %d carries no box number", i);
        ins[(size_t)i] = box_memref(boxes[(size_t)reg.start[0]], nd, cnt);
        if (site != nullptr)
            in_block[(size_t)i] = product_block(*site, boxes[(size_t)reg.start[0]]);
    }
    for (int i = 0; i < n_out; ++i) {
        int rname = 0, tname = 0, is_set = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_output(k, i, &rname, &tname, &is_set, &reg))
            return rc;
        CNH_CHECK(is_set && reg.start[0] >= 0 && reg.start[0] < (int)boxes.size(), -26,
                  "statement run: output %d carries no box number", i);
        outs[(size_t)i] = box_memref(boxes[(size_t)reg.start[0]], nd, cnt);
    }
    std::vector<const void*> scalars((size_t)std::max(1, n_scalar), nullptr);
    for (int i = 0; i < n_scalar; ++i) {
        int cname = 0;
        if (int rc = cnh_kernel_scalar(k, i, &cname))
            return rc;
        XArray* sarr;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &sarr, "broadcast scalar"))
            return rc;
        scalars[(size_t)i] = sarr->tiles[0];
    }
    ex->stats[5]++;
    std::string names;
    for (const Stmt& st : run)
        names += (names.empty() ? "" : ",") + std::to_string(st.out.arr->name);
    if (site != nullptr && !ex->dry) {
        // the product's launch evaluates the run on its tile of sums; shapes it does not take (-17)
        // go out as the two launches below
        const int rc = cnh_launch_product_group(k, &site->job, site->blocks, nd, n_in, ins.data(), in_block.data(),
                                                n_scalar, scalars.data(), 1, n_out, outs.data(), ex->stream);
        if (rc != 0 && rc != -17)
            return rc;
        site->fused = rc == 0;
        if (!site->fused)
            if (int rc2 = cnh_gemm_batch(CNH_F64, 1, &site->job, 1, ex->stream))
                return rc2;
    }
    if (site != nullptr && ex->trace_on)
        ex->log(site->what + (site->fused ? " with_statements" : ""));
    if (ex->trace_on) ex->log("group node=" + std::to_string(merged.id) + " path=statements count=" +
            std::to_string(run.size()) + " inputs=" + std::to_string(n_in) + " outputs=" +
            std::to_string(n_out) + " out=" + names + (site != nullptr && site->fused ? " in_product" : ""));
    if (ex->dry || (site != nullptr && site->fused))
        return 0;
    return cnh_launch_group(k, nd, n_in, ins.data(), n_scalar, scalars.data(), 1, n_out, outs.data(),
                            ex->stream);
}

// Nodes [i, ...) of the message: a run of two or more assignments this pass can merge, deletions
// in between put off until the run has been launched. Returns the number of nodes consumed.
struct StatementRun {
    std::vector<Stmt> run;
    std::vector<int> deletions_kept;   // deletions between the statements taken
    size_t last_stmt_end = 0;          // index behind the last statement taken
    bool ran_off_end = false;          // the message ended while the run could still grow
};
void collect_statement_run(Ex* ex, const std::vector<DagNode>& dag, size_t i, StatementRun& out) {
    std::vector<Stmt>& run = out.run;
    std::vector<int> deletions;
    size_t j = i;
    size_t& last_stmt_end = out.last_stmt_end;
    last_stmt_end = i;
    std::vector<int>& deletions_kept = out.deletions_kept;
    for (; j < dag.size(); ++j) {
        const DagNode& n = dag[j];
        if (n.roots.empty())
            break;
        const cnh_ast_node& root = n.nodes[n.roots.back()];
        if (root.opcode == kOpDelete) {
            if (run.empty())
                break;
            deletions.push_back(root.result_name);
            continue;
        }
        Stmt st;
        if (!analyse_statement(ex, n, st))
            break;
        // an array deleted earlier in the run must not be touched by a later statement
        bool touches_deleted = false;
        for (int name : deletions) {
            touches_deleted = touches_deleted || st.out.arr->name == name;
            for (const auto& rd : st.reads)
                touches_deleted = touches_deleted || rd.use.arr->name == name;
        }
        if (touches_deleted)
            break;
        if (!run.empty() && !can_join(run, st)) {
            // extents that differ by a small factor along one dimension: the wider side in pieces
            std::vector<Stmt> pieces, tried;
            bool joined = false;
            if (run.size() == 1 && cut_statement(run[0], st.cnt, pieces)) {
                tried.assign(1, pieces[0]);
                joined = true;
                for (size_t q = 1; q < pieces.size() && joined; ++q) {
                    joined = can_join(tried, pieces[q]);
                    tried.push_back(pieces[q]);
                }
                joined = joined && can_join(tried, st);
                if (joined) {
                    tried.push_back(st);
                    run.swap(tried);
                }
            } else if (cut_statement(st, run.front().cnt, pieces)) {
                tried = run;
                joined = true;
                for (size_t q = 0; q < pieces.size() && joined; ++q) {
                    joined = can_join(tried, pieces[q]);
                    tried.push_back(pieces[q]);
                }
                if (joined)
                    run.swap(tried);
            }
            if (!joined)
                break;
        } else {
            run.push_back(st);
        }
        last_stmt_end = j + 1;
        deletions_kept = deletions;
    }
    // ran off the end of the message with room left: more of the run may follow
    out.ran_off_end = j == dag.size() && !run.empty() && run.size() < kFuseMaxStmts && open_ended_allowed(ex);
}

int try_statement_run(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    StatementRun sr;
    collect_statement_run(ex, dag, i, sr);
    if (sr.ran_off_end) {
        *open_ended = true;
        return 0;
    }
    if (sr.run.empty())
        return 0;
    if (int rc = exec_statement_run(ex, sr.run))
        return rc;
    for (int name : sr.deletions_kept)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(sr.last_stmt_end - i);
    *used = sr.last_stmt_end - i;
    return 0;
}

// ---- reductions taken by the launch that produces what they reduce ----
//
// `z = f(x, y)` followed by `z @ w`, `sum(z)`, `sum((z - w)^2)` or `max|z - w|` (a CG residual
// update and its r.r, a field and its norms) reads z again once per reduction when every node
// runs on its own. Where the group's result is a new array laid out like its operands (the dense
// path) and the reductions that follow take whole arrays of that layout, the reductions become
// reducing roots of the group (CNH_OP_SUM_OF / CNH_OP_MAXABS_OF): one launch stores z and leaves
// the partial results, one or two small launches fold them.

// Will an array of `shape`, created now, have exactly the tiles of `a`?
bool laid_out_like_new(const Ex* ex, const XArray& a, int nd, const int32_t* shape) {
    if (a.ndims != nd || a.tile != tile_rule(ex, nd, shape) || a.flat != flat_rule(ex, nd, shape, a.tile, nullptr))
        return false;
    for (int d = 0; d < nd; ++d)
        if (a.shape[d] != shape[d] || a.offset[d] % a.tile != 0)
            return false;
    return true;
}

int try_group_with_reductions(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    const DagNode& n = dag[i];
    if (n.roots.empty() || !n.fusible)
        return 0;
    const cnh_ast_node& root = n.nodes[n.roots.back()];
    const bool elementwise = (root.opcode >= CNH_OP_ADD && root.opcode <= CNH_OP_DIV) || root.opcode == CNH_OP_TANH ||
                             root.opcode == CNH_OP_EXP || root.opcode == CNH_OP_COPY;
    if (!elementwise || root.is_temp || root.dtype != CNH_F64)
        return 0;
    for (size_t r = 0; r + 1 < n.roots.size(); ++r)
        if (!n.nodes[n.roots[r]].is_temp)
            return 0;
    int32_t shape[3] = {1, 1, 1};
    {
        // every array the group reads: whole, fp64, laid out as the result will be
        bool any = false;
        for (const cnh_ast_node& a : n.nodes) {
            if (a.opcode != CNH_OP_NOOP || a.is_scalar || a.is_broadcast)
                continue;
            auto it = ex->arrays.find(a.result_name);
            if (it == ex->arrays.end() || it->second.dtype != CNH_F64)
                return 0;
            if (!any)
                for (int d = 0; d < it->second.ndims; ++d)
                    shape[d] = it->second.shape[d];
            any = true;
            if (it->second.ndims != root.ndims || !laid_out_like_new(ex, it->second, root.ndims, shape))
                return 0;
        }
        if (!any)
            return 0;
        for (int32_t r : n.roots) {
            const cnh_ast_node& a = n.nodes[r];
            for (int oi = 0; oi < a.n_operands; ++oi)
                if (a.has_operand_region[oi] && !a.operand_regions[oi].is_global) {
                    const cnh_ast_node& op = n.nodes[a.operands[oi]];
                    auto it = ex->arrays.find(op.result_name);
                    if (it == ex->arrays.end() || !region_is_whole(a.operand_regions[oi], it->second))
                        return 0;
                }
        }
    }
    const int result = root.result_name;

    // the reductions that follow, deletions in between put off until after the launch
    struct Red { const DagNode* node; int op; int other; };      // other: the second array (0: none, -1: the result itself)
    std::vector<Red> reds;
    std::vector<int> deletions, deletions_kept;
    size_t j = i + 1, end = i + 1;
    for (; j < dag.size() && reds.size() < (size_t)kFoldMaxVectors; ++j) {
        const DagNode& m = dag[j];
        if (m.roots.empty())
            break;
        const cnh_ast_node& r = m.nodes[m.roots.back()];
        if (r.opcode == kOpDelete) {
            if (r.result_name == result)
                break;
            deletions.push_back(r.result_name);
            continue;
        }
        const bool paired = r.opcode == CNH_OP_REDUCE || r.opcode == kOpSumsqDiff || r.opcode == kOpMaxabsDiff;
        if (!(paired || r.opcode == kOpSum) || m.roots.size() != 1 || r.n_operands != (paired ? 2 : 1) ||
            r.dtype != CNH_F64)
            break;
        if (r.opcode == CNH_OP_REDUCE && root.ndims != 1)
            break;
        int names[2] = {0, 0};
        bool ok = true;
        for (int oi = 0; oi < r.n_operands && ok; ++oi) {
            const cnh_ast_node& op = m.nodes[r.operands[oi]];
            ok = op.opcode == CNH_OP_NOOP && !op.is_scalar && !op.is_broadcast &&
                 (!r.has_operand_region[oi] || r.operand_regions[oi].is_global);
            names[oi] = op.result_name;
        }
        if (!ok || (names[0] != result && !(paired && names[1] == result)))
            break;
        int other = 0;
        if (paired) {
            const int b = names[0] == result ? names[1] : names[0];
            if (b == result) {
                other = -1;
            } else {
                auto it = ex->arrays.find(b);
                if (it == ex->arrays.end() || it->second.dtype != CNH_F64 ||
                    !laid_out_like_new(ex, it->second, root.ndims, shape) ||
                    std::find(deletions.begin(), deletions.end(), b) != deletions.end())
                    break;
                other = b;
            }
        }
        reds.push_back({&m, r.opcode, other});
        end = j + 1;
        deletions_kept = deletions;
    }
    if (j == dag.size() && reds.size() < (size_t)kFoldMaxVectors && open_ended_allowed(ex)) {
        *open_ended = true;           // the reductions may be in the next message
        return 0;
    }
    if (reds.empty())
        return 0;

    // the group with the reductions as reducing roots
    DagNode merged = n;
    const int value = n.roots.back();
    int next_tmp = 0x7f000000;
    auto leaf_of = [&](int name) {
        for (size_t q = 0; q < merged.nodes.size(); ++q)
            if (merged.nodes[q].opcode == CNH_OP_NOOP && !merged.nodes[q].is_scalar &&
                !merged.nodes[q].is_broadcast && merged.nodes[q].result_name == name)
                return (int)q;
        cnh_ast_node leaf;
        std::memset(&leaf, 0, sizeof leaf);
        leaf.result_name = name;
        leaf.opcode = CNH_OP_NOOP;
        leaf.ndims = root.ndims;
        leaf.dtype = CNH_F64;
        leaf.region.is_global = 1;
        merged.nodes.push_back(leaf);
        return (int)merged.nodes.size() - 1;
    };
    auto add_root = [&](int name, int opcode, bool is_temp, int a, int b) {
        cnh_ast_node r;
        std::memset(&r, 0, sizeof r);
        r.result_name = name;
        r.opcode = opcode;
        r.is_temp = is_temp;
        r.ndims = root.ndims;
        r.dtype = CNH_F64;
        r.n_operands = b >= 0 ? 2 : 1;
        r.operands[0] = a;
        r.operands[1] = b;
        r.region.is_global = 1;
        r.operand_regions[0].is_global = r.operand_regions[1].is_global = 1;
        merged.nodes.push_back(r);
        merged.roots.push_back((int)merged.nodes.size() - 1);
        return (int)merged.nodes.size() - 1;
    };
    for (const Red& rd : reds) {
        const int out_name = rd.node->nodes[rd.node->roots.back()].result_name;
        const int b = rd.other == 0 ? -1 : rd.other == -1 ? value : leaf_of(rd.other);
        if (rd.op == kOpSum) {
            add_root(out_name, CNH_OP_SUM_OF, false, value, -1);
        } else if (rd.op == CNH_OP_REDUCE) {
            const int t = add_root(next_tmp++, CNH_OP_MUL, true, value, b);
            add_root(out_name, CNH_OP_SUM_OF, false, t, -1);
        } else {
            const int d = add_root(next_tmp++, CNH_OP_SUB, true, value, b);
            if (rd.op == kOpSumsqDiff) {
                const int t = add_root(next_tmp++, CNH_OP_MUL, true, d, d);
                add_root(out_name, CNH_OP_SUM_OF, false, t, -1);
            } else {
                add_root(out_name, CNH_OP_MAXABS_OF, false, d, -1);
            }
        }
    }

    Group g;
    canonicalise(merged, g);
    cnh_kernel* k = nullptr;
    if (int rc = compile_cached(ex, g, &k))
        return rc;
    int n_in = 0, n_scalar = 0, n_out = 0;
    if (int rc = cnh_kernel_signature(k, &n_in, &n_scalar, &n_out))
        return rc;
    CNH_CHECK(n_out == 1 + (int)reds.size(), -26, "node %d: %d outputs for %d reductions", n.id, n_out,
              (int)reds.size());
    std::vector<XArray*> in_arr((size_t)n_in);
    for (int q = 0; q < n_in; ++q) {
        int cname = 0, has = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_input(k, q, &cname, &has, &reg))
            return rc;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &in_arr[(size_t)q], "group input"))
            return rc;
    }
    std::vector<const void*> scalars((size_t)std::max(1, n_scalar), nullptr);
    for (int q = 0; q < n_scalar; ++q) {
        int cname = 0;
        if (int rc = cnh_kernel_scalar(k, q, &cname))
            return rc;
        XArray* sarr;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &sarr, "broadcast scalar"))
            return rc;
        CNH_CHECK(sarr->elems == 1 && sarr->dtype == CNH_F64, -27, "node %d: broadcast operand %d", n.id, sarr->name);
        scalars[(size_t)q] = sarr->tiles[0];
    }
    // outputs by name: the group's result first created, then one element per reduction
    std::vector<XArray*> out_arr((size_t)n_out);
    XArray* target = nullptr;
    for (int q = 0; q < n_out; ++q) {
        int rname = 0, tname = 0, is_set = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_output(k, q, &rname, &tname, &is_set, &reg))
            return rc;
        const int actual = g.canon_to_actual[rname];
        if (actual == result) {
            if (int rc = make_array(ex, result, root.ndims, CNH_F64, shape, false, &out_arr[(size_t)q]))
                return rc;
        } else if (int rc = new_scalar_array(ex, actual, CNH_F64, &out_arr[(size_t)q])) {
            return rc;
        }
    }
    // std::map keeps element addresses: the pointers taken above stay valid
    if (int rc = find_array(ex, result, &target, "group result"))
        return rc;
    for (XArray* a : in_arr)
        CNH_CHECK(same_decomposition(*a, *target), -26, "node %d: operand %d is laid out differently", n.id, a->name);
    const int nd = target->ndims;
    const int64_t parts = target->flat ? 1 : target->ntiles;
    std::vector<cnh_memref> in(std::max<size_t>(1, (size_t)parts * n_in)), out((size_t)parts * n_out);
    for (int64_t t = 0; t < parts; ++t) {
        int32_t lo[3], ext[3];
        target->tile_extent(t, lo, ext);
        if (target->flat)
            for (int d = 0; d < nd; ++d)
                ext[d] = target->shape[d];
        auto fill = [&](cnh_memref& m, void* ptr, bool one) {
            std::memset(&m, 0, sizeof m);
            m.allocated = m.aligned = ptr;
            int64_t stride = 1;
            for (int d = nd - 1; d >= 0; --d) {
                m.sizes[d] = one ? 1 : ext[d];
                m.strides[d] = stride;
                stride *= m.sizes[d];
            }
        };
        for (int q = 0; q < n_in; ++q)
            fill(in[(size_t)t * n_in + q], in_arr[(size_t)q]->tiles[t], false);
        for (int q = 0; q < n_out; ++q)
            fill(out[(size_t)t * n_out + q], out_arr[(size_t)q] == target ? target->tiles[t] : out_arr[(size_t)q]->tiles[0],
                 out_arr[(size_t)q] != target);
    }
    ex->stats[5]++;
    if (ex->trace_on) ex->log("group node=" + std::to_string(n.id) + " path=dense+reduce parts=" + std::to_string(parts) +
            " inputs=" + std::to_string(n_in) + " scalars=" + std::to_string(n_scalar) + " reductions=" +
            std::to_string(reds.size()) + " out=" + std::to_string(target->name));
    int rc = 0;
    if (!ex->dry)
        rc = cnh_launch_group_batched(k, nd, (int)parts, n_in, in.data(), n_scalar, scalars.data(), 1, n_out,
                                      out.data(), ex->stream);
    if (rc)
        return rc;
    for (int name : deletions_kept)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(end - i);
    *used = end - i;
    return 0;
}

// ---- partial sums that wait for their consumer ----
//
// A launch that reduces on the way leaves one partial sum per workgroup. Folding them takes a
// launch of its own, and the value is usually wanted by exactly one thing: the next launch, as a
// kernel scalar (alpha = r.r / p.Ap). Such a launch can sum a few hundred partials itself, every
// workgroup in the same order, and store the value on the way. So the result array of a reduction
// may stay "pending": its partials sit in a buffer of their own until a launch takes them
// (pending_done) or something else needs the value (resolve_pending: one small fold launch in the
// same order of additions).
constexpr int64_t kDeferMaxPartials = 1024;

int pending_buffer(Ex* ex, int64_t count, Ex::PendingSum* out) {
    out->count = count;
    out->bytes = (size_t)((count * 8 + 255) & ~(int64_t)255);
    return slab_alloc(ex, out->bytes, false, &out->partials);
}

void pending_done(Ex* ex, int name) {
    auto it = ex->pending.find(name);
    if (it == ex->pending.end())
        return;
    slab_release(ex, it->second.bytes, it->second.partials);
    ex->pending.erase(it);
}

int resolve_pending(Ex* ex, int name) {
    auto it = ex->pending.find(name);
    if (it == ex->pending.end())
        return 0;
    int rc = 0;
    auto arr = ex->arrays.find(name);
    if (arr != ex->arrays.end()) {
        if (ex->trace_on) ex->log("fold " + std::to_string(name) + " partials=" + std::to_string(it->second.count));
        if (!ex->dry)
            rc = cnh_fold_sums(it->second.partials, it->second.count, arr->second.tiles[0], ex->stream);
    }
    pending_done(ex, name);
    return rc;
}

int resolve_all(Ex* ex) {
    while (!ex->pending.empty())
        if (int rc = resolve_pending(ex, ex->pending.begin()->first))
            return rc;
    return 0;
}

// The first node at or after j that is not a deletion; the names deleted on the way go to `dels`.
size_t skip_deletions(const std::vector<DagNode>& dag, size_t j, std::vector<int>& dels) {
    for (; j < dag.size(); ++j) {
        if (dag[j].roots.empty())
            break;
        const cnh_ast_node& r = dag[j].nodes[dag[j].roots.back()];
        if (r.opcode != kOpDelete)
            break;
        dels.push_back(r.result_name);
    }
    return j;
}

bool operand_is_whole(const cnh_ast_node& r, int oi, const int32_t* shape, int nd) {
    if (!r.has_operand_region[oi] || r.operand_regions[oi].is_global)
        return true;
    const cnh_region& g = r.operand_regions[oi];
    if (g.ndims != nd)
        return false;
    for (int d = 0; d < nd; ++d)
        if (g.start[d] != 0 || g.stop[d] != shape[d] || g.step[d] != 1)
            return false;
    return true;
}

cnh_memref dense_memref_of(void* ptr, int nd, const int32_t* shape) {
    cnh_memref m;
    std::memset(&m, 0, sizeof m);
    m.allocated = m.aligned = ptr;
    int64_t stride = 1;
    for (int d = nd - 1; d >= 0; --d) {
        m.sizes[d] = shape[d];
        m.strides[d] = stride;
        stride *= shape[d];
    }
    return m;
}

// ---- a matvec with the vector work of a Krylov iteration around it ----
//
//   [beta = a / b ; p = xa + beta * xb ;]  y = A @ p  [; d = p @ y]
// (examples/cg.py:40-52 upstream: the p update of one iteration, the product and the dot of the
// next) as ONE launch of the matvec that stages its vector in LDS: it forms the vector while it
// stages it, stores it, beta and the numerator's sum on the way, and leaves the partial sums of the
// dot. Deletions between these nodes wait until the launch is out. Applies to whole fp64 matrices
// of 16384 rows or more cut into even tiles of at most 8192 columns; everything else runs node by
// node as before.
struct MatvecSite {
    XArray* A = nullptr;
    int x_name = 0, y_name = 0;
    int64_t rows = 0, cols = 0;
};

bool fusable_matvec(Ex* ex, const DagNode& n, MatvecSite* site) {
    if (n.roots.size() != 1)
        return false;
    const cnh_ast_node& root = n.nodes[n.roots.back()];
    if (root.opcode != CNH_OP_MATMUL || root.n_operands != 2 || root.dtype != CNH_F64)
        return false;
    const cnh_ast_node& oa = n.nodes[root.operands[0]];
    const cnh_ast_node& ox = n.nodes[root.operands[1]];
    if (oa.opcode != CNH_OP_NOOP || oa.is_scalar || ox.opcode != CNH_OP_NOOP || ox.is_scalar)
        return false;
    auto it = ex->arrays.find(oa.result_name);
    if (it == ex->arrays.end())
        return false;
    XArray& A = it->second;
    if (A.ndims != 2 || A.dtype != CNH_F64 || A.flat || A.phased() || A.offset[0] != 0 || A.offset[1] != 0)
        return false;
    if (!operand_is_whole(root, 0, A.shape, 2))
        return false;
    const int32_t xshape[3] = {A.shape[1], 1, 1};
    if (!operand_is_whole(root, 1, xshape, 1))
        return false;
    if (A.shape[0] < 16384 || (int64_t)A.tile * 8 > 65536 || A.tile % 2 != 0 || A.shape[1] % 2 != 0)
        return false;
    site->A = &A;
    site->x_name = ox.result_name;
    site->y_name = root.result_name;
    site->rows = A.shape[0];
    site->cols = A.shape[1];
    return true;
}

bool vector_f64(const Ex* ex, int name, int64_t len, const XArray** out) {
    auto it = ex->arrays.find(name);
    if (it == ex->arrays.end() || it->second.ndims != 1 || it->second.dtype != CNH_F64 ||
        it->second.shape[0] != len || it->second.offset[0] != 0)
        return false;
    *out = &it->second;
    return true;
}

int try_fused_matvec(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    if (dag[i].roots.empty())
        return 0;
    std::vector<int> dels, dels_kept;
    size_t at = i;
    // the prologue, if the run starts with one
    bool form = false;
    int beta_name = 0, num_name = 0, den_name = 0, xa_name = 0, xb_name = 0, p_name = 0;
    {
        const DagNode& s = dag[i];
        const cnh_ast_node& r = s.nodes[s.roots.back()];
        if (r.opcode == CNH_OP_DIV && s.roots.size() == 1 && s.fusible && !r.is_temp && r.dtype == CNH_F64 &&
            r.n_operands == 2) {
            const cnh_ast_node& a = s.nodes[r.operands[0]];
            const cnh_ast_node& b = s.nodes[r.operands[1]];
            auto one = [&](const cnh_ast_node& op) {
                if (op.opcode != CNH_OP_NOOP || op.is_scalar)
                    return false;
                auto it = ex->arrays.find(op.result_name);
                return it != ex->arrays.end() && it->second.elems == 1 && it->second.dtype == CNH_F64;
            };
            if (!one(a) || !one(b) || a.result_name == b.result_name)
                return 0;
            beta_name = r.result_name;
            num_name = a.result_name;
            den_name = b.result_name;
            size_t j = skip_deletions(dag, i + 1, dels);
            if (j == dag.size()) {
                *open_ended = open_ended_allowed(ex);
                return 0;
            }
            const DagNode& v = dag[j];
            if (v.roots.size() != 2 || !v.fusible)
                return 0;
            const cnh_ast_node& t = v.nodes[v.roots[0]];
            const cnh_ast_node& sum = v.nodes[v.roots[1]];
            if (t.opcode != CNH_OP_MUL || !t.is_temp || t.n_operands != 2 || sum.opcode != CNH_OP_ADD || sum.is_temp ||
                sum.n_operands != 2 || sum.dtype != CNH_F64)
                return 0;
            // t = beta * xb, either way round
            int which_b = -1;
            for (int oi = 0; oi < 2; ++oi) {
                const cnh_ast_node& op = v.nodes[t.operands[oi]];
                if (op.opcode == CNH_OP_NOOP && !op.is_scalar && op.is_broadcast && op.result_name == beta_name)
                    which_b = oi;
            }
            if (which_b < 0)
                return 0;
            const cnh_ast_node& xb = v.nodes[t.operands[1 - which_b]];
            if (xb.opcode != CNH_OP_NOOP || xb.is_scalar || xb.is_broadcast)
                return 0;
            // p = xa + t, either way round
            int which_t = -1;
            for (int oi = 0; oi < 2; ++oi) {
                const cnh_ast_node& op = v.nodes[sum.operands[oi]];
                if (sum.operands[oi] == v.roots[0] || (!op.is_scalar && op.result_name == t.result_name))
                    which_t = oi;
            }
            if (which_t < 0)
                return 0;
            const cnh_ast_node& xa = v.nodes[sum.operands[1 - which_t]];
            if (xa.opcode != CNH_OP_NOOP || xa.is_scalar || xa.is_broadcast)
                return 0;
            xa_name = xa.result_name;
            xb_name = xb.result_name;
            p_name = sum.result_name;
            const XArray *pa = nullptr, *pb = nullptr;
            auto ita = ex->arrays.find(xa_name);
            if (ita == ex->arrays.end() || !vector_f64(ex, xa_name, ita->second.shape[0], &pa) ||
                !vector_f64(ex, xb_name, pa->shape[0], &pb))
                return 0;
            const int32_t vshape[3] = {pa->shape[0], 1, 1};
            if (!operand_is_whole(t, 1 - which_b, vshape, 1) || !operand_is_whole(sum, 1 - which_t, vshape, 1))
                return 0;
            at = skip_deletions(dag, j + 1, dels);
            if (at == dag.size()) {
                *open_ended = open_ended_allowed(ex);
                return 0;
            }
            form = true;
        }
    }
    MatvecSite mv;
    if (!fusable_matvec(ex, dag[at], &mv))
        return 0;
    const XArray *xa = nullptr, *xb = nullptr, *xv = nullptr;
    if (form) {
        if (mv.x_name != p_name || mv.rows != mv.cols || !vector_f64(ex, xa_name, mv.cols, &xa) ||
            !vector_f64(ex, xb_name, mv.cols, &xb))
            return 0;
    } else if (!vector_f64(ex, mv.x_name, mv.cols, &xv)) {
        return 0;
    }
    dels_kept = dels;
    size_t end = at + 1;
    // the dot of the vector with the product
    int dot_name = 0;
    {
        size_t k = skip_deletions(dag, at + 1, dels);
        if (k == dag.size() && open_ended_allowed(ex)) {
            *open_ended = true;
            return 0;
        }
        if (k < dag.size() && dag[k].roots.size() == 1) {
            const cnh_ast_node& r = dag[k].nodes[dag[k].roots.back()];
            if (r.opcode == CNH_OP_REDUCE && r.n_operands == 2 && r.dtype == CNH_F64) {
                const cnh_ast_node& a = dag[k].nodes[r.operands[0]];
                const cnh_ast_node& b = dag[k].nodes[r.operands[1]];
                const int32_t xs[3] = {(int32_t)mv.cols, 1, 1}, ys[3] = {(int32_t)mv.rows, 1, 1};
                const bool xy = a.result_name == mv.x_name && b.result_name == mv.y_name &&
                                operand_is_whole(r, 0, xs, 1) && operand_is_whole(r, 1, ys, 1);
                const bool yx = a.result_name == mv.y_name && b.result_name == mv.x_name &&
                                operand_is_whole(r, 0, ys, 1) && operand_is_whole(r, 1, xs, 1);
                if (mv.rows == mv.cols && a.opcode == CNH_OP_NOOP && b.opcode == CNH_OP_NOOP && !a.is_scalar &&
                    !b.is_scalar && (xy || yx)) {
                    dot_name = r.result_name;
                    end = k + 1;
                    dels_kept = dels;
                }
            }
        }
    }
    if (!form && dot_name == 0)
        return 0;                      // nothing to take along: the plain node does the same

    // from here on the nodes [i, end) are this launch
    const int32_t yshape[3] = {(int32_t)mv.rows, 1, 1}, xshape[3] = {(int32_t)mv.cols, 1, 1};
    XArray *y = nullptr, *p = nullptr, *beta = nullptr, *dot = nullptr;
    cnh_gemv_fusion fu;
    std::memset(&fu, 0, sizeof fu);
    bool num_was_pending = false;
    if (form) {
        if (int rc = resolve_pending(ex, den_name))
            return rc;
        if (int rc = make_array(ex, p_name, 1, CNH_F64, xshape, false, &p))
            return rc;
        if (int rc = new_scalar_array(ex, beta_name, CNH_F64, &beta))
            return rc;
        XArray *num = nullptr, *den = nullptr;
        if (int rc = find_array(ex, num_name, &num, "matvec numerator"))
            return rc;
        if (int rc = find_array(ex, den_name, &den, "matvec denominator"))
            return rc;
        fu.xa = xa->tiles[0];
        fu.xb = xb->tiles[0];
        auto pend = ex->pending.find(num_name);
        if (pend != ex->pending.end()) {
            fu.num = pend->second.partials;
            fu.num_count = pend->second.count;
            fu.num_folded = num->tiles[0];
            num_was_pending = true;
        } else {
            fu.num = num->tiles[0];
            fu.num_count = 1;
        }
        fu.den = den->tiles[0];
        fu.quotient_out = beta->tiles[0];
    }
    if (int rc = make_array(ex, mv.y_name, 1, CNH_F64, yshape, false, &y))
        return rc;
    void* xptr = form ? p->tiles[0] : const_cast<XArray*>(xv)->tiles[0];
    Ex::PendingSum dot_sums;
    const int64_t nb = (mv.rows + 63) / 64;
    if (dot_name != 0) {
        if (int rc = new_scalar_array(ex, dot_name, CNH_F64, &dot))
            return rc;
        if (int rc = pending_buffer(ex, nb, &dot_sums))
            return rc;
        fu.w = xptr;
        fu.dot_partials = dot_sums.partials;
        fu.dot_capacity = nb;
    }
    if (ex->trace_on) ex->log("matmul A=" + std::to_string(mv.A->name) + " tiles=" + std::to_string(mv.A->ntiles) + " x=" +
            std::to_string(mv.x_name) + " out=" + std::to_string(mv.y_name) + " fused" +
            (form ? " vector=" + std::to_string(xa_name) + "+(" + std::to_string(num_name) + "/" +
                        std::to_string(den_name) + ")*" + std::to_string(xb_name)
                  : std::string()) +
            (dot_name ? " dot=" + std::to_string(dot_name) : std::string()));
    int rc = 0;
    if (!ex->dry) {
        cnh_event t0 = matvec_timer_start(ex);
        rc = cnh_gemv_tiles_fused(mv.rows, mv.cols, mv.A->tile, mv.A->tiles.data(), xptr, y->tiles[0], &fu, nullptr,
                                  ex->stream);
        matvec_timer_stop(ex, t0);
    }
    if (rc)
        return rc;
    if (num_was_pending)
        pending_done(ex, num_name);
    if (dot_name != 0) {
        ex->pending[dot_name] = dot_sums;
        if (nb > kDeferMaxPartials)
            if (int rc2 = resolve_pending(ex, dot_name))
                return rc2;
    }
    for (int name : dels_kept)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(end - i);
    ex->stats[5]++;
    *used = end - i;
    return 0;
}

// ---- dense statements, the scalars between them and the reductions behind them as one launch ----
//
//   alpha = rr / pAp ; x2 = x + alpha * p ; r2 = r - alpha * Ap ; rr2 = r2 @ r2
// Statements that make new arrays of one shape from whole arrays laid out alike (the no-region fast
// path, src/execute_node.cpp:1263-1336 upstream), statements on one-element arrays (which upstream
// runs as kernels of their own, src/executor_core.cpp:390-605) and reductions of the new arrays
// become ONE group with several roots: a scalar statement is formed in registers by every lane and
// stored once (CNH_OP_SCALAR_OF), later statements read earlier results from registers, the
// reductions leave partial sums that wait for their consumer. A run ends before the first statement
// that needs the value of one of its own reductions. One partition only (a 1-D array up to the
// minimum tile, an array with a single tile, a rank-3 block).
constexpr size_t kRunMaxStatements = 8;

int try_dense_run(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    struct RunStmt { const DagNode* n; bool scalar; };
    struct RunRed { const DagNode* n; int op; int a, b; };
    std::vector<RunStmt> stmts;
    std::vector<RunRed> reds;
    std::set<int> vec_results, scal_results, red_results;
    std::vector<int> deletions, deletions_kept;
    int32_t shape[3] = {1, 1, 1};
    int nd = 0;
    bool reads_pending = false;
    size_t n_vec = 0, end = i, j = i;

    auto is_deleted = [&](int name) { return std::find(deletions.begin(), deletions.end(), name) != deletions.end(); };
    // 0: not part of a run; 1: scalar statement; 2: vector statement
    auto classify = [&](const DagNode& m) -> int {
        if (!m.fusible || m.roots.empty())
            return 0;
        const cnh_ast_node& root = m.nodes[m.roots.back()];
        const bool arith = root.opcode >= CNH_OP_ADD && root.opcode <= CNH_OP_DIV;
        if (!(arith || root.opcode == CNH_OP_TANH || root.opcode == CNH_OP_EXP || root.opcode == CNH_OP_COPY) ||
            root.is_temp || root.dtype != CNH_F64)
            return 0;
        std::set<int> own;
        bool only_arith = true;
        for (size_t r = 0; r < m.roots.size(); ++r) {
            const cnh_ast_node& a = m.nodes[m.roots[r]];
            if ((r + 1 < m.roots.size()) != (a.is_temp != 0) || a.dtype != CNH_F64)
                return 0;
            own.insert(a.result_name);
            only_arith = only_arith && a.opcode >= CNH_OP_ADD && a.opcode <= CNH_OP_DIV;
        }
        bool any_vector = false, plain_scalar_operand = false;
        int32_t shp[3] = {shape[0], shape[1], shape[2]};
        int rank = nd;
        for (int32_t ri : m.roots) {
            const cnh_ast_node& a = m.nodes[ri];
            for (int oi = 0; oi < a.n_operands; ++oi) {
                if (a.operands[oi] < 0 || a.operands[oi] >= (int)m.nodes.size())
                    return 0;
                const cnh_ast_node& op = m.nodes[a.operands[oi]];
                if (op.is_scalar)
                    continue;
                if (own.count(op.result_name))
                    continue;                                  // another root of this statement
                if (op.opcode != CNH_OP_NOOP)
                    return 0;
                const int name = op.result_name;
                if (red_results.count(name) || is_deleted(name))
                    return 0;
                if (scal_results.count(name)) {
                    plain_scalar_operand = plain_scalar_operand || !op.is_broadcast;
                    continue;
                }
                if (vec_results.count(name)) {
                    if (op.is_broadcast || !operand_is_whole(a, oi, shape, nd))
                        return 0;
                    any_vector = true;
                    continue;
                }
                auto it = ex->arrays.find(name);
                if (it == ex->arrays.end() || it->second.dtype != CNH_F64)
                    return 0;
                const XArray& arr = it->second;
                if (arr.elems == 1) {
                    plain_scalar_operand = plain_scalar_operand || !op.is_broadcast;
                    continue;
                }
                if (op.is_broadcast)
                    return 0;
                if (rank == 0) {
                    rank = arr.ndims;
                    for (int d = 0; d < 3; ++d)
                        shp[d] = d < arr.ndims ? arr.shape[d] : 1;
                }
                if (arr.ndims != rank || !laid_out_like_new(ex, arr, rank, shp) || !(arr.flat || arr.ntiles == 1) ||
                    !operand_is_whole(a, oi, shp, rank))
                    return 0;
                any_vector = true;
            }
        }
        if (!any_vector)
            return only_arith ? 1 : 0;             // exp and tanh of a scalar have no generated form
        if (plain_scalar_operand || root.ndims != rank)
            return 0;
        if (!root.region.is_global) {              // a result region, where given, spells the same shape
            if (root.region.ndims != rank)
                return 0;
            for (int d = 0; d < rank; ++d)
                if (region_count(root.region, d) != shp[d])
                    return 0;
        }
        nd = rank;
        for (int d = 0; d < 3; ++d)
            shape[d] = shp[d];
        return 2;
    };

    for (; j < dag.size(); ++j) {
        const DagNode& m = dag[j];
        if (m.roots.empty())
            break;
        const cnh_ast_node& root = m.nodes[m.roots.back()];
        if (root.opcode == kOpDelete) {
            const int name = root.result_name;
            if (stmts.empty() || vec_results.count(name) || scal_results.count(name) || red_results.count(name))
                break;
            deletions.push_back(name);
            continue;
        }
        const bool paired = root.opcode == CNH_OP_REDUCE || root.opcode == kOpSumsqDiff || root.opcode == kOpMaxabsDiff;
        if (paired || root.opcode == kOpSum) {
            if (n_vec == 0 || reds.size() >= (size_t)kFoldMaxVectors || m.roots.size() != 1 ||
                root.n_operands != (paired ? 2 : 1) || root.dtype != CNH_F64 ||
                (root.opcode == CNH_OP_REDUCE && nd != 1))
                break;
            int names[2] = {0, 0};
            bool ok = true, from_run = false;
            for (int oi = 0; oi < root.n_operands && ok; ++oi) {
                const cnh_ast_node& op = m.nodes[root.operands[oi]];
                ok = op.opcode == CNH_OP_NOOP && !op.is_scalar && !op.is_broadcast && operand_is_whole(root, oi, shape, nd) &&
                     !is_deleted(op.result_name);
                names[oi] = op.result_name;
                if (!ok)
                    break;
                if (vec_results.count(op.result_name)) {
                    from_run = true;
                } else {
                    auto it = ex->arrays.find(op.result_name);
                    ok = it != ex->arrays.end() && it->second.dtype == CNH_F64 && it->second.ndims == nd &&
                         laid_out_like_new(ex, it->second, nd, shape) && (it->second.flat || it->second.ntiles == 1);
                }
            }
            if (!ok || !from_run)
                break;
            reds.push_back({&m, root.opcode, names[0], names[1]});
            red_results.insert(root.result_name);
        } else {
            if (stmts.size() >= kRunMaxStatements)
                break;
            const int kind = classify(m);
            if (kind == 0)
                break;
            stmts.push_back({&m, kind == 1});
            (kind == 1 ? scal_results : vec_results).insert(root.result_name);
            n_vec += kind == 2;
            // does it read a value that still stands as partial sums?
            for (const cnh_ast_node& a : m.nodes)
                if (a.opcode == CNH_OP_NOOP && !a.is_scalar && ex->pending.count(a.result_name))
                    reads_pending = true;
        }
        end = j + 1;
        deletions_kept = deletions;
    }
    if (j == dag.size() && !stmts.empty() && stmts.size() < kRunMaxStatements && open_ended_allowed(ex)) {
        *open_ended = true;            // the run may go on in the next message
        return 0;
    }
    if (n_vec == 0 || !(stmts.size() >= 2 || reads_pending))
        return 0;
    // ---- the run as one group ----
    DagNode merged;
    merged.id = dag[i].id;
    merged.fusible = 1;
    std::map<int, int> produced;                 // result name -> node of `merged` that holds the value
    int next_literal = -1, next_temporary = 0x7d000000;
    auto whole = [](cnh_region& r) {
        std::memset(&r, 0, sizeof r);
        r.is_global = 1;
    };
    for (const RunStmt& st : stmts) {
        const DagNode& n = *st.n;
        const int base = (int)merged.nodes.size();
        for (const cnh_ast_node& a : n.nodes) {
            merged.nodes.push_back(a);
            cnh_ast_node& c = merged.nodes.back();
            for (int oi = 0; oi < c.n_operands; ++oi)
                if (c.operands[oi] >= 0)
                    c.operands[oi] += base;
            if (c.is_scalar)
                c.result_name = next_literal--;
        }
        std::map<int, int> renamed;
        for (size_t ri = 0; ri + 1 < n.roots.size(); ++ri)
            renamed[n.nodes[(size_t)n.roots[ri]].result_name] = next_temporary++;
        for (size_t q = (size_t)base; q < merged.nodes.size(); ++q) {
            cnh_ast_node& c = merged.nodes[q];
            if (c.is_scalar)
                continue;
            auto it = renamed.find(c.result_name);
            if (it != renamed.end())
                c.result_name = it->second;
        }
        for (size_t q = (size_t)base; q < merged.nodes.size(); ++q) {
            cnh_ast_node& c = merged.nodes[q];
            if (c.is_scalar || c.opcode == CNH_OP_NOOP)
                continue;
            for (int oi = 0; oi < c.n_operands; ++oi) {
                if (c.operands[oi] < 0)
                    continue;
                const cnh_ast_node& op = merged.nodes[(size_t)c.operands[oi]];
                if (op.is_scalar || op.opcode != CNH_OP_NOOP)
                    continue;
                auto pr = produced.find(op.result_name);
                if (pr != produced.end()) {      // made earlier in this launch: the value is in registers
                    c.operands[oi] = pr->second;
                    c.has_operand_region[oi] = 0;
                    whole(c.operand_regions[oi]);
                }
            }
        }
        // one-element arrays are kernel scalars here
        for (size_t q = (size_t)base; q < merged.nodes.size(); ++q) {
            cnh_ast_node& c = merged.nodes[q];
            if (c.opcode != CNH_OP_NOOP || c.is_scalar || c.is_broadcast)
                continue;
            auto it = ex->arrays.find(c.result_name);
            if (it != ex->arrays.end() && it->second.elems == 1)
                c.is_broadcast = 1;
        }
        for (int32_t r : n.roots)
            merged.roots.push_back(base + r);
        const int last = base + n.roots.back();
        const int actual = merged.nodes[(size_t)last].result_name;
        produced[actual] = last;
        if (st.scalar) {
            merged.nodes[(size_t)last].is_temp = 1;
            merged.nodes[(size_t)last].result_name = next_temporary++;
            cnh_ast_node once;
            std::memset(&once, 0, sizeof once);
            once.result_name = actual;
            once.opcode = CNH_OP_SCALAR_OF;
            once.ndims = nd;
            once.dtype = CNH_F64;
            once.n_operands = 1;
            once.operands[0] = last;
            once.operands[1] = -1;
            whole(once.region);
            whole(once.operand_regions[0]);
            whole(once.operand_regions[1]);
            merged.nodes.push_back(once);
            merged.roots.push_back((int)merged.nodes.size() - 1);
        }
    }
    auto value_of = [&](int name) {
        auto pr = produced.find(name);
        if (pr != produced.end())
            return pr->second;
        for (size_t q = 0; q < merged.nodes.size(); ++q)
            if (merged.nodes[q].opcode == CNH_OP_NOOP && !merged.nodes[q].is_scalar && !merged.nodes[q].is_broadcast &&
                merged.nodes[q].result_name == name)
                return (int)q;
        cnh_ast_node leaf;
        std::memset(&leaf, 0, sizeof leaf);
        leaf.result_name = name;
        leaf.opcode = CNH_OP_NOOP;
        leaf.ndims = nd;
        leaf.dtype = CNH_F64;
        whole(leaf.region);
        whole(leaf.operand_regions[0]);
        whole(leaf.operand_regions[1]);
        merged.nodes.push_back(leaf);
        return (int)merged.nodes.size() - 1;
    };
    auto add_root = [&](int name, int opcode, bool is_temp, int a, int b) {
        cnh_ast_node r;
        std::memset(&r, 0, sizeof r);
        r.result_name = name;
        r.opcode = opcode;
        r.is_temp = is_temp;
        r.ndims = nd;
        r.dtype = CNH_F64;
        r.n_operands = b >= 0 ? 2 : 1;
        r.operands[0] = a;
        r.operands[1] = b;
        whole(r.region);
        whole(r.operand_regions[0]);
        whole(r.operand_regions[1]);
        merged.nodes.push_back(r);
        merged.roots.push_back((int)merged.nodes.size() - 1);
        return (int)merged.nodes.size() - 1;
    };
    std::map<int, bool> red_is_sum;
    for (const RunRed& rd : reds) {
        const int out_name = rd.n->nodes[rd.n->roots.back()].result_name;
        const int a = value_of(rd.a);
        red_is_sum[out_name] = rd.op != kOpMaxabsDiff;
        if (rd.op == kOpSum) {
            add_root(out_name, CNH_OP_SUM_OF, false, a, -1);
            continue;
        }
        const int b = value_of(rd.b);
        if (rd.op == CNH_OP_REDUCE) {
            const int t = add_root(next_temporary++, CNH_OP_MUL, true, a, b);
            add_root(out_name, CNH_OP_SUM_OF, false, t, -1);
        } else {
            const int d = add_root(next_temporary++, CNH_OP_SUB, true, a, b);
            if (rd.op == kOpSumsqDiff) {
                const int t = add_root(next_temporary++, CNH_OP_MUL, true, d, d);
                add_root(out_name, CNH_OP_SUM_OF, false, t, -1);
            } else {
                add_root(out_name, CNH_OP_MAXABS_OF, false, d, -1);
            }
        }
    }
    merged.nodes[(size_t)merged.roots.back()].ndims = nd;

    Group g;
    canonicalise(merged, g);
    cnh_kernel* k = nullptr;
    if (int rc = compile_cached(ex, g, &k))
        return rc;
    int n_in = 0, n_scalar = 0, n_out = 0;
    if (int rc = cnh_kernel_signature(k, &n_in, &n_scalar, &n_out))
        return rc;
    int64_t elems = 1;
    for (int d = 0; d < nd; ++d)
        elems *= shape[d];
    std::vector<cnh_memref> in((size_t)std::max(1, n_in)), out((size_t)std::max(1, n_out));
    for (int q = 0; q < n_in; ++q) {
        int cname = 0, has = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_input(k, q, &cname, &has, &reg))
            return rc;
        XArray* a;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &a, "group input"))
            return rc;
        CNH_CHECK(a->elems == elems && (a->flat || a->ntiles == 1), -26, "node %d: operand %d is laid out differently",
                  merged.id, a->name);
        in[(size_t)q] = dense_memref_of(a->flat ? a->slab : a->tiles[0], nd, shape);
    }
    std::vector<cnh_scalar_sum> sums((size_t)std::max(1, n_scalar));
    std::vector<const void*> scalar_ptrs((size_t)std::max(1, n_scalar), nullptr);
    std::vector<int> taken;                    // pending sums this launch folds and stores
    for (int q = 0; q < n_scalar; ++q) {
        int cname = 0;
        if (int rc = cnh_kernel_scalar(k, q, &cname))
            return rc;
        XArray* sarr;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &sarr, "kernel scalar"))
            return rc;
        CNH_CHECK(sarr->elems == 1 && sarr->dtype == CNH_F64, -27, "node %d: kernel scalar %d", merged.id, sarr->name);
        auto pend = ex->pending.find(sarr->name);
        if (pend != ex->pending.end()) {
            sums[(size_t)q] = cnh_scalar_sum{pend->second.partials, pend->second.count, sarr->tiles[0]};
            taken.push_back(sarr->name);
        } else {
            sums[(size_t)q] = cnh_scalar_sum{sarr->tiles[0], 1, nullptr};
        }
        scalar_ptrs[(size_t)q] = sarr->tiles[0];
    }
    // a launch that reduces, or that sums partials on the way in, runs 256 lanes a workgroup and
    // leaves one partial per workgroup: per 512 elements
    const int64_t nslots = (elems + 511) / 512;
    std::map<int, Ex::PendingSum> left;
    const int32_t one[3] = {1, 1, 1};
    std::string out_names;
    for (int q = 0; q < n_out; ++q) {
        int rname = 0, tname = 0, is_set = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_output(k, q, &rname, &tname, &is_set, &reg))
            return rc;
        const int actual = g.canon_to_actual[rname];
        XArray* o = nullptr;
        if (vec_results.count(actual)) {
            if (int rc = make_array(ex, actual, nd, CNH_F64, shape, false, &o))
                return rc;
            CNH_CHECK(o->flat || o->ntiles == 1, -26, "node %d: result %d has several tiles", merged.id, actual);
            out[(size_t)q] = dense_memref_of(o->flat ? o->slab : o->tiles[0], nd, shape);
            out_names += (out_names.empty() ? "" : ",") + std::to_string(actual);
            continue;
        }
        if (int rc = new_scalar_array(ex, actual, CNH_F64, &o))
            return rc;
        out[(size_t)q] = dense_memref_of(o->tiles[0], nd, one);
        if (red_results.count(actual) && red_is_sum[actual] && nslots > 1 && nslots <= kDeferMaxPartials) {
            Ex::PendingSum ps;
            if (int rc = pending_buffer(ex, nslots, &ps))
                return rc;
            int32_t room[3] = {1, 1, 1};
            room[nd - 1] = (int32_t)nslots;
            out[(size_t)q] = dense_memref_of(ps.partials, nd, room);
            left[actual] = ps;
        }
    }
    ex->stats[5]++;
    if (ex->trace_on) ex->log("group node=" + std::to_string(merged.id) + " path=run statements=" + std::to_string(stmts.size()) +
            " scalars_formed=" + std::to_string(scal_results.size()) + " reductions=" + std::to_string(reds.size()) +
            " inputs=" + std::to_string(n_in) + " scalars=" + std::to_string(n_scalar) + " sums_taken=" +
            std::to_string(taken.size()) + " out=" + out_names);
    int rc = 0;
    if (!ex->dry) {
        if (!taken.empty())
            rc = cnh_launch_group_sums(k, nd, n_in, in.data(), n_scalar, sums.data(), n_out, out.data(), ex->stream);
        else
            rc = cnh_launch_group(k, nd, n_in, in.data(), n_scalar, scalar_ptrs.data(), 1, n_out, out.data(),
                                  ex->stream);
    }
    if (rc)
        return rc;
    for (int name : taken)
        pending_done(ex, name);
    for (auto& kv : left)
        ex->pending[kv.first] = kv.second;
    for (int name : deletions_kept)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(end - i);
    *used = end - i;
    return 0;
}

// ---- two lattices of one colour as one sweep ----
//
// A red-black sweep (examples/gauss_seidel.py upstream) updates each colour with two statements,
//   phi[1:-1:2, 1:-1:2] = f(neighbours, g[1:-1:2, 1:-1:2]);  phi[2:-1:2, 2:-1:2] = f(...)
// which read only points of the other colour: neither reads what the other assigns. Run one by one
// each is a pass of its own over all of phi's cache lines. Together they are one pass: a group with
// two SET_REGION roots, launched as a register-window sweep that evaluates both at every point and
// stores whichever lattice the point belongs to, in place. That sweep works on arrays stored as one
// row-major block, so arrays still cut into tiles with buffers of their own are laid out anew
// first (once: they stay that way).

// Stores `a` as one row-major block (tiles become views into it).
int make_block(Ex* ex, XArray& a) {
    if (a.flat)
        return 0;
    CNH_CHECK(!a.phased(), -26, "array %d: tiles that do not start at element 0", a.name);
    const int esz = dtype_size(a.dtype), nd = a.ndims;
    const size_t bytes = (size_t)std::max<int64_t>(((int64_t)a.elems * esz + 255) & ~(int64_t)255, 256);
    void* block = nullptr;
    if (int rc = slab_alloc(ex, bytes, false, &block))
        return rc;
    int64_t pitch[3] = {0, 0, 0};
    {
        int64_t run = 1;
        for (int d = nd - 1; d >= 0; --d) {
            pitch[d] = run;
            run *= a.shape[d];
        }
    }
    std::vector<int64_t> offs;
    for (int64_t t = 0; t < a.ntiles; ++t) {
        int32_t lo[3], ext[3];
        a.tile_extent(t, lo, ext);
        int64_t sstr[3], zero[3] = {0, 0, 0}, one[3] = {1, 1, 1}, counts[3] = {1, 1, 1}, off = 0;
        a.tile_strides(ext, sstr);
        for (int d = 0; d < nd; ++d) {
            counts[d] = ext[d];
            off += lo[d] * pitch[d];
        }
        offs.push_back(off * esz);
        if (!ex->dry)
            if (int rc = cnh_copy_region(nd, esz, static_cast<char*>(block) + off * esz, pitch, zero, one, a.tiles[(size_t)t],
                                         sstr, zero, one, counts, ex->stream))
                return rc;
    }
    slab_release(ex, a.bytes, a.slab);
    slab_release(ex, a.bytes, a.alt);
    a.slab = block;
    a.alt = nullptr;
    a.alt_tiles.clear();
    a.bytes = bytes;
    a.flat = true;
    for (int d = 0; d < 3; ++d)
        a.pitch[d] = d < nd ? pitch[d] : 0;
    a.tile_off = offs;
    for (int64_t t = 0; t < a.ntiles; ++t)
        a.tiles[(size_t)t] = static_cast<char*>(block) + offs[(size_t)t];
    if (ex->trace_on) ex->log("block " + std::to_string(a.name) + " tiles=" + std::to_string(a.ntiles));
    return 0;
}

// `target[lattice] = f(...)` with steps of 1 or 2, at least one of them 2, on an array of rank 2 or 3.
bool lattice_statement(Ex* ex, const DagNode& n, XArray** target, const cnh_ast_node** set) {
    if (!n.fusible || n.roots.empty())
        return false;
    const cnh_ast_node& root = n.nodes[n.roots.back()];
    if (root.opcode != CNH_OP_SET_REGION || root.n_operands != 2 || root.region.is_global ||
        n.nodes[root.operands[1]].is_scalar)
        return false;
    for (size_t r = 0; r + 1 < n.roots.size(); ++r)
        if (!n.nodes[n.roots[r]].is_temp)
            return false;
    auto it = ex->arrays.find(n.nodes[root.operands[0]].result_name);
    if (it == ex->arrays.end() || it->second.ndims < 2 || it->second.ndims != root.region.ndims)
        return false;
    bool stepped = false;
    for (int d = 0; d < root.region.ndims; ++d) {
        if (root.region.step[d] != 1 && root.region.step[d] != 2)
            return false;
        stepped = stepped || root.region.step[d] == 2;
    }
    *target = &it->second;
    *set = &root;
    return stepped;
}

// One group out of several statements: the roots of the first, then those of the next, and so on.
// Literals and temporaries get names of their own per statement; every statement's SET_REGION
// root becomes an output.
void merge_statements(const std::vector<const DagNode*>& parts, DagNode& merged) {
    merged.id = parts.front()->id;
    merged.fusible = 1;
    int next_literal = -1, next_temporary = 0x7c000000;
    for (const DagNode* n : parts) {
        const int base = (int)merged.nodes.size();
        for (const cnh_ast_node& a : n->nodes) {
            merged.nodes.push_back(a);
            cnh_ast_node& c = merged.nodes.back();
            for (int oi = 0; oi < c.n_operands; ++oi)
                if (c.operands[oi] >= 0)
                    c.operands[oi] += base;
            if (c.is_scalar)
                c.result_name = next_literal--;
        }
        std::map<int, int> renamed;
        for (size_t ri = 0; ri + 1 < n->roots.size(); ++ri)
            renamed[n->nodes[(size_t)n->roots[ri]].result_name] = next_temporary++;
        for (size_t q = (size_t)base; q < merged.nodes.size(); ++q) {
            cnh_ast_node& c = merged.nodes[q];
            auto it = c.is_scalar ? renamed.end() : renamed.find(c.result_name);
            if (it != renamed.end())
                c.result_name = it->second;
        }
        merged.nodes[(size_t)base + (size_t)n->roots.back()].result_name = next_temporary++;
        for (int32_t r : n->roots)
            merged.roots.push_back(base + r);
    }
}

// Does a statement read array `name` (other than as the array it assigns into)?
bool statement_reads(const DagNode& n, int name) {
    for (int32_t ri : n.roots) {
        const cnh_ast_node& r = n.nodes[(size_t)ri];
        for (int oi = 0; oi < r.n_operands; ++oi) {
            if (r.opcode == CNH_OP_SET_REGION && oi == 0)
                continue;
            if (r.operands[oi] < 0 || r.operands[oi] >= (int)n.nodes.size())
                return true;
            const cnh_ast_node& op = n.nodes[(size_t)r.operands[oi]];
            if (!op.is_scalar && op.result_name == name)
                return true;
        }
    }
    return false;
}

// ---- interleaved lattices of one array assigned from other arrays, as one launch ----
//
// The prolongation of examples/multigrid2d.py upstream fills a fine grid with four statements,
//   e[2:-2:2, 2:-2:2] = c[1:-1, 1:-1];  e[1:-1:2, 2:-2:2] = 0.5 * (c[:-1, 1:-1] + c[1:, 1:-1]);  ...
// each a pass over all of e's cache lines that writes a quarter of every line. None of them reads
// e and their lattices share no point, so up to four of them run as one launch that reads the
// coarse array once and stores all four lattices, in place, over arrays stored as one block each.
int try_scatter_run(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    XArray* ta = nullptr;
    const cnh_ast_node* sa = nullptr;
    if (!lattice_statement(ex, dag[i], &ta, &sa) || statement_reads(dag[i], ta->name))
        return 0;
    std::vector<const DagNode*> parts{&dag[i]};
    std::vector<const cnh_ast_node*> sets{sa};
    std::vector<int> dels;
    size_t end = i + 1;
    bool ran_out = false;
    while (parts.size() < 4) {
        std::vector<int> d2;
        const size_t j = skip_deletions(dag, end, d2);
        if (j == dag.size()) {
            ran_out = true;
            break;
        }
        XArray* tb = nullptr;
        const cnh_ast_node* sb = nullptr;
        if (!lattice_statement(ex, dag[j], &tb, &sb) || tb != ta || statement_reads(dag[j], ta->name))
            break;
        bool fits = true;
        for (int d = 0; d < sa->region.ndims; ++d)
            fits = fits && sb->region.step[d] == sa->region.step[d];
        for (const cnh_ast_node* other : sets) {
            bool apart = false;
            for (int d = 0; d < sa->region.ndims; ++d)
                apart = apart || progressions_disjoint(other->region.start[d], other->region.stop[d], other->region.step[d],
                                                       sb->region.start[d], sb->region.stop[d], sb->region.step[d]);
            fits = fits && apart;
        }
        for (int name : d2)
            fits = fits && name != ta->name;
        if (!fits)
            break;
        parts.push_back(&dag[j]);
        sets.push_back(sb);
        dels.insert(dels.end(), d2.begin(), d2.end());
        end = j + 1;
    }
    if (ran_out && open_ended_allowed(ex)) {
        *open_ended = true;                     // more statements of the run may follow
        return 0;
    }
    if (parts.size() < 2)
        return 0;
    DagNode merged;
    merge_statements(parts, merged);
    Group g;
    canonicalise(merged, g);
    cnh_kernel* k = nullptr;
    if (int rc = compile_cached(ex, g, &k))
        return rc;
    int n_in = 0, n_scalar = 0, n_out = 0;
    if (int rc = cnh_kernel_signature(k, &n_in, &n_scalar, &n_out))
        return rc;
    if (n_out != (int)parts.size() || ta->phased() || ta->elems >= (1ll << 31))
        return 0;
    std::vector<XArray*> in_arr((size_t)n_in);
    for (int q = 0; q < n_in; ++q) {
        int cname = 0, has = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_input(k, q, &cname, &has, &reg))
            return rc;
        auto it = ex->arrays.find(g.canon_to_actual[cname]);
        if (it == ex->arrays.end() || it->second.dtype != ta->dtype || it->second.ndims != ta->ndims ||
            it->second.phased() || &it->second == ta || it->second.elems >= (1ll << 31))
            return 0;
        in_arr[(size_t)q] = &it->second;
    }
    std::vector<const void*> scalars((size_t)std::max(1, n_scalar), nullptr);
    for (int q = 0; q < n_scalar; ++q) {
        int cname = 0;
        if (int rc = cnh_kernel_scalar(k, q, &cname))
            return rc;
        XArray* sarr;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &sarr, "broadcast scalar"))
            return rc;
        if (sarr->elems != 1 || sarr->dtype != ta->dtype || sarr == ta)
            return 0;
        scalars[(size_t)q] = sarr->tiles[0];
    }
    // from here on the statements are this launch
    if (int rc = make_block(ex, *ta))
        return rc;
    for (XArray* a : in_arr)
        if (int rc = make_block(ex, *a))
            return rc;
    std::vector<cnh_tiled> tin((size_t)std::max(1, n_in));
    for (int q = 0; q < n_in; ++q)
        tin[(size_t)q] = in_arr[(size_t)q]->tiled();
    const cnh_tiled cur = ta->tiled();
    if (!ex->dry)
        if (int rc = cnh_launch_group_tiles(k, n_in, tin.data(), n_scalar, scalars.data(), 1, &cur, &cur, ex->stream))
            return rc == -17 ? 0 : rc;          // not a shape the scatter takes: statement by statement
    ex->stats[5]++;
    if (ex->trace_on) ex->log("group node=" + std::to_string(merged.id) + " path=scatter roots=" + std::to_string(parts.size()) +
            " inputs=" + std::to_string(n_in) + " scalars=" + std::to_string(n_scalar) + " out=" +
            std::to_string(ta->name) + " inplace");
    for (int name : dels)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(end - i);
    *used = end - i;
    return 0;
}

int try_lattice_pair(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    XArray *ta = nullptr, *tb = nullptr;
    const cnh_ast_node *sa = nullptr, *sb = nullptr;
    if (!lattice_statement(ex, dag[i], &ta, &sa))
        return 0;
    std::vector<int> dels;
    const size_t j = skip_deletions(dag, i + 1, dels);
    if (j == dag.size()) {
        *open_ended = open_ended_allowed(ex);
        return 0;
    }
    if (!lattice_statement(ex, dag[j], &tb, &sb) || tb != ta)
        return 0;
    for (int d = 0; d < sa->region.ndims; ++d)
        if (sa->region.step[d] != sb->region.step[d])
            return 0;
    for (int name : dels)
        if (name == ta->name)
            return 0;
    // one group: the first statement's roots, then the second's
    DagNode merged;
    merge_statements({&dag[i], &dag[j]}, merged);
    Group g;
    canonicalise(merged, g);
    cnh_kernel* k = nullptr;
    if (int rc = compile_cached(ex, g, &k))
        return rc;
    if (cnh_kernel_lattice(k) != 2)
        return 0;                               // not two lattices that can be swept in place
    int n_in = 0, n_scalar = 0, n_out = 0;
    if (int rc = cnh_kernel_signature(k, &n_in, &n_scalar, &n_out))
        return rc;
    std::vector<XArray*> in_arr((size_t)n_in);
    for (int q = 0; q < n_in; ++q) {
        int cname = 0, has = 0;
        cnh_region reg;
        if (int rc = cnh_kernel_input(k, q, &cname, &has, &reg))
            return rc;
        auto it = ex->arrays.find(g.canon_to_actual[cname]);
        if (it == ex->arrays.end() || it->second.dtype != ta->dtype || it->second.ndims != ta->ndims ||
            it->second.tile != ta->tile || it->second.phased())
            return 0;
        for (int d = 0; d < ta->ndims; ++d)
            if (it->second.shape[d] != ta->shape[d])
                return 0;
        in_arr[(size_t)q] = &it->second;
    }
    if (ta->phased() || ta->elems >= (1ll << 31))
        return 0;
    std::vector<const void*> scalars((size_t)std::max(1, n_scalar), nullptr);
    for (int q = 0; q < n_scalar; ++q) {
        int cname = 0;
        if (int rc = cnh_kernel_scalar(k, q, &cname))
            return rc;
        XArray* sarr;
        if (int rc = find_array(ex, g.canon_to_actual[cname], &sarr, "broadcast scalar"))
            return rc;
        if (sarr->elems != 1 || sarr->dtype != ta->dtype)
            return 0;
        scalars[(size_t)q] = sarr->tiles[0];
    }
    // from here on the two statements are this launch
    if (int rc = make_block(ex, *ta))
        return rc;
    for (XArray* a : in_arr)
        if (int rc = make_block(ex, *a))
            return rc;
    std::vector<cnh_tiled> tin((size_t)std::max(1, n_in));
    for (int q = 0; q < n_in; ++q)
        tin[(size_t)q] = in_arr[(size_t)q]->tiled();
    const cnh_tiled cur = ta->tiled();
    ex->stats[5]++;
    if (ex->trace_on) ex->log("group node=" + std::to_string(merged.id) + " path=lattices roots=2 inputs=" + std::to_string(n_in) +
            " scalars=" + std::to_string(n_scalar) + " out=" + std::to_string(ta->name) + " inplace");
    if (!ex->dry)
        if (int rc = cnh_launch_group_tiles(k, n_in, tin.data(), n_scalar, scalars.data(), 1, &cur, &cur, ex->stream))
            return rc;
    for (int name : dels)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(j + 1 - i);
    *used = j + 1 - i;
    return 0;
}

int parse_dag(const char* msg, int64_t size, std::vector<DagNode>& out) {
    Reader r{msg, msg + size};
    int32_t magic = r.get<int32_t>(), version = r.get<int32_t>(), count = r.get<int32_t>();
    CNH_CHECK(r.ok && magic == CNX_DAG_MAGIC, -40, "not a DAG message (bad magic)");
    CNH_CHECK(version == 1, -40, "DAG message version %d (1 expected)", version);
    CNH_CHECK(count >= 0 && count <= (1 << 24), -40, "DAG message: %d nodes", count);
    out.resize((size_t)count);
    for (auto& n : out) {
        n.id = r.get<int32_t>();
        n.fusible = r.get<int32_t>();
        int32_t na = r.get<int32_t>(), nr = r.get<int32_t>();
        CNH_CHECK(r.ok && na >= 1 && na <= (1 << 20) && nr >= 1 && nr <= na, -41,
                  "DAG node %d: %d AST nodes, %d roots", n.id, na, nr);
        n.nodes.resize((size_t)na);
        for (int i = 0; i < na; ++i) {
            cnh_ast_node& a = n.nodes[i];
            std::memset(&a, 0, sizeof a);
            a.result_name = r.get<int32_t>();
            a.opcode = r.get<int32_t>();
            a.is_temp = r.get<int32_t>();
            a.is_scalar = r.get<int32_t>();
            a.is_broadcast = r.get<int32_t>();
            a.ndims = r.get<int32_t>();
            a.dtype = r.get<int32_t>();
            a.n_operands = r.get<int32_t>();
            CNH_CHECK(r.ok && a.n_operands >= 0 && a.n_operands <= 2, -41,
                      "DAG node %d: AST node %d has %d operands", n.id, i, a.n_operands);
            for (int j = 0; j < a.n_operands; ++j) {
                a.operands[j] = r.get<int32_t>();
                CNH_CHECK(r.ok && a.operands[j] >= 0 && a.operands[j] < i, -41,
                          "DAG node %d: AST node %d refers to node %d", n.id, i, a.operands[j]);
            }
            a.scalar = r.get<double>();
            for (int j = 0; j < a.n_operands; ++j) {
                CNH_CHECK(read_region(r, a.operand_regions[j]), -41, "DAG node %d: bad region", n.id);
                a.has_operand_region[j] = a.operand_regions[j].is_global ? 0 : 1;
            }
            CNH_CHECK(read_region(r, a.region), -41, "DAG node %d: bad region", n.id);
            CNH_CHECK(a.ndims >= 0 && a.ndims <= 3, -41, "DAG node %d: rank %d", n.id, a.ndims);
        }
        n.roots.resize((size_t)nr);
        for (auto& x : n.roots) {
            x = r.get<int32_t>();
            CNH_CHECK(r.ok && x >= 0 && x < na, -41, "DAG node %d: root index out of range", n.id);
        }
    }
    CNH_CHECK(r.ok, -42, "DAG message truncated");
    CNH_CHECK(r.p == r.end, -42, "DAG message has %lld trailing bytes", (long long)(r.end - r.p));
    return 0;
}

} // namespace

namespace {

// The metadata pass and the solver call of src/dag_group_receive.cpp:222-399: the shape of every
// array the message will produce, then tile and offset for all of them at once. A result whose
// shape cannot be told in advance is left to the tile rule when it is created.
void plan_message(Ex* ex, const std::vector<DagNode>& dag) {
    std::map<int, DecompMeta> meta;
    auto existing = [&](int name) {
        if (meta.count(name))
            return;
        auto it = ex->arrays.find(name);
        if (it == ex->arrays.end())
            return;
        DecompMeta m;
        m.ndims = it->second.ndims;
        m.tile = it->second.tile;
        m.final = true;
        for (int d = 0; d < m.ndims; ++d) {
            m.shape[d] = it->second.shape[d];
            m.offset[d] = it->second.offset[d];
        }
        meta[name] = m;
    };
    auto known = [&](const DagNode& n, const cnh_ast_node& root, int i) -> const DecompMeta* {
        if (i >= root.n_operands)
            return nullptr;
        const cnh_ast_node& op = n.nodes[root.operands[i]];
        if (op.is_scalar || op.opcode != CNH_OP_NOOP)
            return nullptr;
        auto it = meta.find(op.result_name);
        return it == meta.end() ? nullptr : &it->second;
    };
    // rows and columns of operand i seen as a matrix: a 2-D array (or window of one), or the plane
    // that a 3-D window with an extent of 1 leaves (src/dag_group_receive.cpp:251-323)
    auto matrix_dims = [](const DecompMeta& m, const cnh_ast_node& root, int i, int* rows, int* cols) {
        int ext[3] = {m.shape[0], m.shape[1], m.shape[2]};
        if (root.has_operand_region[i] && !root.operand_regions[i].is_global &&
            root.operand_regions[i].ndims == m.ndims)
            for (int d = 0; d < m.ndims; ++d)
                ext[d] = root.operand_regions[i].stop[d] - root.operand_regions[i].start[d];
        if (m.ndims == 2) {
            *rows = ext[0];
            *cols = ext[1];
            return true;
        }
        if (m.ndims != 3)
            return false;
        int dropped = -1;
        for (int d = 0; d < 3 && dropped < 0; ++d)
            if (ext[d] == 1)
                dropped = d;
        if (dropped < 0)
            return false;
        *rows = ext[dropped == 0 ? 1 : 0];
        *cols = ext[dropped == 2 ? 1 : 2];
        return true;
    };
    std::vector<int> fresh;
    auto result = [&](int name, int nd, const int32_t* shape) {
        if (nd < 1 || nd > 3 || meta.count(name) || ex->arrays.count(name))
            return;
        DecompMeta m;
        m.ndims = nd;
        for (int d = 0; d < nd; ++d) {
            if (shape[d] < 1)
                return;
            m.shape[d] = shape[d];
        }
        meta[name] = m;
        fresh.push_back(name);
    };
    for (const DagNode& n : dag) {
        if (n.roots.empty())
            continue;
        for (const cnh_ast_node& a : n.nodes)
            if (!a.is_scalar && a.opcode == CNH_OP_NOOP)
                existing(a.result_name);
        const cnh_ast_node& root = n.nodes[n.roots.back()];
        int32_t shape[3] = {1, 1, 1};
        switch (root.opcode) {
        case CNH_OP_CREATE:
        case CNH_OP_TILE:
            if (!root.region.is_global && root.region.ndims == root.ndims) {
                for (int d = 0; d < root.ndims; ++d)
                    shape[d] = region_count(root.region, d);
                result(root.result_name, root.ndims, shape);
            }
            break;
        case CNH_OP_REDUCE:
        case kOpSum:
        case kOpSumsqDiff:
        case kOpMaxabsDiff: result(root.result_name, 1, shape); break;
        case kOpAstype: {
            const DecompMeta* in = known(n, root, 0);
            if (in)
                result(root.result_name, in->ndims, in->shape);
            break;
        }
        case CNH_OP_MATMUL: {
            int rows, cols;
            const DecompMeta* A = known(n, root, 0);
            if (A && matrix_dims(*A, root, 0, &rows, &cols)) {
                shape[0] = rows;
                result(root.result_name, 1, shape);
            }
            break;
        }
        case CNH_OP_MATMATMUL: {
            int ar, ac, br, bc;
            const DecompMeta *A = known(n, root, 0), *B = known(n, root, 1);
            if (A && B && matrix_dims(*A, root, 0, &ar, &ac) && matrix_dims(*B, root, 1, &br, &bc)) {
                shape[0] = ar;
                shape[1] = bc;
                result(root.result_name, 2, shape);
            }
            break;
        }
        case CNH_OP_DIAG: {
            const DecompMeta* in = known(n, root, 0);
            int k = root.n_operands >= 2 && n.nodes[root.operands[1]].is_scalar
                        ? (int)n.nodes[root.operands[1]].scalar
                        : 0;
            if (in && in->ndims == 1) {
                shape[0] = shape[1] = in->shape[0] + std::abs(k);
                result(root.result_name, 2, shape);
            } else if (in && in->ndims == 2) {
                shape[0] = k >= 0 ? std::min(in->shape[0], in->shape[1] - k)
                                  : std::min(in->shape[0] + k, in->shape[1]);
                result(root.result_name, 1, shape);
            }
            break;
        }
        case CNH_OP_ADD:
        case CNH_OP_SUB:
        case CNH_OP_MUL:
        case CNH_OP_DIV:
        case CNH_OP_TANH:
        case CNH_OP_EXP:
        case CNH_OP_COPY: {
            // as result_shape(): the root's own region, else the first region an array is read
            // through, else the shape of an operand array
            bool found = false;
            if (!root.region.is_global && root.region.ndims == root.ndims) {
                for (int d = 0; d < root.ndims; ++d)
                    shape[d] = region_count(root.region, d);
                found = true;
            }
            for (size_t ai = 0; ai < n.nodes.size() && !found; ++ai) {
                const cnh_ast_node& a = n.nodes[ai];
                if (a.is_scalar || a.opcode == CNH_OP_NOOP)
                    continue;
                bool settled = false;
                for (int i = 0; i < a.n_operands && !settled; ++i) {
                    const cnh_ast_node& op = n.nodes[a.operands[i]];
                    if (op.is_scalar || op.opcode != CNH_OP_NOOP)
                        continue;
                    if (a.has_operand_region[i] && !a.operand_regions[i].is_global) {
                        for (int d = 0; d < op.ndims && d < 3; ++d)
                            shape[d] = region_count(a.operand_regions[i], d);
                        found = settled = true;
                        break;
                    }
                    auto it = meta.find(op.result_name);
                    if (it == meta.end())
                        continue;
                    for (int d = 0; d < 3; ++d)
                        shape[d] = d < it->second.ndims ? it->second.shape[d] : 1;
                    found = true;
                    settled = !op.is_broadcast;
                }
                if (settled)
                    break;
            }
            if (found)
                result(root.result_name, root.ndims, shape);
            break;
        }
        default: break;
        }
    }
    if (fresh.empty())
        return;
    solve_decompositions(meta, dag, ex->odf, ex->num_pes, ex->min_tile);
    for (int name : fresh) {
        const DecompMeta& m = meta[name];
        Ex::Planned p;
        p.ndims = m.ndims;
        p.tile = m.tile;
        for (int d = 0; d < m.ndims; ++d) {
            p.shape[d] = m.shape[d];
            p.offset[d] = m.offset[d];
        }
        ex->planned[name] = p;
        if (ex->trace_on) ex->log("plan " + std::to_string(name) + " tile=" + std::to_string(p.tile) + " offset=" +
                shape_str(p.offset, p.ndims));
    }
}

// MATMATMUL -> tmp; target[box] = tmp; delete tmp: the product is written into the box directly.
int try_product_into_region(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    if (!dag[i].roots.empty() && dag[i].nodes[dag[i].roots.back()].opcode == CNH_OP_MATMATMUL &&
        i + 2 >= dag.size() && open_ended_allowed(ex)) {
        // the assignment that takes the product, or the deletion of the temporary, may be the
        // first nodes of the next message
        *open_ended = true;
        return 0;
    }
    if (i + 2 >= dag.size() || dag[i].roots.empty() || dag[i + 1].roots.size() != 1 || dag[i + 2].roots.empty())
        return 0;
    const cnh_ast_node& mm = dag[i].nodes[dag[i].roots.back()];
    const cnh_ast_node& set = dag[i + 1].nodes[dag[i + 1].roots.back()];
    const cnh_ast_node& del = dag[i + 2].nodes[dag[i + 2].roots.back()];
    if (mm.opcode != CNH_OP_MATMATMUL || set.opcode != CNH_OP_SET_REGION || del.opcode != kOpDelete ||
        set.n_operands != 2 || set.region.is_global || del.result_name != mm.result_name)
        return 0;
    const cnh_ast_node& value = dag[i + 1].nodes[set.operands[1]];
    if (value.is_scalar || value.opcode != CNH_OP_NOOP || value.result_name != mm.result_name ||
        (set.has_operand_region[1] && !set.operand_regions[1].is_global))
        return 0;
    for (int d = 0; d < set.region.ndims; ++d)
        if (set.region.step[d] != 1)
            return 0;
    bool taken = false;
    if (int rc = exec_matmatmul(ex, dag[i], mm, &dag[i + 1], &taken))
        return rc;
    if (taken) {
        ex->stats[2] += 3;
        *used = 3;
    } else {
        ex->stats[2] += 1;
        *used = 1;               // the product went to a temporary as usual; the rest follows node by node
    }
    return 0;
}

// ---- a product and the statements on its result as one launch ----
//
// `target[box] = A @ B` followed by a run of statements that read the box column block by column
// block (the gate statements of an LSTM step read the four gates' columns of IFOG[t],
// examples/lstm_forward.py:40-49 upstream): the product's launch evaluates the run on each
// workgroup's tile of sums (cnh_launch_product_group), so the step is one launch and nothing waits
// for a second one to start. Taken when
//   - the product is a single fp64 panel product into the box, in whole 64 x 64 x 16 tiles of
//     aligned operands (what the fused kernel is built for);
//   - the run's extents are (rows of the product) x (its columns / q), q = 1, 2 or 4, and every read
//     of the target that meets the box is exactly one of its q column blocks;
//   - no statement assigns into the box or into a window the product reads (workgroups finish at
//     different times: a statement's stores must not reach what another workgroup still multiplies).
// The statements of one element depend on that element's values only (what a statement run is), so
// evaluating them tile by tile as the tiles complete gives what the two launches give.
bool unit_regions_disjoint(const cnh_region& a, const cnh_region& b, int nd) {
    for (int d = 0; d < nd; ++d)
        if (a.stop[d] <= b.start[d] || b.stop[d] <= a.start[d])
            return true;
    return false;
}

int try_product_with_statements(Ex* ex, const std::vector<DagNode>& dag, size_t i, size_t* used, bool* open_ended) {
    *used = 0;
    *open_ended = false;
    if (!product_statements_on() || i + 2 >= dag.size() || dag[i].roots.empty() || dag[i + 1].roots.size() != 1 ||
        dag[i + 2].roots.empty())
        return 0;
    const cnh_ast_node& mm = dag[i].nodes[dag[i].roots.back()];
    const cnh_ast_node& set = dag[i + 1].nodes[dag[i + 1].roots.back()];
    const cnh_ast_node& del = dag[i + 2].nodes[dag[i + 2].roots.back()];
    if (mm.opcode != CNH_OP_MATMATMUL || set.opcode != CNH_OP_SET_REGION || del.opcode != kOpDelete ||
        set.n_operands != 2 || set.region.is_global || del.result_name != mm.result_name)
        return 0;
    const cnh_ast_node& value = dag[i + 1].nodes[set.operands[1]];
    if (value.is_scalar || value.opcode != CNH_OP_NOOP || value.result_name != mm.result_name ||
        (set.has_operand_region[1] && !set.operand_regions[1].is_global))
        return 0;
    for (int d = 0; d < set.region.ndims; ++d)
        if (set.region.step[d] != 1)
            return 0;
    // why a product that has statements behind it keeps a launch of its own, for the trace
    auto no = [&](const char* why) {
        if (ex->trace_on) ex->log(std::string("product node=") + std::to_string(dag[i].id) + " statements_not_taken: " + why);
        return 0;
    };
    // the product as it would be launched, without launching it
    std::vector<cnh_gemm_job> jobs;
    ProductOperands ops;
    bool taken = false;
    if (int rc = exec_matmatmul(ex, dag[i], mm, &dag[i + 1], &taken, &jobs, &ops))
        return rc;
    if (!taken || jobs.empty())
        return no("the product does not go into the box as panel products");
    if (!gemm_form(ops.M, ops.N, ops.K, nullptr, ops.K, nullptr, ops.N))
        return no("extents no multiples of the 64 x 64 x 16 tile");
    if (i + 3 >= dag.size()) {
        // the statements that read it may be the first nodes of the next message
        *open_ended = open_ended_allowed(ex);
        return 0;
    }
    ProductSite site;
    auto tgt = ex->arrays.find(dag[i + 1].nodes[set.operands[0]].result_name);
    if (tgt == ex->arrays.end() || set.region.ndims != tgt->second.ndims)
        return no("target unknown");
    site.target = &tgt->second;
    site.region = set.region;
    const int tnd = site.target->ndims, last = tnd - 1;
    if (site.region.stop[last] - site.region.start[last] != ops.N)
        return no("the box's columns are not the target's last dimension");
    StatementRun sr;
    collect_statement_run(ex, dag, i + 3, sr);
    if (sr.run.empty())
        return no("no statement run follows");
    // the run may go on in the next message (and its extents settle only when it is complete: a
    // wider first statement is cut to fit the ones that follow): the product waits with it
    if (sr.ran_off_end) {
        *open_ended = true;
        return 0;
    }
    // the run's extents: (1, ..., M, N / q)
    const Stmt& first = sr.run.front();
    if (first.nd < 2 || first.dtype != CNH_F64 || first.cnt[first.nd - 2] != ops.M ||
        first.cnt[first.nd - 1] <= 0 || ops.N % first.cnt[first.nd - 1] != 0)
        return no("the run's extents are not the product's rows by a fraction of its columns");
    for (int d = 0; d + 2 < first.nd; ++d)
        if (first.cnt[d] != 1)
            return no("the run's extents are not the product's rows by a fraction of its columns");
    site.blocks = (int)(ops.N / first.cnt[first.nd - 1]);
    if (site.blocks != 1 && site.blocks != 2 && site.blocks != 4)
        return no("column blocks other than 1, 2 or 4");
    bool reads_product = false;
    for (const Stmt& st : sr.run) {
        if (!st.scalars_read.empty())
            return no("a statement reads a one-element array");
        // nothing is assigned where the product writes or reads
        if (st.out.arr == site.target && !unit_regions_disjoint(st.out.reg, site.region, tnd))
            return no("a statement assigns into the product's box");
        if (st.out.arr == ops.A && !unit_regions_disjoint(st.out.reg, ops.wA, ops.A->ndims))
            return no("a statement assigns into the left operand's window");
        if (st.out.arr == ops.B && !unit_regions_disjoint(st.out.reg, ops.wB, ops.B->ndims))
            return no("a statement assigns into the right operand's window");
        for (const auto& rd : st.reads) {
            if (rd.use.arr != site.target || unit_regions_disjoint(rd.use.reg, site.region, tnd))
                continue;
            if (product_block(site, rd.use) < 0)
                return no("a statement reads the box other than by column blocks");
            reads_product = true;
        }
    }
    if (!reads_product)
        return no("the run does not read the product");
    if (jobs.size() != 1) {
        // operands cut into tiles (a weight matrix of rank 2 is, by default) give one panel product
        // per tile: laid out as one block each, once, they give a single one from now on
        for (XArray* a : {ops.A, ops.B})
            if (!ex->dry && ex->flat3 && a->ndims == 2 && !a->flat && a->ntiles > 1 && !a->phased())
                if (int rc = make_block(ex, *a))
                    return rc;
        if (int rc = exec_matmatmul(ex, dag[i], mm, &dag[i + 1], &taken, &jobs, &ops))
            return rc;
        if (!taken || jobs.size() != 1)
            return no("not a single panel product into the box");
    }
    if (!gemm_form(jobs[0].M, jobs[0].N, jobs[0].K, jobs[0].A, jobs[0].lda, jobs[0].B, jobs[0].ldb))
        return no("operands the buffer loads do not take");
    site.job = jobs[0];
    site.what = "matmatmul A=" + std::to_string(ops.A->name) + " B=" + std::to_string(ops.B->name) + " out=" +
                std::to_string(site.target->name) + " into_region panel_products=1";
    if (ex->dry) {
        // a planning pass launches nothing: the product and the run are noted as they would go out
        if (ex->trace_on) ex->log(site.what);
        if (int rc = exec_statement_run(ex, sr.run))
            return rc;
    } else if (int rc = exec_statement_run(ex, sr.run, &site)) {
        return rc;
    }
    for (int name : sr.deletions_kept)
        drop_array(ex, name);
    ex->stats[2] += (int64_t)(sr.last_stmt_end - i);
    *used = sr.last_stmt_end - i;
    return 0;
}

// Named ranges around the work of every DAG node, for profilers that trace roctx markers
// (rocprofv3 --marker-trace): kernels then group by what the program asked for instead of by
// grid size. Off unless CHARMNUMERIC_ROCTX is set to something other than 0; the marker library is
// looked up at run time, so nothing links against it.
struct Markers {
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
    Markers() {
        const char* on = std::getenv("CHARMNUMERIC_ROCTX");
        if (on == nullptr || on[0] == '\0' || (on[0] == '0' && on[1] == '\0'))
            return;
        for (const char* lib : {"librocprofiler-sdk-roctx.so", "libroctx64.so"}) {
            void* h = dlopen(lib, RTLD_NOW | RTLD_GLOBAL);
            if (h == nullptr)
                continue;
            push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
            pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
            if (push != nullptr && pop != nullptr)
                return;
            push = nullptr;
            pop = nullptr;
        }
    }
};
const Markers& markers() {
    static const Markers m;
    return m;
}
const char* node_kind(const DagNode& n) {
    if (n.roots.empty())
        return "cnx:empty";
    switch (n.nodes[n.roots.back()].opcode) {
    case CNH_OP_CREATE: return "cnx:create";
    case kOpDelete: return "cnx:delete";
    case CNH_OP_REDUCE: return "cnx:reduce";
    case kOpSum: return "cnx:sum";
    case kOpSumsqDiff: return "cnx:sumsq_diff";
    case kOpMaxabsDiff: return "cnx:maxabs_diff";
    case kOpAstype: return "cnx:astype";
    case CNH_OP_MATMUL: return "cnx:matmul";
    case CNH_OP_MATMATMUL: return "cnx:matmatmul";
    case CNH_OP_TILE: return "cnx:tile";
    case CNH_OP_DIAG: return "cnx:diag";
    case CNH_OP_SET_REGION: return "cnx:assign";
    default: return "cnx:elementwise";
    }
}
struct Range {
    bool open = false;
    explicit Range(const char* name) {
        if (markers().push != nullptr) {
            markers().push(name);
            open = true;
        }
    }
    ~Range() {
        if (open)
            markers().pop();
    }
};

int run_nodes(Ex* ex, std::vector<DagNode>& dag) {
    if (ex->solver_on)
        plan_message(ex, dag);
    int rc = 0;
    for (size_t i = 0; i < dag.size() && rc == 0;) {
        size_t used = 0;
        const Range range(node_kind(dag[i]));   // covers the nodes a rewrite takes along with this one
        // a deletion needs no value: a pending sum nobody read goes with its array
        if (!dag[i].roots.empty() && dag[i].nodes[dag[i].roots.back()].opcode == kOpDelete) {
            rc = exec_node(ex, dag[i]);
            ++i;
            continue;
        }
        if (ex->fuse_on && !ex->solver_on) {
            bool open_ended = false;
            // the two rewrites that know about pending sums go first ...
            rc = try_fused_matvec(ex, dag, i, &used, &open_ended);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_dense_run(ex, dag, i, &used, &open_ended);
            // ... everything else reads arrays as they are
            if (rc == 0 && used == 0 && !open_ended)
                rc = resolve_all(ex);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_scatter_run(ex, dag, i, &used, &open_ended);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_lattice_pair(ex, dag, i, &used, &open_ended);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_product_with_statements(ex, dag, i, &used, &open_ended);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_product_into_region(ex, dag, i, &used, &open_ended);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_statement_run(ex, dag, i, &used, &open_ended);
            if (rc == 0 && used == 0 && !open_ended)
                rc = try_group_with_reductions(ex, dag, i, &used, &open_ended);
            if (rc == 0 && open_ended) {
                ex->held.assign(dag.begin() + (std::ptrdiff_t)i, dag.end());
                break;
            }
        }
        if (rc == 0 && used == 0) {
            rc = resolve_all(ex);
            if (rc == 0)
                rc = exec_node(ex, dag[i]);
            used = 1;
        }
        i += used;
    }
    ex->planned.clear();
    // sums may stay pending only while nodes are held: their consumer may be among what follows
    if (rc == 0 && ex->held.empty())
        rc = resolve_all(ex);
    return rc;
}

// Runs freshly arrived nodes behind what the previous message left open.
int run_fresh(Ex* ex, std::vector<DagNode>& fresh) {
    std::vector<DagNode> dag;
    dag.swap(ex->held);
    dag.insert(dag.end(), std::make_move_iterator(fresh.begin()), std::make_move_iterator(fresh.end()));
    return run_nodes(ex, dag);
}

int run_log(Ex* ex, const char* log, int64_t size, int window);

// Statements an automatic flush held back are older than anything that arrives now: plan them to
// the end and run them.
int finish_log(Ex* ex) {
    return ex->plog.empty() ? 0 : run_log(ex, nullptr, 0, -1);
}

int run_message(Ex* ex, const char* msg, int64_t size) {
    std::vector<DagNode> fresh;
    if (int rc = parse_dag(msg, size, fresh))
        return rc;
    if (int rc = finish_log(ex))
        return rc;
    return run_fresh(ex, fresh);
}

// A stretch of the statement log: appended to what an earlier automatic flush held back, planned
// up to the hold-back cut (window >= 0) or to the end (window < 0), and run.
int run_log(Ex* ex, const char* log, int64_t size, int window) {
    if (int rc = stmtlog::parse(log, size, ex->plog)) {
        ex->plog.clear();
        return rc;
    }
    if (ex->plog.empty())
        return 0;
    const size_t cut = window >= 0 ? stmtlog::hold_back_cut(ex->plog, window) : ex->plog.size();
    std::set<int32_t> dead, fused_away;
    if (cut < ex->plog.size())
        dead = stmtlog::dead_later(ex->plog, cut);
    std::vector<DagNode> fresh;
    stmtlog::plan(ex->plog, cut, dead, &ex->next_set_name, fresh, &fused_away);
    // what stays behind; deletions of results that never became arrays have nothing to delete
    std::vector<stmtlog::Instr> tail;
    for (size_t i = cut; i < ex->plog.size(); ++i)
        if (!(ex->plog[i].kind == stmtlog::kDelete && fused_away.count(ex->plog[i].name)))
            tail.push_back(ex->plog[i]);
    ex->plog.swap(tail);
    if (ex->capture_on) {
        const std::vector<char> bytes = stmtlog::to_message(fresh);
        const int64_t len = (int64_t)bytes.size();
        const char* lp = reinterpret_cast<const char*>(&len);
        ex->captured.insert(ex->captured.end(), lp, lp + 8);
        ex->captured.insert(ex->captured.end(), bytes.begin(), bytes.end());
    }
    if (fresh.empty())
        return 0;
    return run_fresh(ex, fresh);
}

// Executes whatever waits in `held`, to the end.
int flush_held(Ex* ex) {
    if (ex->held.empty())
        return 0;
    std::vector<DagNode> dag;
    dag.swap(ex->held);
    ex->final_pass = true;
    const int rc = run_nodes(ex, dag);
    ex->final_pass = false;
    return rc;
}

void worker_loop(Ex* ex) {
    if (!ex->dry)
        (void)hipSetDevice(ex->device);   // the current device is a per-thread setting
    std::unique_lock<std::mutex> lk(ex->qmu);
    for (;;) {
        ex->qcv.wait(lk, [&] { return ex->stop || !ex->queue.empty(); });
        if (ex->queue.empty())
            return;   // stop requested and nothing left
        Ex::Queued msg = std::move(ex->queue.front());
        ex->queue.pop_front();
        if (ex->deferred_rc != 0) {   // work behind a failed message is dropped
            if (ex->queue.empty())
                ex->idle_cv.notify_all();
            continue;
        }
        ex->busy = true;
        lk.unlock();
        const int rc = msg.is_log ? run_log(ex, msg.bytes.data(), (int64_t)msg.bytes.size(), msg.window)
                                  : run_message(ex, msg.bytes.data(), (int64_t)msg.bytes.size());
        std::string text = rc ? cnh_last_error() : "";
        lk.lock();
        ex->busy = false;
        if (rc) {
            ex->deferred_rc = rc;
            ex->deferred_msg = std::move(text);
        }
        if (ex->queue.empty())
            ex->idle_cv.notify_all();
    }
}

// Waits for queued messages and hands over the error one of them may have left.
int drain(Ex* ex) {
    if (ex->async_on) {
        std::unique_lock<std::mutex> lk(ex->qmu);
        ex->idle_cv.wait(lk, [&] { return ex->queue.empty() && !ex->busy; });
        if (ex->deferred_rc != 0) {
            const int rc = ex->deferred_rc;
            const std::string text = std::move(ex->deferred_msg);
            ex->deferred_rc = 0;
            ex->deferred_msg.clear();
            ex->held.clear();           // work behind a failed message is dropped
            ex->plog.clear();
            lk.unlock();
            return set_error(rc, "%s", text.c_str());
        }
    }
    // the worker is idle now (or there is none): the statements it left open run on this thread
    return flush_held(ex);
}

// For calls that read or write array state (get, put, fills, sync, array_info): everything
// received so far has run when this returns, the statements a hold-back flush left unplanned
// included.
int settle(Ex* ex) {
    if (int rc = drain(ex))
        return rc;
    if (int rc = finish_log(ex))
        return rc;
    if (int rc = flush_held(ex))
        return rc;
    return resolve_all(ex);
}

void stop_worker(Ex* ex) {
    {
        std::unique_lock<std::mutex> lk(ex->qmu);
        ex->stop = true;
        ex->qcv.notify_all();
    }
    if (ex->worker.joinable())
        ex->worker.join();
    ex->async_on = false;
}

} // namespace

extern "C" {

int cnx_create(int device, int num_pes, int odf, cnx_executor** out) {
    CNH_CHECK(out != nullptr, -2, "null argument");
    CNH_CHECK(num_pes >= 1 && odf >= 1, -2, "num_pes and odf must be positive");
    auto ex = std::make_unique<cnx_executor>();
    ex->dry = device < 0;
    ex->num_pes = num_pes;
    ex->odf = odf;
    ex->device = device;
    if (!ex->dry) {
        if (int rc = cnh_init(device))
            return rc;
        if (int rc = cnh_stream_create(&ex->stream))
            return rc;
    }
    *out = ex.release();
    return 0;
}

int cnx_destroy(cnx_executor* ex) {
    if (!ex)
        return 0;
    (void)drain(ex);
    if (ex->async_on)
        stop_worker(ex);
    if (!ex->dry) {
        cnh_stream_sync(ex->stream);
        for (auto& kv : ex->arrays) {
            cnh_free(kv.second.slab);
            if (kv.second.alt)
                cnh_free(kv.second.alt);
        }
        for (auto& kv : ex->pending)
            cnh_free(kv.second.partials);
        for (auto& pr : ex->matvec_events) {
            cnh_event_destroy(pr.first);
            cnh_event_destroy(pr.second);
        }
        for (auto& kv : ex->free_list)
            for (void* p : kv.second)
                cnh_free(p);
        cnh_stream_destroy(ex->stream);
    }
    for (auto& kv : ex->kernels)
        cnh_kernel_release(kv.second);
    delete ex;
    return 0;
}

int cnx_set_min_tile(cnx_executor* ex, int ndims, int min_tile) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = drain(ex))
        return rc;
    CNH_CHECK(ndims >= 1 && ndims <= 3 && min_tile >= 1, -2, "bad minimum tile %d for rank %d",
              min_tile, ndims);
    ex->min_tile[ndims] = min_tile;
    return 0;
}

int cnx_set_solver(cnx_executor* ex, int on) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = drain(ex))
        return rc;
    ex->solver_on = on != 0;
    return 0;
}

int cnx_set_layout(cnx_executor* ex, int flat_rank3) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = drain(ex))
        return rc;
    ex->flat3 = flat_rank3 != 0;
    return 0;
}

int cnx_set_fusion(cnx_executor* ex, int on) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = drain(ex))
        return rc;
    ex->fuse_on = on != 0;
    return 0;
}

int cnx_set_trace(cnx_executor* ex, int on) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = drain(ex))
        return rc;
    ex->trace_on = on != 0;
    return 0;
}

int64_t cnx_trace(cnx_executor* ex, char* buf, size_t cap) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = drain(ex))
        return rc;
    int64_t need = (int64_t)ex->trace.size() + 1;
    if (buf && cap >= (size_t)need) {
        std::memcpy(buf, ex->trace.c_str(), (size_t)need);
        ex->trace.clear();
    }
    return need;
}

int cnx_receive_dag(cnx_executor* ex, int epoch, int64_t size, const char* msg) {
    (void)epoch;
    CNH_CHECK(ex != nullptr && msg != nullptr && size >= 12, -2, "bad DAG message");
    if (!ex->async_on)
        return run_message(ex, msg, size);
    {
        std::unique_lock<std::mutex> lk(ex->qmu);
        if (ex->deferred_rc == 0) {
            ex->queue.emplace_back();
            ex->queue.back().bytes.assign(msg, msg + size);
            ex->qcv.notify_one();
            return 0;
        }
    }
    return drain(ex);   // an earlier message failed: report that instead of queueing more
}

int cnx_receive_log(cnx_executor* ex, int64_t size, const char* log, int hold_back_window) {
    CNH_CHECK(ex != nullptr && size >= 0 && (log != nullptr || size == 0), -2, "bad statement log");
    if (!ex->async_on)
        return run_log(ex, log, size, hold_back_window);
    {
        std::unique_lock<std::mutex> lk(ex->qmu);
        if (ex->deferred_rc == 0) {
            ex->queue.emplace_back();
            if (size > 0)
                ex->queue.back().bytes.assign(log, log + size);
            ex->queue.back().is_log = true;
            ex->queue.back().window = hold_back_window;
            ex->qcv.notify_one();
            return 0;
        }
    }
    return drain(ex);
}

int cnx_discard_log(cnx_executor* ex) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    const int rc = drain(ex);
    ex->plog.clear();
    return rc;
}

int cnx_set_capture(cnx_executor* ex, int on) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    const int rc = drain(ex);
    ex->capture_on = on != 0;
    ex->captured.clear();
    return rc;
}

int64_t cnx_captured(cnx_executor* ex, char* buf, size_t cap) {
    if (ex == nullptr)
        return -2;
    if (int rc = drain(ex))
        return rc;
    const size_t need = ex->captured.size();
    if (buf != nullptr && cap >= need) {
        if (need)
            std::memcpy(buf, ex->captured.data(), need);
        ex->captured.clear();
    }
    return (int64_t)need;
}

int cnx_set_async(cnx_executor* ex, int on) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    const int rc = drain(ex);
    if (on && !ex->async_on) {
        ex->stop = false;
        ex->async_on = true;
        ex->worker = std::thread(worker_loop, ex);
    } else if (!on && ex->async_on) {
        stop_worker(ex);
    }
    return rc;
}

int cnx_get(cnx_executor* ex, int ndims, int epoch, int name, int64_t size, int dtype, void* host_out) {
    (void)epoch;
    CNH_CHECK(ex != nullptr && host_out != nullptr, -2, "null argument");
    if (int rc = settle(ex))
        return rc;
    XArray* a;
    if (int rc = find_array(ex, name, &a, "get"))
        return rc;
    CNH_CHECK(a->ndims == ndims && a->dtype == dtype && a->elems == size, -50,
              "get of array %d: asked for rank %d dtype %d size %lld, array has rank %d dtype %d size %lld",
              name, ndims, dtype, (long long)size, a->ndims, a->dtype, (long long)a->elems);
    if (ex->trace_on) ex->log("get " + std::to_string(name) + " tiles=" + std::to_string(a->ntiles));
    if (ex->dry) {
        std::memset(host_out, 0, (size_t)size * dtype_size(dtype));
        return 0;
    }
    const int esz = dtype_size(dtype);
    int64_t gstr[3] = {1, 1, 1};
    {
        int64_t s = 1;
        for (int d = ndims - 1; d >= 0; --d) {
            gstr[d] = s;
            s *= a->shape[d];
        }
    }
    if (a->flat) {
        // one block in the global row-major order already
        if (int rc = cnh_d2h(host_out, a->slab, (size_t)a->elems * esz, ex->stream))
            return rc;
        return cnh_stream_sync(ex->stream);
    }
    for (int64_t t = 0; t < a->ntiles; ++t) {
        int32_t lo[3], ext[3];
        a->tile_extent(t, lo, ext);
        int64_t dstart[3], sstart[3] = {0, 0, 0}, counts[3], sstr[3];
        a->tile_strides(ext, sstr);
        for (int d = 0; d < ndims; ++d) {
            dstart[d] = lo[d];
            counts[d] = ext[d];
        }
        if (int rc = cnh_d2h_region(ndims, esz, host_out, gstr, dstart, a->tiles[t], sstr, sstart, counts,
                                    ex->stream))
            return rc;
    }
    return cnh_stream_sync(ex->stream);
}

int cnx_put(cnx_executor* ex, int name, int64_t size, int dtype, const void* host_in) {
    CNH_CHECK(ex != nullptr && host_in != nullptr, -2, "null argument");
    if (int rc = settle(ex))
        return rc;
    XArray* a;
    if (int rc = find_array(ex, name, &a, "put"))
        return rc;
    CNH_CHECK(a->dtype == dtype && a->elems == size, -50,
              "put into array %d: %lld elements of dtype %d offered, array has %lld of dtype %d", name,
              (long long)size, dtype, (long long)a->elems, a->dtype);
    if (ex->trace_on) ex->log("put " + std::to_string(name));
    if (ex->dry)
        return 0;
    const int esz = dtype_size(dtype);
    const int nd = a->ndims;
    std::vector<char> stage;
    for (int64_t t = 0; t < a->ntiles; ++t) {
        int32_t lo[3], ext[3];
        a->tile_extent(t, lo, ext);
        const char* src = static_cast<const char*>(host_in);
        if (a->ntiles == 1 || a->flat) {
            if (int rc = cnh_h2d(a->tiles[0], src, (size_t)a->elems * esz, ex->stream))
                return rc;
            break;
        }
        stage.resize((size_t)a->tile_elems[t] * esz);
        // rows of the innermost dimension are contiguous on both sides
        int32_t e0 = nd >= 3 ? ext[0] : 1, e1 = nd >= 2 ? ext[nd - 2] : 1, e2 = ext[nd - 1];
        int64_t g2 = 1, g1 = a->shape[nd - 1], g0 = nd >= 2 ? (int64_t)a->shape[nd - 1] * a->shape[nd - 2] : 0;
        int32_t l0 = nd >= 3 ? lo[0] : 0, l1 = nd >= 2 ? lo[nd - 2] : 0, l2 = lo[nd - 1];
        (void)g2;
        size_t w = 0;
        for (int i = 0; i < e0; ++i)
            for (int j = 0; j < e1; ++j) {
                const char* row = src + ((int64_t)(l0 + i) * g0 + (int64_t)(l1 + j) * g1 + l2) * esz;
                std::memcpy(stage.data() + w, row, (size_t)e2 * esz);
                w += (size_t)e2 * esz;
            }
        if (int rc = cnh_h2d(a->tiles[t], stage.data(), stage.size(), ex->stream))
            return rc;
    }
    return 0;
}

int cnx_fill_uniform(cnx_executor* ex, int name, uint64_t seed, uint64_t stream_id, double lo, double hi) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = settle(ex))
        return rc;
    XArray* a;
    if (int rc = find_array(ex, name, &a, "fill_uniform"))
        return rc;
    CNH_CHECK(a->dtype == CNH_F64, -27, "fill_uniform needs an fp64 array");
    if (ex->trace_on) ex->log("fill_uniform " + std::to_string(name));
    if (ex->dry)
        return 0;
    int64_t gshape[3];
    for (int d = 0; d < 3; ++d)
        gshape[d] = a->shape[d];
    if (a->flat)   // the counter of an element is its global row-major index: one run over the block
        return cnh_fill_uniform(static_cast<double*>(a->slab), a->elems, seed, stream_id, 0, lo, hi,
                                ex->stream);
    for (int64_t t = 0; t < a->ntiles; ++t) {
        int32_t lo3[3], ext[3];
        a->tile_extent(t, lo3, ext);
        int64_t e[3], o[3];
        for (int d = 0; d < 3; ++d) {
            e[d] = ext[d];
            o[d] = lo3[d];
        }
        if (int rc = cnh_fill_uniform_tile(static_cast<double*>(a->tiles[t]), a->ndims, e, o, gshape, seed,
                                           stream_id, lo, hi, ex->stream))
            return rc;
    }
    return 0;
}

int cnx_fill_cg_matrix(cnx_executor* ex, int name, uint64_t seed) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = settle(ex))
        return rc;
    XArray* a;
    if (int rc = find_array(ex, name, &a, "fill_cg_matrix"))
        return rc;
    CNH_CHECK(a->dtype == CNH_F64 && a->ndims == 2 && a->shape[0] == a->shape[1], -27,
              "fill_cg_matrix needs a square fp64 array");
    if (ex->trace_on) ex->log("fill_cg_matrix " + std::to_string(name));
    if (ex->dry)
        return 0;
    for (int64_t t = 0; t < a->ntiles; ++t) {
        int32_t lo[3], ext[3];
        a->tile_extent(t, lo, ext);
        int64_t tstr[3];
        a->tile_strides(ext, tstr);
        if (int rc = cnh_fill_cg_matrix(static_cast<double*>(a->tiles[t]), a->shape[0], lo[0], ext[0], lo[1],
                                        ext[1], tstr[0], seed, ex->stream))
            return rc;
    }
    return 0;
}

int cnx_sync(cnx_executor* ex) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = settle(ex))
        return rc;
    if (ex->dry)
        return 0;
    return cnh_stream_sync(ex->stream);
}

int cnx_array_info(cnx_executor* ex, int name, int* ndims, int* dtype, int* tile, int32_t* shape3,
                   int32_t* offset3) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = settle(ex))
        return rc;
    XArray* a;
    if (int rc = find_array(ex, name, &a, "array_info"))
        return rc;
    if (ndims)
        *ndims = a->ndims;
    if (dtype)
        *dtype = a->dtype;
    if (tile)
        *tile = a->tile;
    for (int d = 0; d < 3; ++d) {
        if (shape3)
            shape3[d] = a->shape[d];
        if (offset3)
            offset3[d] = a->offset[d];
    }
    return 0;
}

int cnx_set_matvec_timing(cnx_executor* ex, int on) {
    CNH_CHECK(ex != nullptr, -2, "null executor");
    if (int rc = settle(ex))
        return rc;
    ex->time_matvec = on != 0;
    for (auto& pr : ex->matvec_events) {
        cnh_event_destroy(pr.first);
        cnh_event_destroy(pr.second);
    }
    ex->matvec_events.clear();
    return 0;
}

int64_t cnx_matvec_times(cnx_executor* ex, float* ms, int64_t cap) {
    CNH_CHECK(ex != nullptr && (ms != nullptr || cap == 0), -2, "bad arguments");
    if (int rc = settle(ex))
        return rc;
    if (!ex->dry)
        if (int rc = cnh_stream_sync(ex->stream))
            return rc;
    int64_t n = 0;
    for (auto& pr : ex->matvec_events) {
        if (n < cap) {
            if (int rc = cnh_event_elapsed_ms(pr.first, pr.second, &ms[n]))
                return rc;
            ++n;
        }
        cnh_event_destroy(pr.first);
        cnh_event_destroy(pr.second);
    }
    ex->matvec_events.clear();
    return n;
}

int cnx_stats(cnx_executor* ex, int64_t out[8]) {
    CNH_CHECK(ex != nullptr && out != nullptr, -2, "null argument");
    if (int rc = drain(ex))
        return rc;
    ex->stats[6] = (int64_t)ex->arrays.size();
    for (int i = 0; i < 8; ++i)
        out[i] = ex->stats[i];
    return 0;
}

int cnx_solve_decompositions(int odf, int num_pes, const int32_t min_tile[3], int n_arrays,
                             cnx_decomp* arrays, int64_t size, const char* msg) {
    CNH_CHECK(min_tile != nullptr && n_arrays >= 0 && (n_arrays == 0 || arrays != nullptr), -2,
              "null argument");
    CNH_CHECK(size == 0 || msg != nullptr, -2, "null DAG message");
    std::vector<DagNode> dag;
    if (size > 0)
        if (int rc = parse_dag(msg, size, dag))
            return rc;
    std::map<int, DecompMeta> meta;
    for (int i = 0; i < n_arrays; ++i) {
        const cnx_decomp& a = arrays[i];
        CNH_CHECK(a.ndims >= 1 && a.ndims <= 3 && a.tile >= 0, -20, "array %d: rank %d, tile %d", a.name,
                  a.ndims, a.tile);
        CNH_CHECK(meta.find(a.name) == meta.end(), -21, "array %d listed twice", a.name);
        DecompMeta m;
        m.ndims = a.ndims;
        m.tile = a.tile;
        m.final = a.final != 0;
        for (int d = 0; d < 3; ++d) {
            CNH_CHECK(d >= a.ndims || a.shape[d] >= 1, -20, "array %d: extent %d in dim %d", a.name,
                      a.shape[d], d);
            m.shape[d] = d < a.ndims ? a.shape[d] : 0;
            m.offset[d] = d < a.ndims ? a.offset[d] : 0;
        }
        meta[a.name] = m;
    }
    const int mt[4] = {1, min_tile[0], min_tile[1], min_tile[2]};
    for (int r = 1; r <= 3; ++r)
        CNH_CHECK(mt[r] >= 1 && mt[r] <= (1 << 30), -20, "minimum tile %d for rank %d", mt[r], r);
    solve_decompositions(meta, dag, odf, num_pes, mt);
    for (int i = 0; i < n_arrays; ++i) {
        const DecompMeta& m = meta[arrays[i].name];
        arrays[i].tile = m.tile;
        arrays[i].final = 1;
        for (int d = 0; d < 3; ++d)
            arrays[i].offset[d] = m.offset[d];
    }
    return 0;
}

} // extern "C"
