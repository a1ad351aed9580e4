// Statement log: record parsing, the hold-back rule of automatic flushes, and the planner that
// groups recorded operations into DAG nodes. Pure host code.
//
// Record layout (little endian, int32 words unless noted):
//   delete      := 5, name
//   create      := head, shape
//   op          := head, shape, operand * n_operands          element-wise, n_operands <= 2
//   nonfusible  := head, shape, operand * n_operands          reductions, products, tile, diag
//   set         := head, shape, region, operand               target[region] = operand
//   head        := kind, name, opcode, dtype, n_operands, aux (set: rank of the target array)
//   shape       := ndims, extent[3]                           of the result / of the assigned region
//   region      := ndims, start[3], stop[3], step[3]
//   operand     := 0, 0, float64 value                        a literal
//                | 1, name, base_ndims, dtype, broadcast, has_region, start[3], stop[3], step[3]
#include "stmtlog.h"
#include "../../include/cnexec.h"
#include "common.h"

#include <cstring>

namespace cnh {
namespace stmtlog {

namespace {

// int32 -> int32 table for array names (open addressing, sized for the batch at hand): the planner
// looks names up a few times per record, and tree or node-based tables spend more time in the
// allocator than in the plan.
class NameTable {
public:
    explicit NameTable(size_t expected) {
        size_t cap = 16;
        while (cap < expected * 2 + 2)
            cap *= 2;
        keys_.assign(cap, kEmpty);
        vals_.assign(cap, 0);
    }
    int32_t* find(int32_t key) {
        const size_t i = slot(key);
        return keys_[i] == key ? &vals_[i] : nullptr;
    }
    const int32_t* find(int32_t key) const { return const_cast<NameTable*>(this)->find(key); }
    bool has(int32_t key) const { return find(key) != nullptr; }
    // the value for `key`, inserted as `fresh` when new
    int32_t& at(int32_t key, int32_t fresh = 0) {
        if ((count_ + 1) * 2 > keys_.size())
            grow();
        const size_t i = slot(key);
        if (keys_[i] != key) {
            keys_[i] = key;
            vals_[i] = fresh;
            ++count_;
        }
        return vals_[i];
    }
    void insert(int32_t key) { (void)at(key, 1); }

private:
    static constexpr int32_t kEmpty = INT32_MIN;     // no record carries this name
    size_t slot(int32_t key) const {
        size_t i = ((uint32_t)key * 2654435761u) & (keys_.size() - 1);
        while (keys_[i] != kEmpty && keys_[i] != key)
            i = (i + 1) & (keys_.size() - 1);
        return i;
    }
    void grow() {
        std::vector<int32_t> k(keys_.size() * 2, kEmpty), v(keys_.size() * 2, 0);
        k.swap(keys_);
        v.swap(vals_);
        count_ = 0;
        for (size_t i = 0; i < k.size(); ++i)
            if (k[i] != kEmpty)
                at(k[i]) = v[i];
    }
    std::vector<int32_t> keys_, vals_;
    size_t count_ = 0;
};

struct Words {
    const char* p;
    const char* end;
    bool ok = true;
    int32_t i32() {
        int32_t v = 0;
        if (!ok || end - p < 4) {
            ok = false;
            return 0;
        }
        std::memcpy(&v, p, 4);
        p += 4;
        return v;
    }
    double f64() {
        double v = 0;
        if (!ok || end - p < 8) {
            ok = false;
            return 0;
        }
        std::memcpy(&v, p, 8);
        p += 8;
        return v;
    }
};

bool read_box(Words& w, cnh_region& r) {
    std::memset(&r, 0, sizeof r);
    r.ndims = w.i32();
    int32_t v[9];
    for (int32_t& x : v)
        x = w.i32();
    if (!w.ok || r.ndims < 1 || r.ndims > 3)
        return false;
    for (int d = 0; d < r.ndims; ++d) {
        r.start[d] = v[d];
        r.stop[d] = v[3 + d];
        r.step[d] = v[6 + d];
    }
    return true;
}

cnh_region global_region() {
    cnh_region r;
    std::memset(&r, 0, sizeof r);
    r.is_global = 1;
    return r;
}

cnh_region full_region(const int32_t* shape, int nd) {
    cnh_region r;
    std::memset(&r, 0, sizeof r);
    r.ndims = nd;
    for (int d = 0; d < nd; ++d) {
        r.stop[d] = shape[d];
        r.step[d] = 1;
    }
    return r;
}

bool same_shape(const Instr& a, const int32_t* shape, int nd) {
    if (a.ndims != nd)
        return false;
    for (int d = 0; d < nd; ++d)
        if (a.shape[d] != shape[d])
            return false;
    return true;
}

// The AST nodes of one DAG node while it is put together.
struct NodeWriter {
    DagNode node;
    struct Leaf { int32_t name, broadcast, index; };
    std::vector<Leaf> leaves;          // a node has a handful of leaves: a list beats a tree
    int32_t next_scalar = -1;

    int32_t add(int32_t name, int32_t opcode, bool is_temp, bool is_scalar, bool is_bc, int32_t ndims,
                int32_t dtype, double scalar) {
        cnh_ast_node a;
        std::memset(&a, 0, sizeof a);
        a.result_name = name;
        a.opcode = opcode;
        a.is_temp = is_temp;
        a.is_scalar = is_scalar;
        a.is_broadcast = is_bc;
        a.ndims = ndims;
        a.dtype = dtype;
        a.scalar = scalar;
        a.region = global_region();
        node.nodes.push_back(a);
        return (int32_t)node.nodes.size() - 1;
    }
    int32_t leaf(int32_t name, bool broadcast, int32_t base_ndims, int32_t dtype) {
        for (const Leaf& l : leaves)
            if (l.name == name && l.broadcast == (int32_t)broadcast)
                return l.index;
        const int32_t idx = add(name, CNH_OP_NOOP, false, false, broadcast, base_ndims, dtype, 0.0);
        leaves.push_back({name, (int32_t)broadcast, idx});
        return idx;
    }
    int32_t leaf(const Ref& r) { return leaf(r.name, r.broadcast != 0, r.base_ndims, r.dtype); }
    int32_t scalar(double value, int32_t ndims, int32_t dtype) {
        return add(next_scalar--, CNH_OP_NOOP, false, true, false, ndims, dtype, value);
    }
    // an operation over `n` operands (node indices with their regions); always a root
    int32_t op(int32_t name, int32_t opcode, bool is_temp, int32_t ndims, int32_t dtype, int n,
               const int32_t* operands, const cnh_region* const* regions, const cnh_region& region) {
        const int32_t idx = add(name, opcode, is_temp, false, false, ndims, dtype, 0.0);
        cnh_ast_node& a = node.nodes.back();
        a.n_operands = n;
        for (int j = 0; j < n; ++j) {
            a.operands[j] = operands[j];
            a.has_operand_region[j] = regions[j] != nullptr;
            a.operand_regions[j] = regions[j] != nullptr ? *regions[j] : global_region();
        }
        a.region = region;
        node.roots.push_back(idx);
        return idx;
    }
};

struct Group {
    std::vector<int> ops;
    int set_idx = -1;
    int32_t shape[3] = {0, 0, 0};
    int nd = 0;
    int32_t dtype = 0;
};

enum ItemKind { kItemGroup, kItemInstr, kItemDelete };
struct Item {
    ItemKind kind;
    int what;   // group number | instruction index | array name
};

} // namespace

int parse(const char* log, int64_t size, std::vector<Instr>& out) {
    Words w{log, log + size};
    while (w.ok && w.p < w.end) {
        Instr in;
        in.region = global_region();
        in.kind = w.i32();
        in.name = w.i32();
        if (in.kind == kDelete) {
            CNH_CHECK(w.ok, -43, "statement log truncated");
            out.push_back(in);
            continue;
        }
        CNH_CHECK(w.ok && in.kind >= kCreate && in.kind <= kNonfusible, -43,
                  "statement log: record kind %d", in.kind);
        in.opcode = w.i32();
        in.dtype = w.i32();
        in.n_operands = w.i32();
        in.target_ndims = w.i32();
        in.ndims = w.i32();
        for (int32_t& s : in.shape)
            s = w.i32();
        CNH_CHECK(w.ok, -43, "statement log truncated");
        CNH_CHECK(in.ndims >= 1 && in.ndims <= 3 && in.n_operands >= 0 && in.n_operands <= 2, -43,
                  "statement log: record of rank %d with %d operands", in.ndims, in.n_operands);
        CNH_CHECK(in.dtype >= 0 && in.dtype <= 3, -43, "statement log: element type %d", in.dtype);
        if (in.kind == kSet) {
            CNH_CHECK(read_box(w, in.region) && in.n_operands == 1 && in.target_ndims >= 1 &&
                          in.target_ndims <= 3,
                      -43, "statement log: malformed assignment into array %d", in.name);
        }
        for (int j = 0; j < in.n_operands; ++j) {
            Ref& r = in.operands[j];
            r.region = global_region();
            const int32_t tag = w.i32();
            if (tag == 0) {
                (void)w.i32();
                r.scalar = w.f64();
                continue;
            }
            CNH_CHECK(w.ok && tag == 1, -43, "statement log: operand tag %d", tag);
            r.is_array = true;
            r.name = w.i32();
            r.base_ndims = w.i32();
            r.dtype = w.i32();
            r.broadcast = w.i32();
            r.has_region = w.i32() != 0;
            int32_t v[9];
            for (int32_t& x : v)
                x = w.i32();
            CNH_CHECK(w.ok && r.base_ndims >= 1 && r.base_ndims <= 3, -43,
                      "statement log: operand of rank %d", r.base_ndims);
            if (r.has_region) {
                std::memset(&r.region, 0, sizeof r.region);
                r.region.ndims = r.base_ndims;
                for (int d = 0; d < r.base_ndims; ++d) {
                    r.region.start[d] = v[d];
                    r.region.stop[d] = v[3 + d];
                    r.region.step[d] = v[6 + d];
                }
            }
        }
        CNH_CHECK(w.ok, -43, "statement log truncated");
        out.push_back(in);
    }
    CNH_CHECK(w.ok, -43, "statement log truncated");
    return 0;
}

size_t hold_back_cut(const std::vector<Instr>& batch, int window) {
    const size_t n = batch.size();
    NameTable deleted(n);
    for (const Instr& in : batch)
        if (in.kind == kDelete)
            deleted.insert(in.name);
    size_t first_live = n;
    for (size_t i = n > (size_t)std::max(0, window) ? n - (size_t)window : 0; i < n; ++i)
        if (batch[i].kind == kOp && !deleted.has(batch[i].name)) {
            first_live = i;
            break;
        }
    if (first_live == n)
        return n;
    // the last statement boundary at or before that producer: a position whose predecessor
    // (deletions aside) is not an element-wise operation
    size_t cut = first_live;
    while (cut > 0) {
        std::ptrdiff_t j = (std::ptrdiff_t)cut - 1;
        while (j >= 0 && batch[(size_t)j].kind == kDelete)
            --j;
        if (j < 0 || batch[(size_t)j].kind != kOp)
            break;
        --cut;
    }
    return cut > 0 ? cut : n;
}

std::set<int32_t> dead_later(const std::vector<Instr>& batch, size_t cut) {
    NameTable touched(batch.size()), produced(batch.size());
    for (size_t i = cut; i < batch.size(); ++i) {
        const Instr& in = batch[i];
        if (in.kind == kDelete)
            continue;
        for (int j = 0; j < in.n_operands; ++j)
            if (in.operands[j].is_array)
                touched.insert(in.operands[j].name);
        if (in.kind == kSet)
            touched.insert(in.name);
    }
    for (size_t i = 0; i < cut; ++i)
        if (batch[i].kind == kOp)
            produced.insert(batch[i].name);
    std::set<int32_t> out;
    for (size_t i = cut; i < batch.size(); ++i)
        if (batch[i].kind == kDelete && produced.has(batch[i].name) && !touched.has(batch[i].name))
            out.insert(batch[i].name);
    return out;
}

void plan(const std::vector<Instr>& batch, size_t count, const std::set<int32_t>& dead,
          int32_t* next_set_name, std::vector<DagNode>& out, std::set<int32_t>* fused_away) {
    const int n = (int)count;
    NameTable producer((size_t)n);                    // result name -> index of the operation
    NameTable deleted((size_t)n + dead.size());
    for (int32_t name : dead)
        deleted.insert(name);
    for (int i = 0; i < n; ++i) {
        if (batch[(size_t)i].kind == kOp)
            producer.at(batch[(size_t)i].name) = i;
        else if (batch[(size_t)i].kind == kDelete)
            deleted.insert(batch[(size_t)i].name);
    }
    std::vector<char> dropped((size_t)n, 0);          // dead code: operations never emitted
    NameTable forced((size_t)n);                      // results that must exist as arrays

    // Who reads the result of operation p (as instruction indices; -(i+1) marks instruction i
    // assigning into it, which always counts as a use from outside any group): built once, as
    // one list with an offset per operation; readers dropped later are skipped when it is read.
    std::vector<int> use_first((size_t)n + 1, 0), use_list;
    {
        auto reader_of = [&](int32_t name) -> int {
            const int32_t* p = producer.find(name);
            return p != nullptr ? *p : -1;
        };
        for (int pass = 0; pass < 2; ++pass) {
            std::vector<int> fill;
            if (pass == 1) {
                for (int i = 0; i < n; ++i)
                    use_first[(size_t)i + 1] += use_first[(size_t)i];
                use_list.assign((size_t)use_first[(size_t)n], 0);
                fill.assign(use_first.begin(), use_first.end() - 1);
            }
            for (int i = 0; i < n; ++i) {
                const Instr& in = batch[(size_t)i];
                if (in.kind == kDelete || in.kind == kCreate)
                    continue;
                for (int j = 0; j < in.n_operands; ++j)
                    if (in.operands[j].is_array) {
                        const int p = reader_of(in.operands[j].name);
                        if (p >= 0) {
                            if (pass == 0) use_first[(size_t)p + 1]++;
                            else use_list[(size_t)fill[(size_t)p]++] = i;
                        }
                    }
                if (in.kind == kSet) {
                    const int p = reader_of(in.name);
                    if (p >= 0) {
                        if (pass == 0) use_first[(size_t)p + 1]++;
                        else use_list[(size_t)fill[(size_t)p]++] = -(i + 1);
                    }
                }
            }
        }
    }

    std::vector<Item> items;
    std::vector<Group> groups;
    std::vector<int> group_of;
    for (;;) {
        items.clear();
        groups.clear();
        group_of.assign((size_t)n, -1);
        int cur = -1;
        std::vector<int32_t> deferred;
        auto close = [&]() {
            if (cur >= 0 && !groups[(size_t)cur].ops.empty())
                items.push_back({kItemGroup, cur});
            cur = -1;
            for (int32_t name : deferred)
                items.push_back({kItemDelete, name});
            deferred.clear();
        };
        for (int i = 0; i < n; ++i) {
            if (dropped[(size_t)i])
                continue;
            const Instr& in = batch[(size_t)i];
            if (in.kind == kOp) {
                bool reads_slice_of_own = false;
                if (cur >= 0)
                    for (int j = 0; j < in.n_operands; ++j) {
                        const Ref& o = in.operands[j];
                        if (o.is_array && o.has_region) {
                            // a slice of a result of the group that is open right now
                            const int32_t* p = producer.find(o.name);
                            reads_slice_of_own = reads_slice_of_own ||
                                                 (p != nullptr && !dropped[(size_t)*p] && group_of[(size_t)*p] == cur);
                        }
                    }
                if (cur < 0 || !same_shape(in, groups[(size_t)cur].shape, groups[(size_t)cur].nd) ||
                    groups[(size_t)cur].dtype != in.dtype || reads_slice_of_own) {
                    close();
                    groups.emplace_back();
                    cur = (int)groups.size() - 1;
                    Group& g = groups.back();
                    g.nd = in.ndims;
                    std::memcpy(g.shape, in.shape, sizeof g.shape);
                    g.dtype = in.dtype;
                }
                groups[(size_t)cur].ops.push_back(i);
                group_of[(size_t)i] = cur;
                if (forced.has(in.name))
                    close();
            } else if (in.kind == kDelete) {
                const int32_t* p = producer.find(in.name);
                if (p != nullptr && dropped[(size_t)*p])
                    continue;
                deferred.push_back(in.name);
                if (cur < 0)
                    close();
            } else if (in.kind == kSet) {
                const Ref& v = in.operands[0];
                const bool fuse = cur >= 0 && v.is_array && !v.has_region &&
                                  batch[(size_t)groups[(size_t)cur].ops.back()].name == v.name &&
                                  !forced.has(v.name) && !v.broadcast &&
                                  groups[(size_t)cur].nd == in.target_ndims && groups[(size_t)cur].dtype == in.dtype;
                if (fuse) {
                    groups[(size_t)cur].set_idx = i;
                    group_of[(size_t)i] = cur;
                    close();
                } else {
                    close();
                    items.push_back({kItemInstr, i});
                }
            } else {
                close();
                items.push_back({kItemInstr, i});
            }
        }
        close();

        bool changed = false;
        for (int i = 0; i < n; ++i) {
            const Instr& in = batch[(size_t)i];
            if (in.kind != kOp || dropped[(size_t)i])
                continue;
            const int gi = group_of[(size_t)i];
            const Group& g = groups[(size_t)gi];
            // the readers of this result that are still part of the program (a result computed
            // twice under one name does not occur: names are handed out once)
            const int32_t* own = producer.find(in.name);
            const int first = own != nullptr && *own == i ? use_first[(size_t)i] : 0;
            const int past = own != nullptr && *own == i ? use_first[(size_t)i + 1] : 0;
            bool any_reader = false, inside = true;
            for (int q = first; q < past; ++q) {
                const int x = use_list[(size_t)q];
                if (x >= 0 && dropped[(size_t)x])
                    continue;
                any_reader = true;
                inside = inside && x >= 0 && group_of[(size_t)x] == gi;
            }
            const bool is_dead = deleted.has(in.name);
            if (is_dead && !any_reader) {
                dropped[(size_t)i] = 1;       // computed, never read, handle gone
                changed = true;
                continue;
            }
            const bool is_last = g.ops.back() == i;
            const bool temp_ok = is_dead && inside && (!is_last || g.set_idx >= 0);
            if (!temp_ok && !forced.has(in.name)) {
                // must exist as an array: its group has to end here
                if (!(is_last && g.set_idx < 0)) {
                    forced.insert(in.name);
                    changed = true;
                }
            }
        }
        if (!changed)
            break;
    }

    // ---- emission ----
    NameTable materialised((size_t)n);
    int node_id = 0;
    for (const Item& item : items) {
        if (item.kind == kItemDelete) {
            if (producer.has(item.what) && !materialised.has(item.what))
                continue;               // a temporary: it never became an array
            NodeWriter w;
            w.node.id = node_id++;
            w.node.fusible = 0;
            const int32_t idx = w.add(item.what, CNX_OP_DELETE, false, false, false, 1, CNH_F64, 0.0);
            w.node.roots.push_back(idx);
            out.push_back(std::move(w.node));
            continue;
        }
        NodeWriter w;
        w.node.id = node_id++;
        if (item.kind == kItemGroup) {
            const Group& g = groups[(size_t)item.what];
            NameTable index_of(g.ops.size());                 // result name -> AST node of this group
            const int last = g.ops.back();
            for (int i : g.ops) {
                const Instr& in = batch[(size_t)i];
                int32_t opnds[2] = {0, 0};
                const cnh_region* oregs[2] = {nullptr, nullptr};
                for (int j = 0; j < in.n_operands; ++j) {
                    const Ref& o = in.operands[j];
                    if (o.is_array) {
                        const int32_t* it = index_of.find(o.name);
                        if (it != nullptr && !o.has_region) {
                            opnds[j] = *it;
                        } else {
                            opnds[j] = w.leaf(o);
                            oregs[j] = o.has_region ? &o.region : nullptr;
                        }
                    } else {
                        opnds[j] = w.scalar(o.scalar, g.nd, in.dtype);
                    }
                }
                const bool is_root_result = i == last && g.set_idx < 0;
                index_of.at(in.name) = w.op(in.name, in.opcode, !is_root_result, g.nd, in.dtype, in.n_operands, opnds,
                                            oregs, is_root_result ? full_region(in.shape, in.ndims) : global_region());
            }
            if (g.set_idx >= 0) {
                const Instr& s = batch[(size_t)g.set_idx];
                const int32_t opnds[2] = {w.leaf(s.name, false, s.target_ndims, s.dtype),
                                          index_of.at(batch[(size_t)last].name)};
                const cnh_region* oregs[2] = {nullptr, nullptr};
                w.op((*next_set_name)++, CNH_OP_SET_REGION, false, s.target_ndims, s.dtype, 2, opnds, oregs, s.region);
            } else {
                materialised.insert(batch[(size_t)last].name);
            }
            w.node.fusible = 1;
        } else {
            const Instr& in = batch[(size_t)item.what];
            if (in.kind == kCreate) {
                w.op(in.name, CNH_OP_CREATE, false, in.ndims, in.dtype, 0, nullptr, nullptr,
                     full_region(in.shape, in.ndims));
                w.node.fusible = 0;
            } else if (in.kind == kSet) {
                const Ref& v = in.operands[0];
                int32_t opnds[2];
                const cnh_region* oregs[2] = {nullptr, nullptr};
                opnds[0] = w.leaf(in.name, false, in.target_ndims, in.dtype);
                if (v.is_array) {
                    opnds[1] = w.leaf(v);
                    oregs[1] = v.has_region ? &v.region : nullptr;
                } else {
                    opnds[1] = w.scalar(v.scalar, in.target_ndims, in.dtype);
                }
                w.op((*next_set_name)++, CNH_OP_SET_REGION, false, in.target_ndims, in.dtype, 2, opnds, oregs,
                     in.region);
                w.node.fusible = v.is_array ? 1 : 0;
            } else {   // kNonfusible
                int32_t opnds[2] = {0, 0};
                const cnh_region* oregs[2] = {nullptr, nullptr};
                for (int j = 0; j < in.n_operands; ++j) {
                    const Ref& o = in.operands[j];
                    if (o.is_array) {
                        opnds[j] = w.leaf(o);
                        oregs[j] = o.has_region ? &o.region : nullptr;
                    } else {
                        opnds[j] = w.scalar(o.scalar, in.ndims, in.dtype);
                    }
                }
                w.op(in.name, in.opcode, false, in.ndims, in.dtype, in.n_operands, opnds, oregs,
                     full_region(in.shape, in.ndims));
                w.node.fusible = 0;
            }
        }
        out.push_back(std::move(w.node));
    }
    if (fused_away != nullptr)
        for (int32_t name : dead)
            if (producer.has(name) && !materialised.has(name))
                fused_away->insert(name);
}

std::vector<char> to_message(const std::vector<DagNode>& nodes) {
    std::vector<char> out;
    auto put32 = [&](int32_t v) {
        const char* p = reinterpret_cast<const char*>(&v);
        out.insert(out.end(), p, p + 4);
    };
    auto put_region = [&](const cnh_region& r) {
        put32(r.is_global ? 1 : 0);
        if (r.is_global)
            return;
        put32(r.ndims);
        for (int d = 0; d < r.ndims; ++d) {
            put32(r.start[d]);
            put32(r.stop[d]);
            put32(r.step[d]);
        }
    };
    put32(CNX_DAG_MAGIC);
    put32(1);
    put32((int32_t)nodes.size());
    for (const DagNode& n : nodes) {
        put32(n.id);
        put32(n.fusible);
        put32((int32_t)n.nodes.size());
        put32((int32_t)n.roots.size());
        for (const cnh_ast_node& a : n.nodes) {
            put32(a.result_name);
            put32(a.opcode);
            put32(a.is_temp);
            put32(a.is_scalar);
            put32(a.is_broadcast);
            put32(a.ndims);
            put32(a.dtype);
            put32(a.n_operands);
            for (int j = 0; j < a.n_operands; ++j)
                put32(a.operands[j]);
            const char* p = reinterpret_cast<const char*>(&a.scalar);
            out.insert(out.end(), p, p + 8);
            for (int j = 0; j < a.n_operands; ++j) {
                cnh_region r = a.operand_regions[j];
                if (!a.has_operand_region[j])
                    r.is_global = 1;
                put_region(r);
            }
            put_region(a.region);
        }
        for (int32_t r : n.roots)
            put32(r);
    }
    return out;
}

} // namespace stmtlog
} // namespace cnh
