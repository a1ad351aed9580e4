// Tile and offset planning, restated from src/decomposition_solver.hpp:94-1714.
//
// What it decides, in upstream's order:
//   1. every undecided array starts from the tile rule (power of two >= the rank's minimum, doubled
//      until the array has at most odf * PEs tiles) with offset 0            (:113-122)
//   2. tiles shrink along data flow: a result read through a region of step s takes its source's
//      tile / gcd of the steps, a lower-rank partner of a cross-rank assignment takes the
//      higher-rank tile; repeated to a fixed point, then clamped again       (:211-380)
//   3. arrays that an elementwise statement combines without a shift form one class (:478-597)
//   4. every shifted or strided read, and every assignment into a region, is an edge between two
//      classes that says which offset of one would line its tiles up with the other (:619-811)
//   5. per connected component without a cycle: a tree rooted at a class whose offset is fixed,
//      candidate phases collected up and down the tree, a per-dimension dynamic programme over
//      them weighted by the volume each edge moves, and absolute offsets chosen closest to what
//      the edges ask for                                                     (:813-1499)
//   6. components with a cycle: each array separately, from the offsets its producers and
//      consumers would like                                                  (:1501-1703)
//   7. operands and results of matrix products keep offset 0                 (:1705-1709)
#include "decomp.h"

#include <algorithm>
#include <array>
#include <limits>
#include <queue>
#include <set>

namespace cnh {
namespace {

using I3 = std::array<int, 3>;
constexpr int64_t kInf = std::numeric_limits<int64_t>::max() / 2;

int next_pow2(int v) {
    int p = 1;
    while (p < v && p < (1 << 30))
        p *= 2;
    return p;
}

int pmod(int v, int m) {
    int r = v % m;
    return r < 0 ? r + m : r;
}

int pmod64(int64_t v, int m) {
    if (m <= 0)
        return (int)v;
    int64_t r = v % m;
    return (int)(r < 0 ? r + m : r);
}

int64_t dist64(int64_t a, int64_t b) { return a >= b ? a - b : b - a; }

int gcd_abs(int a, int b) {
    a = a < 0 ? -a : a;
    b = b < 0 ? -b : b;
    while (b) {
        int t = a % b;
        a = b;
        b = t;
    }
    return a;
}

int circ_dist(int a, int b, int m) {
    int d = ((a - b) % m + m) % m;
    return std::min(d, m - d);
}

bool skipped(const cnh_ast_node& n) { return n.is_scalar || n.is_broadcast; }

// The region an operand is read through; nullptr for "the whole array".
const cnh_region* operand_region(const cnh_ast_node& n, int j) {
    if (j >= n.n_operands || !n.has_operand_region[j] || n.operand_regions[j].is_global)
        return nullptr;
    return &n.operand_regions[j];
}

const cnh_region* node_region(const cnh_ast_node& n) { return n.region.is_global ? nullptr : &n.region; }

bool is_leaf(const DagNode& dn, const cnh_ast_node& n) {
    for (int j = 0; j < n.n_operands; ++j)
        if (!skipped(dn.nodes[n.operands[j]]))
            return false;
    return true;
}

bool elementwise_or_copy(int op) {
    return op == CNH_OP_ADD || op == CNH_OP_SUB || op == CNH_OP_MUL || op == CNH_OP_DIV ||
           op == CNH_OP_TANH || op == CNH_OP_EXP || op == CNH_OP_COPY;
}

I3 region_start(const cnh_region* r, int nd) {
    I3 s = {0, 0, 0};
    if (r)
        for (int d = 0; d < nd && d < r->ndims; ++d)
            s[d] = r->start[d];
    return s;
}

I3 region_step(const cnh_region* r, int nd) {
    I3 s = {1, 1, 1};
    if (r)
        for (int d = 0; d < nd && d < r->ndims; ++d)
            s[d] = r->step[d];
    return s;
}

I3 region_stop(const cnh_region* r, int nd, const int32_t* shape) {
    I3 s = {0, 0, 0};
    for (int d = 0; d < nd; ++d)
        s[d] = r && d < r->ndims ? r->stop[d] : shape[d];
    return s;
}

int stride_factor(const cnh_region* r, int nd) {
    int f = 0;
    if (r)
        for (int d = 0; d < nd && d < r->ndims; ++d) {
            int s = r->step[d] < 0 ? -r->step[d] : r->step[d];
            if (s > 1)
                f = f ? gcd_abs(f, s) : s;
        }
    return f > 1 ? f : 1;
}

bool region_dense(const cnh_region* r, int nd) {
    if (r)
        for (int d = 0; d < nd && d < r->ndims; ++d)
            if (r->step[d] != 1)
                return false;
    return true;
}

struct ClassInfo {
    int tile = 0, ndims = 0;
    bool fixed = false;
    I3 offset = {0, 0, 0};
};

// "offset_to = (offset_from + shift) / stride lines the tiles of `to` up with those of `from`."
struct ShiftEdge {
    int from, to;
    I3 shift, stride;
    int64_t weight;
    I3 from_to_to = {0, 1, 2}, to_to_from = {0, 1, 2};
};

struct AdjEdge {
    int neighbor;
    I3 shift, stride, neighbor_dim;
    int64_t weight;
    bool forward; // the owner of this entry is the edge's `from`
};

struct Proposal {
    int value;
    int64_t weight;
};

struct Solver {
    std::map<int, DecompMeta>& meta;
    const std::vector<DagNode>& dag;
    int odf, pes;
    const int* min_tile;

    int min_edge(int nd) const { return nd >= 1 && nd <= 3 ? std::max(1, min_tile[nd]) : 1; }

    void clamp(DecompMeta& m) const {
        int64_t cap = (int64_t)std::max(1, odf) * std::max(1, pes);
        for (;;) {
            int64_t count = 1;
            for (int d = 0; d < m.ndims; ++d)
                count *= (m.shape[d] + m.tile - 1) / m.tile;
            if (count <= cap || m.tile >= (1 << 30))
                return;
            m.tile *= 2;
        }
    }

    DecompMeta* find(int name) {
        auto it = meta.find(name);
        return it == meta.end() ? nullptr : &it->second;
    }

    // ---- 2. tile propagation (:211-380) ----
    bool try_assign(int name, int cand) {
        DecompMeta* m = find(name);
        if (!m || m->final || cand <= 0)
            return false;
        cand = std::max(next_pow2(cand), min_edge(m->ndims));
        if (m->tile > 0 && cand >= m->tile)
            return false;
        m->tile = cand;
        return true;
    }

    bool propose(int name, int nd, int source, const cnh_region* access) {
        if (source == name)
            return false;
        DecompMeta* s = find(source);
        if (!s || s->ndims != nd)
            return false;
        int cand = s->tile, f = stride_factor(access, nd);
        if (f > 1)
            cand = std::max(1, cand / f);
        return try_assign(name, cand);
    }

    bool collect_tiles(const DagNode& dn, const std::map<int, int>& temp_defs, int name, int nd,
                       int idx, const cnh_region* carried) {
        const cnh_ast_node& n = dn.nodes[idx];
        if (skipped(n))
            return false;
        if (DecompMeta* m = find(n.result_name))
            return m->ndims == nd ? propose(name, nd, n.result_name, carried) : false;
        bool changed = false;
        if (n.n_operands == 0) {
            auto def = temp_defs.find(n.result_name);
            if (def == temp_defs.end())
                return false;
            const cnh_ast_node& root = dn.nodes[def->second];
            for (int j = 0; j < root.n_operands; ++j)
                changed = collect_tiles(dn, temp_defs, name, nd, root.operands[j],
                                        operand_region(root, j)) || changed;
            return changed;
        }
        for (int j = 0; j < n.n_operands; ++j)
            changed = collect_tiles(dn, temp_defs, name, nd, n.operands[j], operand_region(n, j)) ||
                      changed;
        return changed;
    }

    void propagate_tiles() {
        bool changed = true;
        int passes = std::max<int>(64, (int)meta.size());
        for (int it = 0; it < passes && changed; ++it) {
            changed = false;
            for (const DagNode& dn : dag) {
                std::map<int, int> temp_defs;
                for (int r : dn.roots)
                    if (dn.nodes[r].is_temp)
                        temp_defs[dn.nodes[r].result_name] = r;
                for (int r : dn.roots) {
                    const cnh_ast_node& root = dn.nodes[r];
                    if (root.opcode == CNH_OP_SET_REGION) {
                        if (root.n_operands < 2)
                            continue;
                        int dst_name = dn.nodes[root.operands[0]].result_name;
                        DecompMeta* dst = find(dst_name);
                        if (!dst)
                            continue;
                        if (region_dense(node_region(root), dst->ndims))
                            for (int j = 1; j < root.n_operands; ++j)
                                changed = collect_tiles(dn, temp_defs, dst_name, dst->ndims,
                                                        root.operands[j], operand_region(root, j)) ||
                                          changed;
                        for (int j = 1; j < root.n_operands; ++j) {
                            const cnh_ast_node& src = dn.nodes[root.operands[j]];
                            if (!is_leaf(dn, src))
                                continue;
                            DecompMeta* sm = find(src.result_name);
                            if (!sm || sm->ndims == dst->ndims)
                                continue;
                            bool src_higher = sm->ndims > dst->ndims;
                            changed = try_assign(src_higher ? dst_name : src.result_name,
                                                 src_higher ? sm->tile : dst->tile) || changed;
                        }
                    } else if (elementwise_or_copy(root.opcode)) {
                        DecompMeta* out = find(root.result_name);
                        if (!out)
                            continue;
                        int nd = out->ndims;
                        for (int j = 0; j < root.n_operands; ++j)
                            changed = collect_tiles(dn, temp_defs, root.result_name, nd,
                                                    root.operands[j], operand_region(root, j)) ||
                                      changed;
                    }
                }
            }
        }
        for (auto& kv : meta)
            if (!kv.second.final)
                clamp(kv.second);
    }

    // ---- 3. classes (:478-617) ----
    std::map<int, int> uf_parent, uf_rank;
    std::set<int> created, matmul_arrays;

    int uf_find(int x) {
        int r = x;
        while (uf_parent[r] != r)
            r = uf_parent[r];
        while (uf_parent[x] != r) {
            int next = uf_parent[x];
            uf_parent[x] = r;
            x = next;
        }
        return r;
    }

    void uf_unite(int x, int y) {
        int rx = uf_find(x), ry = uf_find(y);
        if (rx == ry)
            return;
        if (uf_rank[rx] < uf_rank[ry])
            std::swap(rx, ry);
        uf_parent[ry] = rx;
        if (uf_rank[rx] == uf_rank[ry])
            uf_rank[rx]++;
    }

    bool is_fixed(int name, const DecompMeta& m) const { return m.final || created.count(name); }

    void unshifted_leaves(const DagNode& dn, int idx, int out_name, int nd, int out_tile,
                          const cnh_region* carried, std::vector<int>& leaves) {
        const cnh_ast_node& n = dn.nodes[idx];
        if (skipped(n))
            return;
        if (is_leaf(dn, n)) {
            if (n.result_name == out_name)
                return;
            DecompMeta* s = find(n.result_name);
            if (!s || s->ndims != nd || s->tile != out_tile || is_fixed(n.result_name, *s))
                return;
            if (carried) {
                I3 st = region_start(carried, nd), sp = region_step(carried, nd);
                for (int d = 0; d < nd; ++d)
                    if (st[d] != 0 || sp[d] != 1)
                        return;
            }
            leaves.push_back(n.result_name);
            return;
        }
        for (int j = 0; j < n.n_operands; ++j) {
            if (skipped(dn.nodes[n.operands[j]]))
                continue;
            const cnh_region* r = operand_region(n, j);
            unshifted_leaves(dn, n.operands[j], out_name, nd, out_tile, r ? r : carried, leaves);
        }
    }

    void build_classes() {
        for (auto& kv : meta) {
            uf_parent[kv.first] = kv.first;
            uf_rank[kv.first] = 0;
        }
        for (const DagNode& dn : dag)
            for (int r : dn.roots)
                if (dn.nodes[r].opcode == CNH_OP_CREATE)
                    created.insert(dn.nodes[r].result_name);
        for (const DagNode& dn : dag)
            for (int r : dn.roots) {
                const cnh_ast_node& root = dn.nodes[r];
                if (elementwise_or_copy(root.opcode)) {
                    DecompMeta* out = find(root.result_name);
                    if (!out)
                        continue;
                    std::vector<int> leaves;
                    for (int j = 0; j < root.n_operands; ++j)
                        if (!skipped(dn.nodes[root.operands[j]]))
                            unshifted_leaves(dn, root.operands[j], root.result_name, out->ndims,
                                             out->tile, operand_region(root, j), leaves);
                    for (int s : leaves)
                        uf_unite(root.result_name, s);
                } else if (root.opcode == CNH_OP_MATMUL || root.opcode == CNH_OP_MATMATMUL) {
                    for (int j = 0; j < root.n_operands; ++j)
                        if (!dn.nodes[root.operands[j]].is_scalar)
                            matmul_arrays.insert(dn.nodes[root.operands[j]].result_name);
                    matmul_arrays.insert(root.result_name);
                }
            }
        for (auto& kv : meta) {
            int rep = uf_find(kv.first);
            bool fixed = is_fixed(kv.first, kv.second);
            auto it = classes.find(rep);
            if (it == classes.end()) {
                ClassInfo ci;
                ci.tile = kv.second.tile;
                ci.ndims = kv.second.ndims;
                ci.fixed = fixed;
                ci.offset = {kv.second.offset[0], kv.second.offset[1], kv.second.offset[2]};
                classes[rep] = ci;
            } else if (fixed) {
                it->second.fixed = true;
                it->second.offset = {kv.second.offset[0], kv.second.offset[1], kv.second.offset[2]};
            }
        }
    }

    // ---- 4. edges (:619-834) ----
    std::map<int, ClassInfo> classes;
    std::vector<ShiftEdge> edges;
    std::map<int, std::vector<AdjEdge>> adj;

    int64_t volume(const DecompMeta& m, int nd) const {
        int64_t w = 1;
        for (int d = 0; d < nd; ++d)
            w *= (int64_t)m.shape[d];
        return w;
    }

    void read_edge(int out_name, int nd, const cnh_ast_node& leaf, const cnh_region* region) {
        if (leaf.result_name == out_name)
            return;
        DecompMeta* s = find(leaf.result_name);
        if (!s || s->ndims != nd)
            return;
        int cs = uf_find(leaf.result_name), co = uf_find(out_name);
        if (cs == co)
            return;
        edges.push_back({cs, co, region_start(region, nd), region_step(region, nd), volume(*s, nd)});
    }

    void read_edges_below(const DagNode& dn, int idx, int out_name, int nd, const cnh_region* carried) {
        const cnh_ast_node& n = dn.nodes[idx];
        if (skipped(n))
            return;
        if (is_leaf(dn, n)) {
            read_edge(out_name, nd, n, carried);
            return;
        }
        for (int j = 0; j < n.n_operands; ++j) {
            const cnh_ast_node& child = dn.nodes[n.operands[j]];
            if (skipped(child))
                continue;
            const cnh_region* r = operand_region(n, j);
            if (is_leaf(dn, child))
                read_edge(out_name, nd, child, r ? r : carried);
            else
                read_edges_below(dn, n.operands[j], out_name, nd, r);
        }
    }

    void assign_edges_below(const DagNode& dn, int idx, int target, int nd, const I3& start) {
        const cnh_ast_node& n = dn.nodes[idx];
        if (skipped(n))
            return;
        if (is_leaf(dn, n)) {
            if (n.result_name == target)
                return;
            DecompMeta* s = find(n.result_name);
            if (!s || s->ndims != nd)
                return;
            int cs = uf_find(n.result_name), ct = uf_find(target);
            if (cs == ct)
                return;
            edges.push_back({ct, cs, start, {1, 1, 1}, volume(*s, nd)});
            return;
        }
        for (int j = 0; j < n.n_operands; ++j)
            assign_edges_below(dn, n.operands[j], target, nd, start);
    }

    void build_edges() {
        for (const DagNode& dn : dag)
            for (int r : dn.roots) {
                const cnh_ast_node& root = dn.nodes[r];
                if (root.opcode == CNH_OP_SET_REGION) {
                    const cnh_region* reg = node_region(root);
                    if (root.n_operands < 2 || !reg)
                        continue;
                    int target = dn.nodes[root.operands[0]].result_name;
                    DecompMeta* tm = find(target);
                    if (!tm)
                        continue;
                    int nd = tm->ndims;
                    I3 start = region_start(reg, nd);
                    for (int j = 1; j < root.n_operands; ++j)
                        assign_edges_below(dn, root.operands[j], target, nd, start);
                    // value of another rank: which of its dimensions meets which of the target's
                    for (int j = 1; j < root.n_operands; ++j) {
                        const cnh_ast_node& src = dn.nodes[root.operands[j]];
                        if (!is_leaf(dn, src) || src.result_name == target)
                            continue;
                        DecompMeta* sm = find(src.result_name);
                        if (!sm || sm->ndims == nd)
                            continue;
                        int nds = sm->ndims;
                        I3 f2t = {-1, -1, -1}, t2f = {-1, -1, -1};
                        if (nd < nds) {
                            int td = 0;
                            for (int sd = 0; sd < nds && td < nd; ++sd)
                                if (sm->shape[sd] > 1) {
                                    f2t[td] = sd;
                                    t2f[sd] = td;
                                    ++td;
                                }
                            if (td != nd)
                                continue;
                        } else {
                            I3 stop = region_stop(reg, nd, tm->shape);
                            int sd = 0;
                            for (int td = 0; td < nd && sd < nds; ++td)
                                if (stop[td] - start[td] > 1) {
                                    f2t[td] = sd;
                                    t2f[sd] = td;
                                    ++sd;
                                }
                            if (sd != nds)
                                continue;
                        }
                        int ct = uf_find(target), cs = uf_find(src.result_name);
                        if (ct == cs)
                            continue;
                        const DecompMeta& lo = nd <= nds ? *tm : *sm;
                        edges.push_back({ct, cs, start, {1, 1, 1}, volume(lo, std::min(nd, nds)), f2t,
                                         t2f});
                    }
                } else if (elementwise_or_copy(root.opcode)) {
                    DecompMeta* out = find(root.result_name);
                    if (!out)
                        continue;
                    int nd = out->ndims;
                    for (int j = 0; j < root.n_operands; ++j) {
                        const cnh_ast_node& operand = dn.nodes[root.operands[j]];
                        if (skipped(operand))
                            continue;
                        const cnh_region* r = operand_region(root, j);
                        if (is_leaf(dn, operand))
                            read_edge(root.result_name, nd, operand, r);
                        else
                            read_edges_below(dn, root.operands[j], root.result_name, nd, r);
                    }
                }
            }
        for (const ShiftEdge& e : edges) {
            if (e.from == e.to)
                continue;
            adj[e.from].push_back({e.to, e.shift, e.stride, e.from_to_to, e.weight, true});
            adj[e.to].push_back({e.from, e.shift, e.stride, e.to_to_from, e.weight, false});
        }
    }

    // ---- 5. trees, candidates, dynamic programme (:836-1499) ----
    std::map<int, int> comp_of;             // class -> component
    std::map<int, int> comp_root;           // component -> class the tree hangs from
    std::set<int> cyclic;                   // components with a cycle
    std::map<int, std::vector<int>> children;
    std::map<int, std::array<std::vector<int>, 3>> cands;
    std::map<int, std::array<std::vector<int64_t>, 3>> cost;
    std::map<int, I3> phase, absolute;

    static void add_cand(std::vector<int>& v, int o) {
        auto it = std::lower_bound(v.begin(), v.end(), o);
        if (it == v.end() || *it != o)
            v.insert(it, o);
    }

    static int desired(int o_from, int shift, int stride, int tile_to) {
        int step = stride > 1 ? stride : 1;
        return pmod((o_from + shift) / step, tile_to);
    }

    // Phases of `from` (mod tile_from) that `desired` maps onto o_target.
    static std::vector<int> reverse_desired(int o_target, int shift, int stride, int tile_from,
                                            int tile_to) {
        int step = stride > 1 ? stride : 1;
        std::vector<int> out;
        int base = o_target * step - shift;
        int period = std::max(1, tile_to * step);
        int periods = (tile_from + period - 1) / period;
        for (int k = 0; k <= periods; ++k)
            for (int delta = 0; delta < step; ++delta) {
                int c = pmod(base + delta + k * period, tile_from);
                if (desired(c, shift, stride, tile_to) == o_target)
                    add_cand(out, c);
            }
        return out;
    }

    int tile_of(int cls) {
        int t = classes[cls].tile;
        return t > 0 ? t : 1;
    }

    void build_trees() {
        std::set<int> all;
        for (auto& kv : meta)
            all.insert(uf_find(kv.first));
        int ncomp = 0;
        std::map<int, int> parent;
        for (int cls : all) {
            if (comp_of.count(cls))
                continue;
            int cid = ncomp++;
            comp_root[cid] = cls;
            std::queue<int> bfs;
            bfs.push(cls);
            comp_of[cls] = cid;
            parent[cls] = -1;
            while (!bfs.empty()) {
                int v = bfs.front();
                bfs.pop();
                std::set<int> seen;
                for (const AdjEdge& e : adj[v]) {
                    if (!seen.insert(e.neighbor).second)
                        continue;
                    if (!comp_of.count(e.neighbor)) {
                        comp_of[e.neighbor] = cid;
                        parent[e.neighbor] = v;
                        bfs.push(e.neighbor);
                    } else if (e.neighbor != parent[v]) {
                        cyclic.insert(cid);
                    }
                }
                auto ci = classes.find(v);
                if (ci != classes.end() && ci->second.fixed)
                    comp_root[cid] = v;
            }
        }
        for (auto& kv : comp_root) {
            std::queue<int> bfs;
            std::set<int> visited;
            bfs.push(kv.second);
            visited.insert(kv.second);
            while (!bfs.empty()) {
                int v = bfs.front();
                bfs.pop();
                for (const AdjEdge& e : adj[v])
                    if (!visited.count(e.neighbor) && comp_of[e.neighbor] == kv.first) {
                        visited.insert(e.neighbor);
                        children[v].push_back(e.neighbor);
                        bfs.push(e.neighbor);
                    }
            }
        }
    }

    std::vector<int> roots_of_trees() {
        std::vector<int> r;
        for (auto& kv : comp_root)
            if (!cyclic.count(kv.first))
                r.push_back(kv.second);
        return r;
    }

    // Cost of one (parent phase ov, child phase oc) pair along dimension d of the parent.
    int64_t pair_cost(const std::vector<const AdjEdge*>& es, int d, int only_dc, int ov, int oc,
                      int tile_v, int tile_c, int64_t base) {
        int64_t c = base;
        for (const AdjEdge* e : es) {
            int dc = e->neighbor_dim[d];
            if (dc < 0 || (only_dc >= 0 && dc != only_dc))
                continue;
            int d_from = e->forward ? d : dc;
            int o_from = e->forward ? ov : oc, o_to = e->forward ? oc : ov;
            int tile_to = e->forward ? tile_c : tile_v;
            c += e->weight * circ_dist(desired(o_from, e->shift[d_from], e->stride[d_from], tile_to),
                                       o_to, tile_to);
            if (c >= kInf)
                break;
        }
        return c;
    }

    void solve_trees() {
        std::vector<int> post;
        for (int root : roots_of_trees()) {
            std::vector<std::pair<int, bool>> stk{{root, false}};
            while (!stk.empty()) {
                auto [v, done] = stk.back();
                stk.pop_back();
                if (done) {
                    post.push_back(v);
                    continue;
                }
                stk.push_back({v, true});
                for (int c : children[v])
                    stk.push_back({c, false});
            }
        }
        // candidates, leaves towards the root (:966-1016)
        for (int v : post) {
            const ClassInfo& ci = classes[v];
            int nd = ci.ndims, tile_v = tile_of(v);
            auto& cv = cands[v];
            if (ci.fixed)
                for (int d = 0; d < nd; ++d)
                    add_cand(cv[d], pmod(ci.offset[d], tile_v));
            for (int c : children[v]) {
                int tile_c = tile_of(c);
                for (const AdjEdge& e : adj[v]) {
                    if (e.neighbor != c)
                        continue;
                    for (int d = 0; d < nd; ++d) {
                        int dc = e.neighbor_dim[d];
                        if (dc < 0)
                            continue;
                        int d_from = e.forward ? d : dc;
                        for (int oc : cands[c][dc]) {
                            if (e.forward) {
                                for (int rv : reverse_desired(oc, e.shift[d_from], e.stride[d_from],
                                                              tile_v, tile_c))
                                    add_cand(cv[d], rv);
                            } else {
                                add_cand(cv[d],
                                         desired(oc, e.shift[d_from], e.stride[d_from], tile_v));
                            }
                        }
                    }
                }
            }
            for (int d = 0; d < nd; ++d)
                if (cv[d].empty())
                    add_cand(cv[d], 0);
        }
        // candidates, root towards the leaves (:1018-1068)
        {
            std::queue<int> work;
            for (int root : roots_of_trees())
                work.push(root);
            while (!work.empty()) {
                int v = work.front();
                work.pop();
                int nd = classes[v].ndims, tile_v = tile_of(v);
                for (int c : children[v]) {
                    int tile_c = tile_of(c);
                    for (const AdjEdge& e : adj[v]) {
                        if (e.neighbor != c)
                            continue;
                        for (int d = 0; d < nd; ++d) {
                            int dc = e.neighbor_dim[d];
                            if (dc < 0)
                                continue;
                            int d_from = e.forward ? d : dc;
                            std::vector<int> from_parent = cands[v][d];
                            for (int ov : from_parent) {
                                if (e.forward) {
                                    add_cand(cands[c][dc], desired(ov, e.shift[d_from],
                                                                   e.stride[d_from], tile_c));
                                } else {
                                    for (int rc : reverse_desired(ov, e.shift[d_from],
                                                                  e.stride[d_from], tile_c, tile_v))
                                        add_cand(cands[c][dc], rc);
                                }
                            }
                        }
                    }
                    work.push(c);
                }
            }
        }
        // cost of each candidate with the best choice below it (:1070-1166)
        for (int v : post) {
            const ClassInfo& ci = classes[v];
            int nd = ci.ndims, tile_v = tile_of(v);
            auto& cv = cands[v];
            auto& dv = cost[v];
            for (int d = 0; d < 3; ++d) {
                dv[d].assign(cv[d].size(), 0);
                if (d < nd && ci.fixed) {
                    int fixed = pmod(ci.offset[d], tile_v);
                    for (size_t i = 0; i < cv[d].size(); ++i)
                        dv[d][i] = cv[d][i] == fixed ? 0 : kInf;
                }
            }
            for (int c : children[v]) {
                int tile_c = tile_of(c);
                std::vector<const AdjEdge*> es;
                for (const AdjEdge& e : adj[v])
                    if (e.neighbor == c)
                        es.push_back(&e);
                auto& cc = cands[c];
                auto& dc_cost = cost[c];
                for (int d = 0; d < nd; ++d) {
                    int dc = d;
                    for (const AdjEdge* e : es)
                        if (e->neighbor_dim[d] != d) {
                            dc = e->neighbor_dim[d];
                            break;
                        }
                    if (dc < 0)
                        continue;
                    for (size_t iv = 0; iv < cv[d].size(); ++iv) {
                        int64_t best = kInf;
                        for (size_t ic = 0; ic < cc[dc].size(); ++ic) {
                            if (dc_cost[dc][ic] >= kInf)
                                continue;
                            best = std::min(best, pair_cost(es, d, -1, cv[d][iv], cc[dc][ic], tile_v,
                                                            tile_c, dc_cost[dc][ic]));
                        }
                        if (dv[d][iv] < kInf && best < kInf)
                            dv[d][iv] += best;
                        else
                            dv[d][iv] = kInf;
                    }
                }
            }
        }
        // phases: the root's cheapest, then every child's cheapest under its parent's (:1168-1294)
        for (int root : roots_of_trees()) {
            I3 best = {0, 0, 0};
            for (int d = 0; d < classes[root].ndims; ++d) {
                int64_t best_cost = kInf;
                for (size_t i = 0; i < cands[root][d].size(); ++i)
                    if (cost[root][d][i] < best_cost) {
                        best_cost = cost[root][d][i];
                        best[d] = cands[root][d][i];
                    }
            }
            phase[root] = best;
        }
        {
            std::queue<int> work;
            for (int root : roots_of_trees())
                work.push(root);
            while (!work.empty()) {
                int v = work.front();
                work.pop();
                int nd = classes[v].ndims, tile_v = tile_of(v);
                for (int c : children[v]) {
                    int tile_c = tile_of(c), nd_c = classes[c].ndims;
                    std::vector<const AdjEdge*> es;
                    for (const AdjEdge& e : adj[v])
                        if (e.neighbor == c)
                            es.push_back(&e);
                    I3 best = {0, 0, 0};
                    for (int dc = 0; dc < nd_c; ++dc) {
                        int d_parent = -1;
                        for (int d = 0; d < nd && d_parent < 0; ++d)
                            for (const AdjEdge* e : es)
                                if (e->neighbor_dim[d] == dc) {
                                    d_parent = d;
                                    break;
                                }
                        int64_t best_cost = kInf;
                        for (size_t ic = 0; ic < cands[c][dc].size(); ++ic) {
                            int64_t here = cost[c][dc][ic];
                            if (d_parent >= 0) {
                                if (here >= kInf)
                                    continue;
                                here = pair_cost(es, d_parent, dc, phase[v][d_parent], cands[c][dc][ic],
                                                 tile_v, tile_c, here);
                            }
                            if (here < best_cost) {
                                best_cost = here;
                                best[dc] = cands[c][dc][ic];
                            }
                        }
                    }
                    phase[c] = best;
                    work.push(c);
                }
            }
        }
        // absolute offsets (:1296-1485)
        for (int root : roots_of_trees()) {
            const ClassInfo& ci = classes[root];
            I3 a = {0, 0, 0};
            for (int d = 0; d < ci.ndims; ++d)
                a[d] = ci.fixed ? ci.offset[d] : nearest_congruent(phase[root][d], phase[root][d], tile_of(root));
            absolute[root] = a;
        }
        std::queue<int> work;
        for (int root : roots_of_trees())
            work.push(root);
        while (!work.empty()) {
            int v = work.front();
            work.pop();
            int nd_v = classes[v].ndims;
            const I3 abs_v = absolute[v];
            for (int c : children[v]) {
                const ClassInfo& cc = classes[c];
                int tile_c = tile_of(c);
                std::vector<const AdjEdge*> es;
                for (const AdjEdge& e : adj[v])
                    if (e.neighbor == c)
                        es.push_back(&e);
                I3 a = {0, 0, 0};
                for (int dc = 0; dc < cc.ndims; ++dc) {
                    if (cc.fixed) {
                        a[dc] = cc.offset[dc];
                        continue;
                    }
                    std::vector<Proposal> props;
                    for (const AdjEdge* e : es)
                        for (int d = 0; d < nd_v; ++d) {
                            if (e->neighbor_dim[d] != dc)
                                continue;
                            int value;
                            if (e->forward) {
                                int step = e->stride[d] > 1 ? e->stride[d] : 1;
                                int64_t anchor = ((int64_t)abs_v[d] + e->shift[d]) / step;
                                value = nearest_congruent(anchor, phase[c][dc], tile_c);
                            } else {
                                value = reverse_absolute(abs_v[d], e->shift[dc], e->stride[dc],
                                                         phase[c][dc], tile_c);
                            }
                            props.push_back({value, e->weight});
                        }
                    a[dc] = choose_absolute(props, phase[c][dc], tile_c);
                }
                absolute[c] = a;
                work.push(c);
            }
        }
        for (auto& kv : meta) {
            if (kv.second.final || matmul_arrays.count(kv.first))
                continue;
            int rep = uf_find(kv.first);
            auto comp = comp_of.find(rep);
            if (comp != comp_of.end() && cyclic.count(comp->second))
                continue;
            auto it = absolute.find(rep);
            if (it != absolute.end())
                for (int d = 0; d < 3; ++d)
                    kv.second.offset[d] = it->second[d];
        }
    }

    // The value congruent to phase (mod tile) nearest to anchor; the lower one on a tie.
    static int nearest_congruent(int64_t anchor, int ph, int tile) {
        if (tile <= 0)
            return (int)anchor;
        int target = pmod(ph, tile);
        int64_t lower = target;
        if (anchor >= target)
            lower += ((anchor - target) / tile) * (int64_t)tile;
        else
            lower -= ((target - anchor + tile - 1) / tile) * (int64_t)tile;
        int64_t upper = lower + tile;
        return (int)(dist64(upper, anchor) < dist64(lower, anchor) ? upper : lower);
    }

    // Offset of `from` with the given phase whose image (offset + shift) / stride is target_abs.
    static int reverse_absolute(int64_t target_abs, int shift, int stride, int phase_from,
                                int tile_from) {
        int step = stride > 1 ? stride : 1;
        int64_t low = target_abs * step - shift, centre2 = 2 * low + (step - 1);
        bool found = false;
        int64_t best = low, best_score = 0;
        int ph = pmod(phase_from, tile_from);
        for (int delta = 0; delta < step; ++delta) {
            int64_t cand = low + delta;
            if (pmod64(cand, tile_from) != ph || (cand + shift) / step != target_abs)
                continue;
            int64_t score = dist64(2 * cand, centre2);
            if (!found || score < best_score || (score == best_score && cand < best)) {
                found = true;
                best = cand;
                best_score = score;
            }
        }
        return found ? (int)best : nearest_congruent(low, phase_from, tile_from);
    }

    // Weighted median over the proposed values and the bare phase; the smaller one on a tie.
    static int choose_absolute(const std::vector<Proposal>& props, int ph, int tile) {
        std::vector<int> c;
        c.push_back(nearest_congruent(ph, ph, tile));
        for (const Proposal& p : props)
            add_cand(c, p.value);
        int best = c.front();
        int64_t best_cost = std::numeric_limits<int64_t>::max();
        for (int cand : c) {
            int64_t k = 0;
            for (const Proposal& p : props)
                k += p.weight * dist64(cand, p.value);
            if (k < best_cost || (k == best_cost && cand < best)) {
                best_cost = k;
                best = cand;
            }
        }
        return best;
    }

    // ---- 6. components with a cycle (:1501-1703) ----
    struct Wish {
        I3 ph, anchor;
        int64_t weight;
    };
    std::map<int, std::vector<Wish>> wishes;

    bool in_cycle(int name) {
        auto it = comp_of.find(uf_find(name));
        return it != comp_of.end() && cyclic.count(it->second);
    }

    void producer_wishes(const DagNode& dn, int idx, int out_name, int nd, int out_tile) {
        const cnh_ast_node& n = dn.nodes[idx];
        if (skipped(n))
            return;
        if (is_leaf(dn, n)) {
            if (n.result_name == out_name || out_tile <= 0)
                return;
            DecompMeta* s = find(n.result_name);
            if (!s || s->ndims != nd)
                return;
            Wish w{{0, 0, 0}, {0, 0, 0}, volume(*s, nd)};
            for (int d = 0; d < nd; ++d) {
                w.anchor[d] = s->offset[d];
                w.ph[d] = pmod(s->offset[d], out_tile);
            }
            wishes[out_name].push_back(w);
            return;
        }
        for (int j = 0; j < n.n_operands; ++j) {
            const cnh_ast_node& child = dn.nodes[n.operands[j]];
            if (skipped(child))
                continue;
            const cnh_region* r = operand_region(n, j);
            if (is_leaf(dn, child) && r) {
                if (child.result_name == out_name || out_tile <= 0)
                    continue;
                DecompMeta* s = find(child.result_name);
                if (!s || s->ndims != nd)
                    continue;
                I3 st = region_start(r, nd), sp = region_step(r, nd);
                Wish w{{0, 0, 0}, {0, 0, 0}, volume(*s, nd)};
                for (int d = 0; d < nd; ++d) {
                    int step = sp[d] > 1 ? sp[d] : 1;
                    int raw = s->offset[d] + st[d];
                    w.anchor[d] = step > 1 ? raw / step : raw;
                    w.ph[d] = pmod(step > 1 ? raw / step : raw, out_tile);
                }
                wishes[out_name].push_back(w);
            } else {
                producer_wishes(dn, n.operands[j], out_name, nd, out_tile);
            }
        }
    }

    void consumer_wishes(const DagNode& dn, int idx, int target, int nd, const DecompMeta& tm,
                         const I3& start) {
        const cnh_ast_node& n = dn.nodes[idx];
        if (skipped(n))
            return;
        if (is_leaf(dn, n)) {
            if (n.result_name == target)
                return;
            DecompMeta* s = find(n.result_name);
            if (!s || s->ndims != nd || s->tile <= 0)
                return;
            Wish w{{0, 0, 0}, {0, 0, 0}, volume(*s, nd)};
            for (int d = 0; d < nd; ++d) {
                w.anchor[d] = tm.offset[d] + start[d];
                w.ph[d] = pmod(tm.offset[d] + start[d], s->tile);
            }
            wishes[n.result_name].push_back(w);
            return;
        }
        for (int j = 0; j < n.n_operands; ++j)
            consumer_wishes(dn, n.operands[j], target, nd, tm, start);
    }

    void solve_cycles() {
        if (cyclic.empty())
            return;
        for (const DagNode& dn : dag)
            for (int r : dn.roots) {
                const cnh_ast_node& root = dn.nodes[r];
                if (root.opcode == CNH_OP_SET_REGION) {
                    const cnh_region* reg = node_region(root);
                    if (root.n_operands < 2 || !reg)
                        continue;
                    int target = dn.nodes[root.operands[0]].result_name;
                    DecompMeta* tm = find(target);
                    if (!tm)
                        continue;
                    I3 start = region_start(reg, tm->ndims);
                    for (int j = 1; j < root.n_operands; ++j)
                        consumer_wishes(dn, root.operands[j], target, tm->ndims, *tm, start);
                } else if (elementwise_or_copy(root.opcode)) {
                    if (!in_cycle(root.result_name))
                        continue;
                    DecompMeta* out = find(root.result_name);
                    if (!out)
                        continue;
                    for (int j = 0; j < root.n_operands; ++j)
                        if (!skipped(dn.nodes[root.operands[j]]))
                            producer_wishes(dn, root.operands[j], root.result_name, out->ndims,
                                            out->tile);
                }
            }
        for (auto& kv : wishes) {
            DecompMeta* m = find(kv.first);
            if (kv.second.empty() || !in_cycle(kv.first) || !m || m->final ||
                matmul_arrays.count(kv.first) || m->tile <= 0)
                continue;
            int tile = m->tile;
            for (int d = 0; d < m->ndims; ++d) {
                std::vector<int> c{0};
                for (const Wish& w : kv.second)
                    add_cand(c, pmod(w.ph[d], tile));
                int64_t best_cost = std::numeric_limits<int64_t>::max();
                int best = 0;
                for (int o : c) {
                    int64_t k = 0;
                    for (const Wish& w : kv.second)
                        k += w.weight * circ_dist(o, w.ph[d], tile);
                    if (k < best_cost) {
                        best_cost = k;
                        best = o;
                    }
                }
                std::vector<Proposal> props;
                for (const Wish& w : kv.second)
                    props.push_back({nearest_congruent(w.anchor[d], best, tile), w.weight});
                m->offset[d] = choose_absolute(props, best, tile);
            }
        }
    }

    void run() {
        for (auto& kv : meta) {
            DecompMeta& m = kv.second;
            if (m.tile == 0)
                m.tile = min_edge(m.ndims);
            if (!m.final) {
                m.tile = std::max(next_pow2(m.tile), min_edge(m.ndims));
                clamp(m);
                m.offset[0] = m.offset[1] = m.offset[2] = 0;
            }
        }
        if (!dag.empty()) {
            propagate_tiles();
            build_classes();
            build_edges();
            build_trees();
            solve_trees();
            solve_cycles();
            for (int name : matmul_arrays)
                if (DecompMeta* m = find(name))
                    if (!m->final)
                        m->offset[0] = m->offset[1] = m->offset[2] = 0;
        }
        for (auto& kv : meta)
            kv.second.final = true;
    }
};

} // namespace

void solve_decompositions(std::map<int, DecompMeta>& meta, const std::vector<DagNode>& dag, int odf,
                          int num_pes, const int min_tile[4]) {
    Solver s{meta, dag, odf, num_pes, min_tile};
    s.run();
}

} // namespace cnh
