// cn_oracle.cpp — CPU restatement of charmnumeric's per-partition array execution path.
// TEST INFRASTRUCTURE ONLY: used by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
// leg as the checker / the timed CPU baseline. The product never links or calls it.
// Build: g++ -O3 -ffp-contract=off -fno-fast-math (see oracle/Makefile).
// Every exported function is pinned by tests/test_oracle_*.py against upstream's own vectors, NumPy
// in the same operand order, closed forms, exactly rounded sums or brute force. Left open at bit
// level (only the 1e-12 bar applies): the summation order inside upstream's Eigen dot / GEMV / GEMM
// and its reduction tree; integer x/0 and MIN/-1 (fixed values here, undefined upstream).
#include "cn_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <thread>
#include <vector>

namespace {

inline int pmod(int v, int m) {
    int r = v % m;
    return r < 0 ? r + m : r;
}

inline int gcd_i(int a, int b) {
    a = std::abs(a);
    b = std::abs(b);
    while (b) {
        int t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Iterative extended Euclid: returns g and x with a*x == g (mod b).
long long egcd_x(long long a, long long b, long long& x_out) {
    long long x0 = 1, x1 = 0;
    while (b != 0) {
        long long q = a / b;
        long long t = a - q * b;
        a = b;
        b = t;
        t = x0 - q * x1;
        x0 = x1;
        x1 = t;
    }
    x_out = x0;
    return a;
}

long long mod_inverse(long long v, long long m) {
    long long x = 0;
    egcd_x(v, m, x);
    x %= m;
    if (x < 0)
        x += m;
    return x;
}

inline bool same_region(const orc_region& a, const orc_region& b) {
    for (int d = 0; d < a.ndims; ++d)
        if (a.start[d] != b.start[d] || a.stop[d] != b.stop[d] || a.step[d] != b.step[d])
            return false;
    return a.ndims == b.ndims;
}

inline int rsize(const orc_region& r, int d) {
    return (r.stop[d] - r.start[d] + r.step[d] - 1) / r.step[d];
}

} // namespace

extern "C" {

// Smallest point >= lo (and < hi) lying on both lattices start_a + k*step_a and
// start_b + k*step_b; the common lattice step is lcm(step_a, step_b).
// Follows src/array_region.hpp:75-108 (solution of the linear congruence by modular inverse).
int orc_first_aligned_point(int start_a, int step_a, int start_b, int step_b, int lo, int hi,
                            int* aligned, int* aligned_step) {
    int g = gcd_i(step_a, step_b);
    if (pmod(start_a - start_b, g) != 0)
        return 0;
    long long ra = step_a / g, rb = step_b / g;
    long long diff = (long long)(start_b - start_a) / g;
    long long t0 = 0;
    if (rb != 1) {
        long long am = ((ra % rb) + rb) % rb;
        long long dm = ((diff % rb) + rb) % rb;
        t0 = (dm * mod_inverse(am, rb)) % rb;
    }
    long long first = (long long)start_a + (long long)step_a * t0;
    long long period = ((long long)step_a / g) * step_b;
    if (first < lo)
        first += ((lo - first + period - 1) / period) * period;
    if (first >= hi)
        return 0;
    *aligned = (int)first;
    *aligned_step = (int)period;
    return 1;
}

int orc_region_size_dim(const orc_region* r, int d) { return rsize(*r, d); }

int orc_region_size(const orc_region* r) {
    int total = 1;
    for (int d = 0; d < r->ndims; ++d)
        total *= rsize(*r, d);
    return total;
}

int orc_region_overlaps(const orc_region* a, const orc_region* b) {
    if (a->is_global || b->is_global)
        return 1;
    if (same_region(*a, *b))
        return 1;
    for (int d = 0; d < a->ndims; ++d) {
        int lo = std::max(a->start[d], b->start[d]);
        int hi = std::min(a->stop[d], b->stop[d]);
        if (lo >= hi)
            return 0;
        int al, as;
        if (!orc_first_aligned_point(a->start[d], a->step[d], b->start[d], b->step[d], lo, hi, &al,
                                     &as))
            return 0;
    }
    return 1;
}

int orc_region_covers(const orc_region* a, const orc_region* b) {
    if (a->is_global)
        return 1;
    if (b->is_global)
        return 0;
    if (same_region(*a, *b))
        return 1;
    for (int d = 0; d < a->ndims; ++d) {
        if (b->start[d] < a->start[d] || b->stop[d] > a->stop[d])
            return 0;
        if (a->step[d] == 1)
            continue;
        if (pmod(b->start[d] - a->start[d], a->step[d]) != 0)
            return 0;
        if (rsize(*b, d) <= 1)
            continue;
        if (b->step[d] % a->step[d] != 0)
            return 0;
    }
    return 1;
}

int orc_region_intersect(const orc_region* a, const orc_region* b, orc_region* out) {
    if (a->is_global) {
        *out = *b;
        return 1;
    }
    if (b->is_global) {
        *out = *a;
        return 1;
    }
    if (same_region(*a, *b)) {
        *out = *a;
        return 1;
    }
    orc_region r;
    std::memset(&r, 0, sizeof r);
    r.ndims = a->ndims;
    for (int d = 0; d < a->ndims; ++d) {
        int lo = std::max(a->start[d], b->start[d]);
        int hi = std::min(a->stop[d], b->stop[d]);
        if (lo >= hi)
            return 0;
        int al, as;
        if (!orc_first_aligned_point(a->start[d], a->step[d], b->start[d], b->step[d], lo, hi, &al,
                                     &as))
            return 0;
        r.start[d] = al;
        r.stop[d] = hi;
        r.step[d] = as;
    }
    *out = r;
    return 1;
}

// r1 minus r2 as up to 2N slabs, peeling one dimension at a time; for a stepped remainder the
// covered stop is snapped back onto the remainder's lattice (src/array_region.hpp:471-519).
int orc_region_subtract(const orc_region* r1, const orc_region* r2, orc_region* out) {
    orc_region ov;
    if (!orc_region_intersect(r1, r2, &ov)) {
        out[0] = *r1;
        return 1;
    }
    int n = 0;
    orc_region rem = *r1;
    for (int d = 0; d < r1->ndims; ++d) {
        int covered_stop = ov.stop[d];
        if (rem.step[d] > 1)
            covered_stop = ov.start[d] + rsize(ov, d) * rem.step[d];
        if (rem.start[d] < ov.start[d]) {
            out[n] = rem;
            out[n].stop[d] = ov.start[d];
            ++n;
        }
        if (covered_stop < rem.stop[d]) {
            out[n] = rem;
            out[n].start[d] = covered_stop;
            ++n;
        }
        rem.start[d] = ov.start[d];
        rem.stop[d] = covered_stop;
    }
    return n;
}

// i-th element of parent1 <-> i-th element of parent2; extent carried by element count
// (src/array_region.hpp:524-545).
void orc_region_map(const orc_region* r1, const orc_region* p1, const orc_region* p2,
                    orc_region* out) {
    orc_region r;
    std::memset(&r, 0, sizeof r);
    r.ndims = r1->ndims;
    for (int d = 0; d < r1->ndims; ++d) {
        int lo = (r1->start[d] - p1->start[d]) / p1->step[d];
        int ls = r1->step[d] / p1->step[d];
        int cnt = rsize(*r1, d);
        r.start[d] = p2->start[d] + lo * p2->step[d];
        r.step[d] = ls * p2->step[d];
        r.stop[d] = r.start[d] + cnt * r.step[d];
    }
    *out = r;
}

int orc_decomp_num_chares(const orc_decomp* dc, int d) {
    int gstart = dc->offset[d];
    int gstop = dc->offset[d] + dc->global_shape[d];
    return (gstop + dc->tile - 1) / dc->tile - gstart / dc->tile;
}

void orc_decomp_chare_region_global(const orc_decomp* dc, const int32_t* ci, orc_region* out) {
    std::memset(out, 0, sizeof *out);
    out->ndims = dc->ndims;
    for (int d = 0; d < dc->ndims; ++d) {
        out->start[d] = std::max(ci[d] * dc->tile, dc->offset[d]);
        out->stop[d] = std::min((ci[d] + 1) * dc->tile, dc->offset[d] + dc->global_shape[d]);
        out->step[d] = 1;
    }
}

int orc_decompose(const orc_region* region, const orc_decomp* dc, int cap, int32_t* chare_idx,
                  orc_region* out) {
    int nd = region->ndims;
    int c0[ORC_MAX_ND], c1[ORC_MAX_ND], ci[ORC_MAX_ND];
    for (int d = 0; d < nd; ++d) {
        c0[d] = region->start[d] / dc->tile;
        c1[d] = (region->stop[d] + dc->tile - 1) / dc->tile;
        ci[d] = c0[d];
        if (c1[d] <= c0[d])
            return 0;
    }
    int n = 0;
    for (;;) {
        orc_region creg, sub;
        orc_decomp_chare_region_global(dc, ci, &creg);
        bool nonempty = true;
        for (int d = 0; d < nd; ++d)
            if (creg.start[d] >= creg.stop[d])
                nonempty = false;
        if (nonempty && orc_region_intersect(region, &creg, &sub)) {
            if (n >= cap)
                return -1;
            for (int d = 0; d < nd; ++d)
                chare_idx[n * nd + d] = ci[d];
            out[n] = sub;
            ++n;
        }
        int d = nd - 1;
        while (d >= 0) {
            if (++ci[d] < c1[d])
                break;
            ci[d] = c0[d];
            --d;
        }
        if (d < 0)
            break;
    }
    return n;
}

int orc_local_inputs(const orc_region* r_out, int n_inputs, const orc_region* inputs,
                     const int32_t* nd_idx, const orc_decomp* out_decomp,
                     const orc_decomp* in_decomps, orc_region* my_inputs, int* expected_msgs) {
    *expected_msgs = 0;
    orc_region chare_out, myout;
    orc_decomp_chare_region_global(out_decomp, nd_idx, &chare_out);
    if (!orc_region_intersect(r_out, &chare_out, &myout))
        return 0;
    std::vector<int32_t> idxbuf(4096 * ORC_MAX_ND);
    std::vector<orc_region> regbuf(4096);
    for (int k = 0; k < n_inputs; ++k) {
        orc_region chare_in, myin;
        orc_decomp_chare_region_global(&in_decomps[k], nd_idx, &chare_in);
        orc_region_map(&myout, r_out, &inputs[k], &myin);
        my_inputs[k] = myin;
        orc_region frags[2 * ORC_MAX_ND + 1];
        int nf = orc_region_subtract(&myin, &chare_in, frags);
        for (int f = 0; f < nf; ++f) {
            int c = orc_decompose(&frags[f], &in_decomps[k], 4096, idxbuf.data(), regbuf.data());
            if (c < 0)
                return -1;
            *expected_msgs += c;
        }
    }
    return n_inputs;
}

int orc_send_remote_inputs(const orc_region* r_out, int n_inputs, const orc_region* inputs,
                           const int32_t* nd_idx, const orc_decomp* out_decomp,
                           const orc_decomp* in_decomps, int cap, int32_t* targets,
                           orc_region* regions, int32_t* input_index) {
    int nd = r_out->ndims;
    orc_region chare_out;
    orc_decomp_chare_region_global(out_decomp, nd_idx, &chare_out);
    std::vector<int32_t> idxbuf(4096 * ORC_MAX_ND);
    std::vector<orc_region> regbuf(4096);
    int n = 0;
    for (int k = 0; k < n_inputs; ++k) {
        orc_region chare_in, myin, myout;
        orc_decomp_chare_region_global(&in_decomps[k], nd_idx, &chare_in);
        if (!orc_region_intersect(&inputs[k], &chare_in, &myin))
            continue;
        orc_region_map(&myin, &inputs[k], r_out, &myout);
        orc_region frags[2 * ORC_MAX_ND + 1];
        int nf = orc_region_subtract(&myout, &chare_out, frags);
        for (int f = 0; f < nf; ++f) {
            int c = orc_decompose(&frags[f], out_decomp, 4096, idxbuf.data(), regbuf.data());
            if (c < 0)
                return -1;
            for (int j = 0; j < c; ++j) {
                if (n >= cap)
                    return -1;
                for (int d = 0; d < nd; ++d)
                    targets[n * nd + d] = idxbuf[j * nd + d];
                orc_region_map(&regbuf[j], r_out, &inputs[k], &regions[n]);
                input_index[n] = k;
                ++n;
            }
        }
    }
    return n;
}

// Common refinement of K fragment lists in logical index space (src/array_region.hpp:675-818).
int orc_align_fragments(int nd, int K, const int32_t* frag_begin, const orc_fragment* frags,
                        const orc_region* parents, int cap, int32_t* out_frag,
                        int64_t* out_offsets, int64_t* out_sizes, int64_t* out_strides,
                        orc_region* out_cells) {
    if (K <= 0)
        return 0;
    std::vector<int> grid[ORC_MAX_ND];
    for (int k = 0; k < K; ++k)
        for (int f = frag_begin[k]; f < frag_begin[k + 1]; ++f)
            for (int d = 0; d < nd; ++d) {
                const orc_region& fr = frags[f].region;
                int gs = parents[k].start[d], gst = parents[k].step[d];
                if (fr.step[d] % gst != 0)
                    return -2;
                int lo = (fr.start[d] - gs) / gst;
                int hi = lo + rsize(fr, d) * (fr.step[d] / gst);
                grid[d].push_back(lo);
                grid[d].push_back(hi);
            }
    for (int d = 0; d < nd; ++d) {
        std::sort(grid[d].begin(), grid[d].end());
        grid[d].erase(std::unique(grid[d].begin(), grid[d].end()), grid[d].end());
    }
    struct Cell {
        int frag;
        int64_t off;
        int64_t sizes[ORC_MAX_ND], strides[ORC_MAX_ND];
        orc_region reg;
        int key[ORC_MAX_ND];
    };
    int M = -1;
    for (int k = 0; k < K; ++k) {
        std::vector<Cell> cells;
        for (int f = frag_begin[k]; f < frag_begin[k + 1]; ++f) {
            const orc_region& fr = frags[f].region;
            int gs[ORC_MAX_ND], gst[ORC_MAX_ND], ilo[ORC_MAX_ND], ihi[ORC_MAX_ND], idx[ORC_MAX_ND];
            bool explicit_strides = false;
            int64_t st[ORC_MAX_ND];
            for (int d = 0; d < nd; ++d)
                if (frags[f].src_strides[d] != 0)
                    explicit_strides = true;
            if (explicit_strides) {
                for (int d = 0; d < nd; ++d)
                    st[d] = frags[f].src_strides[d];
            } else {
                st[nd - 1] = 1;
                for (int d = nd - 2; d >= 0; --d)
                    st[d] = st[d + 1] * rsize(fr, d + 1);
            }
            for (int d = 0; d < nd; ++d) {
                gs[d] = parents[k].start[d];
                gst[d] = parents[k].step[d];
                int flo = (fr.start[d] - gs[d]) / gst[d];
                int fhi = flo + rsize(fr, d) * (fr.step[d] / gst[d]);
                ilo[d] = (int)(std::lower_bound(grid[d].begin(), grid[d].end(), flo) - grid[d].begin());
                ihi[d] = (int)(std::lower_bound(grid[d].begin(), grid[d].end(), fhi) - grid[d].begin());
                idx[d] = ilo[d];
            }
            for (;;) {
                Cell c;
                std::memset(&c, 0, sizeof c);
                c.frag = f;
                c.reg.ndims = nd;
                for (int d = 0; d < nd; ++d) {
                    c.reg.start[d] = gs[d] + grid[d][idx[d]] * gst[d];
                    c.reg.stop[d] = gs[d] + grid[d][idx[d] + 1] * gst[d];
                    c.reg.step[d] = fr.step[d];
                    int delta = c.reg.start[d] - fr.start[d];
                    c.off += (int64_t)(explicit_strides ? delta : delta / fr.step[d]) * st[d];
                    c.sizes[d] = rsize(c.reg, d);
                    c.strides[d] = explicit_strides ? st[d] * c.reg.step[d] : st[d];
                    c.key[d] = (c.reg.start[d] - gs[d]) / gst[d];
                }
                cells.push_back(c);
                int d = nd - 1;
                while (d >= 0) {
                    if (++idx[d] < ihi[d])
                        break;
                    idx[d] = ilo[d];
                    --d;
                }
                if (d < 0)
                    break;
            }
        }
        std::stable_sort(cells.begin(), cells.end(), [nd](const Cell& a, const Cell& b) {
            for (int d = 0; d < nd; ++d)
                if (a.key[d] != b.key[d])
                    return a.key[d] < b.key[d];
            return false;
        });
        if (M < 0)
            M = (int)cells.size();
        if ((int)cells.size() != M)
            return -3;
        if (M > cap)
            return -1;
        for (int m = 0; m < M; ++m) {
            out_frag[k * M + m] = cells[m].frag;
            out_offsets[k * M + m] = cells[m].off;
            for (int d = 0; d < ORC_MAX_ND; ++d) {
                out_sizes[(k * M + m) * ORC_MAX_ND + d] = cells[m].sizes[d];
                out_strides[(k * M + m) * ORC_MAX_ND + d] = cells[m].strides[d];
            }
            out_cells[k * M + m] = cells[m].reg;
        }
    }
    return M;
}

int orc_next_pow2(int v) {
    int p = 1;
    while (p < v)
        p <<= 1;
    return p;
}

// tile = max(next_pow2(min_tile), min_tile), doubled while the tile count exceeds odf*PEs
// (src/decomposition_solver.hpp:100-122; arrays arrive with tile == 0 -> ct_min_tile).
int orc_tile_rule(int nd, const int32_t* shape, int odf, int num_pes, int min_tile) {
    int tile = std::max(orc_next_pow2(min_tile), min_tile);
    long long max_tiles = (long long)std::max(1, odf) * std::max(1, num_pes);
    for (;;) {
        long long count = 1;
        for (int d = 0; d < nd; ++d)
            count *= (shape[d] + tile - 1) / tile;
        if (count <= max_tiles)
            break;
        tile *= 2;
    }
    return tile;
}

} // extern "C"

// ---------------------------------------------------------------------------------------------
// Fused group evaluation
// ---------------------------------------------------------------------------------------------
namespace {

enum ValKind { V_NONE = 0, V_LEAF, V_CONST, V_BCAST, V_SLOT };

struct Val {
    int kind = V_NONE;
    int idx = 0;     // leaf-use index, broadcast index or slot index
    double c = 0.0;  // constant
    bool scalar = false;
};

struct Stmt {
    int opcode;
    Val a, b;
    int slot;
    bool scalar; // both operands scalar -> scalar result (src/jit.cpp:329-333)
};

struct Program {
    struct LeafUse {
        int node, root, operand;
    };
    std::vector<LeafUse> leaves;
    std::vector<int> bcast_nodes;
    std::vector<int> out_roots; // root positions
    std::vector<Stmt> stmts;
    std::vector<Val> out_vals;
    int n_slots = 0;
    int err = 0;
};

std::string region_key(const orc_ast_node& root, int op_idx, const orc_ast_node& operand) {
    // leafUseKey (src/jit.cpp:265-284): name | ndims | region text
    std::string key = std::to_string(operand.result_name) + "|" + std::to_string(operand.ndims);
    if (!root.has_operand_region[op_idx])
        return key + "|null";
    const orc_region& r = root.operand_regions[op_idx];
    if (r.is_global)
        return key + "|global";
    for (int d = 0; d < operand.ndims && d < ORC_MAX_ND; ++d)
        key += "|" + std::to_string(r.start[d]) + ":" + std::to_string(r.stop[d]) + ":" +
               std::to_string(r.step[d]);
    return key;
}

Program build_program(const orc_ast* ast) {
    Program p;
    std::map<int, int> internal; // result_name -> 1
    for (int r = 0; r < ast->n_roots; ++r)
        internal[ast->nodes[ast->roots[r]].result_name] = 1;

    // collectLeaves (src/jit.cpp:223-263)
    std::map<std::string, int> leaf_by_key; // later use wins, as in leafValues[key] = arg
    std::map<int, int> bcast_by_name;
    std::map<int, Val> node_vals; // result_name -> value (nodeValues)
    for (int r = 0; r < ast->n_roots; ++r) {
        const orc_ast_node& root = ast->nodes[ast->roots[r]];
        for (int oi = 0; oi < root.n_operands; ++oi) {
            if (root.operands[oi] < 0)
                continue;
            const orc_ast_node& op = ast->nodes[root.operands[oi]];
            if (internal.count(op.result_name))
                continue;
            if (root.opcode == ORC_OP_SET_REGION && oi == 0)
                continue;
            if (op.opcode != ORC_OP_NOOP && op.opcode != ORC_OP_CREATE)
                continue;
            if (op.is_scalar) {
                Val v;
                v.kind = V_CONST;
                v.c = op.scalar;
                v.scalar = true;
                node_vals[op.result_name] = v;
            } else if (op.is_broadcast) {
                if (!bcast_by_name.count(op.result_name)) {
                    bcast_by_name[op.result_name] = (int)p.bcast_nodes.size();
                    p.bcast_nodes.push_back(root.operands[oi]);
                }
                Val v;
                v.kind = V_BCAST;
                v.idx = bcast_by_name[op.result_name];
                v.scalar = true;
                node_vals[op.result_name] = v;
            } else {
                leaf_by_key[region_key(root, oi, op)] = (int)p.leaves.size();
                p.leaves.push_back({root.operands[oi], r, oi});
            }
        }
    }
    for (int r = 0; r < ast->n_roots; ++r) {
        const orc_ast_node& root = ast->nodes[ast->roots[r]];
        if (root.opcode != ORC_OP_NOOP && root.opcode != ORC_OP_CREATE && !root.is_temp)
            p.out_roots.push_back(r);
    }

    auto lookup = [&](const orc_ast_node& root, int oi) -> Val {
        // lookupOperand (src/jit.cpp:286-297): leaf table first when a region is attached.
        const orc_ast_node& op = ast->nodes[root.operands[oi]];
        if (root.has_operand_region[oi]) {
            auto it = leaf_by_key.find(region_key(root, oi, op));
            if (it != leaf_by_key.end()) {
                Val v;
                v.kind = V_LEAF;
                v.idx = it->second;
                return v;
            }
        }
        auto it = node_vals.find(op.result_name);
        if (it != node_vals.end())
            return it->second;
        // A leaf recorded without region ("|null" key)
        auto it2 = leaf_by_key.find(region_key(root, oi, op));
        if (it2 != leaf_by_key.end()) {
            Val v;
            v.kind = V_LEAF;
            v.idx = it2->second;
            return v;
        }
        return Val();
    };

    // emitOp per root, flat order (src/jit.cpp:299-385)
    for (int r = 0; r < ast->n_roots; ++r) {
        const orc_ast_node& root = ast->nodes[ast->roots[r]];
        int opc = root.opcode;
        if (opc == ORC_OP_NOOP || opc == ORC_OP_CREATE)
            continue;
        Val result;
        if (opc == ORC_OP_SET_REGION) {
            if (root.n_operands < 2) {
                p.err = -10;
                return p;
            }
            result = lookup(root, 1);
        } else if (opc >= ORC_OP_ADD && opc <= ORC_OP_DIV) {
            Val a = lookup(root, 0), b = lookup(root, 1);
            if (a.kind == V_NONE || b.kind == V_NONE) {
                p.err = -11;
                return p;
            }
            Stmt s{opc, a, b, p.n_slots++, a.scalar && b.scalar};
            p.stmts.push_back(s);
            result.kind = V_SLOT;
            result.idx = s.slot;
            result.scalar = s.scalar;
        } else if (opc == ORC_OP_TANH || opc == ORC_OP_EXP) {
            Val a = lookup(root, 0);
            if (a.kind == V_NONE || a.scalar) { // cast<MemRefType> on a scalar: not compilable
                p.err = -12;
                return p;
            }
            Stmt s{opc, a, Val(), p.n_slots++, false};
            p.stmts.push_back(s);
            result.kind = V_SLOT;
            result.idx = s.slot;
        } else {
            p.err = -13; // "Unknown opcode in JIT emitOp"
            return p;
        }
        if (result.kind == V_NONE) {
            p.err = -14;
            return p;
        }
        node_vals[root.result_name] = result;
    }
    for (int r : p.out_roots) {
        const orc_ast_node& root = ast->nodes[ast->roots[r]];
        auto it = node_vals.find(root.result_name);
        if (it == node_vals.end()) {
            p.err = -15;
            return p;
        }
        p.out_vals.push_back(it->second);
    }
    return p;
}

template <typename T>
struct is_int_t {
    static const bool value = false;
};
template <>
struct is_int_t<int32_t> {
    static const bool value = true;
};
template <>
struct is_int_t<int64_t> {
    static const bool value = true;
};

// Scalar constant cast (src/jit.cpp:108-116): ints go through int64_t, floats through double.
template <typename T>
inline T cast_const(double c) {
    if (is_int_t<T>::value)
        return (T)(int64_t)c;
    return (T)c;
}

template <typename T>
inline T wrap_add(T a, T b) {
    return a + b;
}
template <>
inline int32_t wrap_add(int32_t a, int32_t b) {
    return (int32_t)((uint32_t)a + (uint32_t)b);
}
template <>
inline int64_t wrap_add(int64_t a, int64_t b) {
    return (int64_t)((uint64_t)a + (uint64_t)b);
}
template <typename T>
inline T wrap_sub(T a, T b) {
    return a - b;
}
template <>
inline int32_t wrap_sub(int32_t a, int32_t b) {
    return (int32_t)((uint32_t)a - (uint32_t)b);
}
template <>
inline int64_t wrap_sub(int64_t a, int64_t b) {
    return (int64_t)((uint64_t)a - (uint64_t)b);
}
template <typename T>
inline T wrap_mul(T a, T b) {
    return a * b;
}
template <>
inline int32_t wrap_mul(int32_t a, int32_t b) {
    return (int32_t)((uint32_t)a * (uint32_t)b);
}
template <>
inline int64_t wrap_mul(int64_t a, int64_t b) {
    return (int64_t)((uint64_t)a * (uint64_t)b);
}
template <typename T>
inline T trunc_div(T a, T b) {
    return a / b;
}
template <>
inline int32_t trunc_div(int32_t a, int32_t b) {
    if (b == 0)
        return 0;
    if (b == -1)
        return (int32_t)(0u - (uint32_t)a);
    return a / b;
}
template <>
inline int64_t trunc_div(int64_t a, int64_t b) {
    if (b == 0)
        return 0;
    if (b == -1)
        return (int64_t)(0ull - (uint64_t)a);
    return a / b;
}

inline float m_tanh(float x) { return tanhf(x); }
inline double m_tanh(double x) { return tanh(x); }
inline float m_exp(float x) { return expf(x); }
inline double m_exp(double x) { return exp(x); }
inline int32_t m_tanh(int32_t x) { return x; }
inline int64_t m_tanh(int64_t x) { return x; }
inline int32_t m_exp(int32_t x) { return x; }
inline int64_t m_exp(int64_t x) { return x; }

const int CHUNK = 512;

template <typename T>
int eval_group_t(const Program& p, int nd, int n_in, const orc_memref* in, int n_scalar,
                 const void* const* scalars, int n_out, const orc_memref* out) {
    if (n_in != (int)p.leaves.size() || n_scalar != (int)p.bcast_nodes.size() ||
        n_out != (int)p.out_roots.size())
        return -20;
    if (n_out == 0)
        return 0;
    if (is_int_t<T>::value)
        for (const Stmt& s : p.stmts)
            if (s.opcode == ORC_OP_TANH || s.opcode == ORC_OP_EXP)
                return -21; // no integer body registered (src/jit.cpp:445-459)

    int64_t sizes[ORC_MAX_ND] = {1, 1, 1};
    for (int d = 0; d < nd; ++d)
        sizes[d] = out[0].sizes[d];
    for (int d = 0; d < nd; ++d)
        if (sizes[d] <= 0)
            return 0;

    std::vector<T> bvals(p.bcast_nodes.size());
    for (size_t i = 0; i < bvals.size(); ++i)
        std::memcpy(&bvals[i], scalars[i], sizeof(T));

    // Scalar-valued slots are evaluated once.
    std::vector<T> slot_scalar(p.n_slots);
    std::vector<std::vector<T>> slot_buf(p.n_slots);
    for (const Stmt& s : p.stmts)
        if (!s.scalar)
            slot_buf[s.slot].resize(CHUNK);
    std::vector<std::vector<T>> leaf_buf(p.leaves.size(), std::vector<T>(CHUNK));

    auto scalar_of = [&](const Val& v) -> T {
        if (v.kind == V_CONST)
            return cast_const<T>(v.c);
        if (v.kind == V_BCAST)
            return bvals[v.idx];
        return slot_scalar[v.idx];
    };
    for (const Stmt& s : p.stmts)
        if (s.scalar) {
            T a = scalar_of(s.a), b = scalar_of(s.b);
            T r;
            switch (s.opcode) {
            case ORC_OP_ADD: r = wrap_add<T>(a, b); break;
            case ORC_OP_SUB: r = wrap_sub<T>(a, b); break;
            case ORC_OP_MUL: r = wrap_mul<T>(a, b); break;
            default: r = trunc_div<T>(a, b); break;
            }
            slot_scalar[s.slot] = r;
        }

    std::vector<T> splat_a(CHUNK), splat_b(CHUNK);
    int inner = nd - 1;
    int64_t idx[ORC_MAX_ND] = {0, 0, 0};
    for (;;) {
        for (int64_t x0 = 0; x0 < sizes[inner]; x0 += CHUNK) {
            int len = (int)std::min<int64_t>(CHUNK, sizes[inner] - x0);
            for (size_t k = 0; k < p.leaves.size(); ++k) {
                const orc_memref& m = in[k];
                int64_t base = m.offset;
                for (int d = 0; d < inner; ++d)
                    base += idx[d] * m.strides[d];
                base += x0 * m.strides[inner];
                const T* src = (const T*)m.aligned + base;
                int64_t st = m.strides[inner];
                T* dst = leaf_buf[k].data();
                for (int i = 0; i < len; ++i)
                    dst[i] = src[i * st];
            }
            auto operand = [&](const Val& v, std::vector<T>& splat) -> const T* {
                if (v.kind == V_LEAF)
                    return leaf_buf[v.idx].data();
                if (v.kind == V_SLOT && !v.scalar)
                    return slot_buf[v.idx].data();
                T c = scalar_of(v);
                for (int i = 0; i < len; ++i)
                    splat[i] = c;
                return splat.data();
            };
            for (const Stmt& s : p.stmts) {
                if (s.scalar)
                    continue;
                T* r = slot_buf[s.slot].data();
                const T* a = operand(s.a, splat_a);
                switch (s.opcode) {
                case ORC_OP_ADD: {
                    const T* b = operand(s.b, splat_b);
                    for (int i = 0; i < len; ++i)
                        r[i] = wrap_add<T>(a[i], b[i]);
                    break;
                }
                case ORC_OP_SUB: {
                    const T* b = operand(s.b, splat_b);
                    for (int i = 0; i < len; ++i)
                        r[i] = wrap_sub<T>(a[i], b[i]);
                    break;
                }
                case ORC_OP_MUL: {
                    const T* b = operand(s.b, splat_b);
                    for (int i = 0; i < len; ++i)
                        r[i] = wrap_mul<T>(a[i], b[i]);
                    break;
                }
                case ORC_OP_DIV: {
                    const T* b = operand(s.b, splat_b);
                    for (int i = 0; i < len; ++i)
                        r[i] = trunc_div<T>(a[i], b[i]);
                    break;
                }
                case ORC_OP_TANH:
                    for (int i = 0; i < len; ++i)
                        r[i] = m_tanh(a[i]);
                    break;
                default:
                    for (int i = 0; i < len; ++i)
                        r[i] = m_exp(a[i]);
                    break;
                }
            }
            for (size_t o = 0; o < p.out_vals.size(); ++o) {
                const orc_memref& m = out[o];
                int64_t base = m.offset;
                for (int d = 0; d < inner; ++d)
                    base += idx[d] * m.strides[d];
                base += x0 * m.strides[inner];
                T* dst = (T*)m.aligned + base;
                int64_t st = m.strides[inner];
                const T* src = operand(p.out_vals[o], splat_a);
                for (int i = 0; i < len; ++i)
                    dst[i * st] = src[i];
            }
        }
        int d = inner - 1;
        while (d >= 0) {
            if (++idx[d] < sizes[d])
                break;
            idx[d] = 0;
            --d;
        }
        if (d < 0)
            break;
    }
    return 0;
}

} // namespace

extern "C" {

int orc_group_signature(const orc_ast* ast, int cap, int32_t* leaf_node, int32_t* leaf_root,
                        int32_t* leaf_operand, int* n_leaves, int32_t* bcast_node, int* n_bcast,
                        int32_t* out_root, int* n_out) {
    Program p = build_program(ast);
    if (p.err)
        return p.err;
    if ((int)p.leaves.size() > cap || (int)p.bcast_nodes.size() > cap ||
        (int)p.out_roots.size() > cap)
        return -1;
    for (size_t i = 0; i < p.leaves.size(); ++i) {
        leaf_node[i] = p.leaves[i].node;
        leaf_root[i] = p.leaves[i].root;
        leaf_operand[i] = p.leaves[i].operand;
    }
    for (size_t i = 0; i < p.bcast_nodes.size(); ++i)
        bcast_node[i] = p.bcast_nodes[i];
    for (size_t i = 0; i < p.out_roots.size(); ++i)
        out_root[i] = p.out_roots[i];
    *n_leaves = (int)p.leaves.size();
    *n_bcast = (int)p.bcast_nodes.size();
    *n_out = (int)p.out_roots.size();
    return 0;
}

int orc_group_dtype(const orc_ast* ast) {
    for (int r = 0; r < ast->n_roots; ++r)
        if (ast->nodes[ast->roots[r]].dtype != ORC_F32)
            return ast->nodes[ast->roots[r]].dtype;
    return ORC_F32;
}

int orc_eval_group(const orc_ast* ast, int dtype, int nd, int n_in, const orc_memref* in,
                   int n_scalar, const void* const* scalars, int n_out, const orc_memref* out) {
    if (nd < 1 || nd > ORC_MAX_ND)
        return -2;
    Program p = build_program(ast);
    if (p.err)
        return p.err;
    switch (dtype) {
    case ORC_F32: return eval_group_t<float>(p, nd, n_in, in, n_scalar, scalars, n_out, out);
    case ORC_F64: return eval_group_t<double>(p, nd, n_in, in, n_scalar, scalars, n_out, out);
    case ORC_I32: return eval_group_t<int32_t>(p, nd, n_in, in, n_scalar, scalars, n_out, out);
    case ORC_I64: return eval_group_t<int64_t>(p, nd, n_in, in, n_scalar, scalars, n_out, out);
    }
    return -3;
}

// ---------------------------------------------------------------------------------------------
// SET_REGION fill / copy — odometer over the overlap, one element at a time, byte-wise
// (src/executor_ast_visitor.cpp:149-207 fill, :268-311 copy).
// ---------------------------------------------------------------------------------------------
int orc_scalar_to_dtype(int dtype, double s, void* out8) {
    std::memset(out8, 0, 8);
    switch (dtype) {
    case ORC_F32: {
        float v = (float)s;
        std::memcpy(out8, &v, 4);
        return 4;
    }
    case ORC_F64:
        std::memcpy(out8, &s, 8);
        return 8;
    case ORC_I32: {
        int32_t v = (int32_t)s;
        std::memcpy(out8, &v, 4);
        return 4;
    }
    case ORC_I64: {
        int64_t v = (int64_t)s;
        std::memcpy(out8, &v, 8);
        return 8;
    }
    }
    return -1;
}

int orc_fill_region(int nd, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const int64_t* counts,
                    const void* scalar) {
    if (nd < 1 || nd > ORC_MAX_ND)
        return -1;
    for (int d = 0; d < nd; ++d)
        if (counts[d] <= 0)
            return 0;
    int64_t idx[ORC_MAX_ND] = {0, 0, 0};
    for (;;) {
        int64_t off = 0;
        for (int d = 0; d < nd; ++d)
            off += (dst_start[d] + idx[d] * dst_step[d]) * dst_strides[d];
        std::memcpy((char*)dst + off * esz, scalar, esz);
        int d = nd - 1;
        while (d >= 0) {
            if (++idx[d] < counts[d])
                break;
            idx[d] = 0;
            --d;
        }
        if (d < 0)
            break;
    }
    return 0;
}

int orc_copy_region(int nd, int esz, void* dst, const int64_t* dst_strides,
                    const int64_t* dst_start, const int64_t* dst_step, const void* src,
                    const int64_t* src_strides, const int64_t* src_start, const int64_t* src_step,
                    const int64_t* counts) {
    if (nd < 1 || nd > ORC_MAX_ND)
        return -1;
    for (int d = 0; d < nd; ++d)
        if (counts[d] <= 0)
            return 0;
    int64_t idx[ORC_MAX_ND] = {0, 0, 0};
    for (;;) {
        int64_t doff = 0, soff = 0;
        for (int d = 0; d < nd; ++d) {
            doff += (dst_start[d] + idx[d] * dst_step[d]) * dst_strides[d];
            soff += (src_start[d] + idx[d] * src_step[d]) * src_strides[d];
        }
        std::memcpy((char*)dst + doff * esz, (const char*)src + soff * esz, esz);
        int d = nd - 1;
        while (d >= 0) {
            if (++idx[d] < counts[d])
                break;
            idx[d] = 0;
            --d;
        }
        if (d < 0)
            break;
    }
    return 0;
}

} // extern "C"

// ---------------------------------------------------------------------------------------------
// dot / gemv / gemm
// ---------------------------------------------------------------------------------------------
namespace {

template <typename T>
T dot_t(int64_t n, const T* a, const T* b) {
    T acc = T(0);
    for (int64_t i = 0; i < n; ++i)
        acc = wrap_add<T>(acc, wrap_mul<T>(a[i], b[i]));
    return acc;
}

template <typename T>
void gemv_rows_t(const T* mat, int64_t ld, int64_t row_off, int64_t col_off, int64_t r0,
                 int64_t r1, int64_t cols, const T* vec, T* res) {
    for (int64_t i = r0; i < r1; ++i) {
        const T* row = mat + (row_off + i) * ld + col_off;
        T acc = T(0);
        for (int64_t j = 0; j < cols; ++j)
            acc = wrap_add<T>(acc, wrap_mul<T>(row[j], vec[j]));
        res[i] = acc;
    }
}

// C[i][:] += A[i][k] * B[k][:] in k order (row-broadcast form; every C element accumulates its
// products in increasing k, like the plain triple loop).
template <typename T>
void gemm_rows_t(int64_t r0, int64_t r1, int64_t N, int64_t K, const T* A, int64_t lda,
                 const T* B, int64_t ldb, T* C, int64_t ldc) {
    for (int64_t i = r0; i < r1; ++i) {
        T* c = C + i * ldc;
        for (int64_t k = 0; k < K; ++k) {
            T a = A[i * lda + k];
            const T* b = B + k * ldb;
            for (int64_t j = 0; j < N; ++j)
                c[j] = wrap_add<T>(c[j], wrap_mul<T>(a, b[j]));
        }
    }
}

template <typename F>
void run_blocks(int64_t n, int threads, F f) {
    if (threads <= 1 || n < 2) {
        f(0, n);
        return;
    }
    std::vector<std::thread> th;
    int64_t per = (n + threads - 1) / threads;
    for (int t = 0; t < threads; ++t) {
        int64_t a = t * per, b = std::min<int64_t>(n, a + per);
        if (a >= b)
            break;
        th.emplace_back([=] { f(a, b); });
    }
    for (auto& t : th)
        t.join();
}

} // namespace

extern "C" {

int orc_dot(int dtype, int64_t n, const void* a, const void* b, void* out) {
    switch (dtype) {
    case ORC_F32: *(float*)out = dot_t<float>(n, (const float*)a, (const float*)b); return 0;
    case ORC_F64: *(double*)out = dot_t<double>(n, (const double*)a, (const double*)b); return 0;
    case ORC_I32: *(int32_t*)out = dot_t<int32_t>(n, (const int32_t*)a, (const int32_t*)b); return 0;
    case ORC_I64: *(int64_t*)out = dot_t<int64_t>(n, (const int64_t*)a, (const int64_t*)b); return 0;
    }
    return -1;
}

int orc_reduce_partials(int dtype, int n, const void* partials, void* out) {
    if (n <= 0)
        return -1;
    switch (dtype) {
    case ORC_F32: {
        float acc = ((const float*)partials)[0];
        for (int i = 1; i < n; ++i)
            acc += ((const float*)partials)[i];
        *(float*)out = acc;
        return 0;
    }
    case ORC_F64: {
        double acc = ((const double*)partials)[0];
        for (int i = 1; i < n; ++i)
            acc += ((const double*)partials)[i];
        *(double*)out = acc;
        return 0;
    }
    case ORC_I32: {
        int32_t acc = ((const int32_t*)partials)[0];
        for (int i = 1; i < n; ++i)
            acc = wrap_add<int32_t>(acc, ((const int32_t*)partials)[i]);
        *(int32_t*)out = acc;
        return 0;
    }
    case ORC_I64: {
        int64_t acc = ((const int64_t*)partials)[0];
        for (int i = 1; i < n; ++i)
            acc = wrap_add<int64_t>(acc, ((const int64_t*)partials)[i]);
        *(int64_t*)out = acc;
        return 0;
    }
    }
    return -1;
}

int orc_gemv_sub_mt(int dtype, const void* mat, int64_t ld, int64_t row_off, int64_t col_off,
                    int64_t rows, int64_t cols, const void* vec, void* res, int threads) {
    switch (dtype) {
    case ORC_F32:
        run_blocks(rows, threads, [=](int64_t a, int64_t b) {
            gemv_rows_t<float>((const float*)mat, ld, row_off, col_off, a, b, cols,
                               (const float*)vec, (float*)res);
        });
        return 0;
    case ORC_F64:
        run_blocks(rows, threads, [=](int64_t a, int64_t b) {
            gemv_rows_t<double>((const double*)mat, ld, row_off, col_off, a, b, cols,
                                (const double*)vec, (double*)res);
        });
        return 0;
    case ORC_I32:
        run_blocks(rows, threads, [=](int64_t a, int64_t b) {
            gemv_rows_t<int32_t>((const int32_t*)mat, ld, row_off, col_off, a, b, cols,
                                 (const int32_t*)vec, (int32_t*)res);
        });
        return 0;
    case ORC_I64:
        run_blocks(rows, threads, [=](int64_t a, int64_t b) {
            gemv_rows_t<int64_t>((const int64_t*)mat, ld, row_off, col_off, a, b, cols,
                                 (const int64_t*)vec, (int64_t*)res);
        });
        return 0;
    }
    return -1;
}

int orc_gemv_sub(int dtype, const void* mat, int64_t ld, int64_t row_off, int64_t col_off,
                 int64_t rows, int64_t cols, const void* vec, void* res) {
    return orc_gemv_sub_mt(dtype, mat, ld, row_off, col_off, rows, cols, vec, res, 1);
}

int orc_axpy1(int dtype, int64_t n, const void* partial, void* res) {
    switch (dtype) {
    case ORC_F32:
        for (int64_t i = 0; i < n; ++i)
            ((float*)res)[i] += ((const float*)partial)[i];
        return 0;
    case ORC_F64:
        for (int64_t i = 0; i < n; ++i)
            ((double*)res)[i] += ((const double*)partial)[i];
        return 0;
    case ORC_I32:
        for (int64_t i = 0; i < n; ++i)
            ((int32_t*)res)[i] = wrap_add<int32_t>(((int32_t*)res)[i], ((const int32_t*)partial)[i]);
        return 0;
    case ORC_I64:
        for (int64_t i = 0; i < n; ++i)
            ((int64_t*)res)[i] = wrap_add<int64_t>(((int64_t*)res)[i], ((const int64_t*)partial)[i]);
        return 0;
    }
    return -1;
}

int orc_gemm_acc_mt(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                    const void* B, int64_t ldb, void* C, int64_t ldc, int threads) {
    switch (dtype) {
    case ORC_F32:
        run_blocks(M, threads, [=](int64_t a, int64_t b) {
            gemm_rows_t<float>(a, b, N, K, (const float*)A, lda, (const float*)B, ldb, (float*)C, ldc);
        });
        return 0;
    case ORC_F64:
        run_blocks(M, threads, [=](int64_t a, int64_t b) {
            gemm_rows_t<double>(a, b, N, K, (const double*)A, lda, (const double*)B, ldb,
                                (double*)C, ldc);
        });
        return 0;
    case ORC_I32:
        run_blocks(M, threads, [=](int64_t a, int64_t b) {
            gemm_rows_t<int32_t>(a, b, N, K, (const int32_t*)A, lda, (const int32_t*)B, ldb,
                                 (int32_t*)C, ldc);
        });
        return 0;
    case ORC_I64:
        run_blocks(M, threads, [=](int64_t a, int64_t b) {
            gemm_rows_t<int64_t>(a, b, N, K, (const int64_t*)A, lda, (const int64_t*)B, ldb,
                                 (int64_t*)C, ldc);
        });
        return 0;
    }
    return -1;
}

int orc_gemm_acc(int dtype, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
                 const void* B, int64_t ldb, void* C, int64_t ldc) {
    return orc_gemm_acc_mt(dtype, M, N, K, A, lda, B, ldb, C, ldc, 1);
}

int orc_sum(int dtype, int64_t n, const void* a, void* out) {
    switch (dtype) {
    case ORC_F32: {
        float acc = 0;
        for (int64_t i = 0; i < n; ++i)
            acc += ((const float*)a)[i];
        *(float*)out = acc;
        return 0;
    }
    case ORC_F64: {
        double acc = 0;
        for (int64_t i = 0; i < n; ++i)
            acc += ((const double*)a)[i];
        *(double*)out = acc;
        return 0;
    }
    case ORC_I32: {
        int32_t acc = 0;
        for (int64_t i = 0; i < n; ++i)
            acc = wrap_add<int32_t>(acc, ((const int32_t*)a)[i]);
        *(int32_t*)out = acc;
        return 0;
    }
    case ORC_I64: {
        int64_t acc = 0;
        for (int64_t i = 0; i < n; ++i)
            acc = wrap_add<int64_t>(acc, ((const int64_t*)a)[i]);
        *(int64_t*)out = acc;
        return 0;
    }
    }
    return -1;
}

int orc_sumsq_diff(int64_t n, const double* a, const double* b, double* out) {
    double acc = 0;
    for (int64_t i = 0; i < n; ++i) {
        double d = a[i] - b[i];
        acc += d * d;
    }
    *out = acc;
    return 0;
}

int orc_maxabs_diff(int64_t n, const double* a, const double* b, double* out) {
    double m = 0;
    for (int64_t i = 0; i < n; ++i) {
        double d = std::fabs(a[i] - b[i]);
        if (d > m)
            m = d;
    }
    *out = m;
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Synthetic inputs: counter-based SplitMix64.
// ---------------------------------------------------------------------------------------------
uint64_t orc_splitmix(uint64_t seed, uint64_t stream, uint64_t i) {
    uint64_t s = seed * 0x9E3779B97F4A7C15ull + stream * 0xD1B54A32D192ED03ull + i;
    uint64_t z = s + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

double orc_u01(uint64_t seed, uint64_t stream, uint64_t i) {
    return (double)(orc_splitmix(seed, stream, i) >> 11) * 0x1.0p-53;
}

void orc_fill_uniform(double* out, int64_t n, uint64_t seed, uint64_t stream, uint64_t first,
                      double lo, double hi) {
    double w = hi - lo;
    for (int64_t k = 0; k < n; ++k) {
        double prod = w * orc_u01(seed, stream, first + (uint64_t)k);
        out[k] = lo + prod;
    }
}

void orc_fill_cg_matrix(double* out, int64_t n, int64_t row0, int64_t nrows, int64_t col0,
                        int64_t ncols, int64_t ld, uint64_t seed) {
    double denom = 2.0 * (double)n;
    for (int64_t i = 0; i < nrows; ++i)
        for (int64_t j = 0; j < ncols; ++j) {
            int64_t gi = row0 + i, gj = col0 + j;
            double v;
            if (gi == gj)
                v = 2.0;
            else {
                double s = orc_u01(seed, 0, (uint64_t)(gi * n + gj)) +
                           orc_u01(seed, 0, (uint64_t)(gj * n + gi));
                v = s / denom;
            }
            out[i * ld + j] = v;
        }
}

} // extern "C"

// ---------------------------------------------------------------------------------------------
// One fused SET_REGION group over one tiled array, carried out chare by chare the way the
// reference does it: every chare packs the pieces of its tile that other chares' shifted
// operands need (send_remote_inputs + send_remote_input, src/executor_core.cpp:8-143,684-690),
// the receiving chare lists its local fragment and the received buffers per operand, refines them
// into aligned cells, runs the group once per cell into a packed result buffer
// (src/execute_node.cpp:1376-1585) and finally copies the buffer into its tile
// (SET_REGION, src/executor_ast_visitor.cpp:268-311). Offsets 0, every leaf is the assigned array.
// ---------------------------------------------------------------------------------------------
namespace {

struct RemoteBuffer {
    int input_index;
    orc_region region;
    std::vector<char> data;
};

int tile_count(const orc_decomp& dc, int d) { return orc_decomp_num_chares(&dc, d); }

} // namespace

extern "C" int orc_world_group(const orc_ast* ast, int dtype, int nd, const int32_t* shape, int tile,
                               void* const* tiles, int threads, int64_t* stats) {
    if (nd < 1 || nd > ORC_MAX_ND || dtype < 0 || dtype > 3)
        return -2;
    const int esz = (dtype == ORC_F32 || dtype == ORC_I32) ? 4 : 8;
    Program p = build_program(ast);
    if (p.err)
        return p.err;
    if (p.out_roots.size() != 1)
        return -3;
    const orc_ast_node& root = ast->nodes[ast->roots[p.out_roots[0]]];
    if (root.opcode != ORC_OP_SET_REGION || root.region.is_global || !p.bcast_nodes.empty())
        return -3;
    const int target = ast->nodes[root.operands[0]].result_name;
    const orc_region r_out = root.region;
    const int K = (int)p.leaves.size();
    std::vector<orc_region> inputs(K);
    for (int k = 0; k < K; ++k) {
        const orc_ast_node& leaf = ast->nodes[p.leaves[k].node];
        const orc_ast_node& user = ast->nodes[ast->roots[p.leaves[k].root]];
        if (leaf.result_name != target || !user.has_operand_region[p.leaves[k].operand])
            return -3;
        inputs[k] = user.operand_regions[p.leaves[k].operand];
    }
    orc_decomp dc;
    std::memset(&dc, 0, sizeof dc);
    dc.ndims = nd;
    dc.tile = tile;
    int grid[ORC_MAX_ND] = {1, 1, 1};
    int64_t nchares = 1;
    for (int d = 0; d < nd; ++d) {
        dc.global_shape[d] = shape[d];
        grid[d] = tile_count(dc, d);
        nchares *= grid[d];
    }
    std::vector<orc_decomp> in_dc(K, dc);
    auto chare_index = [&](int64_t c, int32_t* idx) {
        for (int d = nd - 1; d >= 0; --d) {
            idx[d] = (int32_t)(c % grid[d]);
            c /= grid[d];
        }
    };
    auto chare_flat = [&](const int32_t* idx) {
        int64_t c = 0;
        for (int d = 0; d < nd; ++d)
            c = c * grid[d] + idx[d];
        return c;
    };
    auto tile_strides = [&](const orc_region& chare, int64_t* st) {
        int64_t sdim = 1;
        for (int d = nd - 1; d >= 0; --d) {
            st[d] = sdim;
            sdim *= rsize(chare, d);
        }
    };
    int64_t n_msgs = 0, n_bytes = 0, n_kernels = 0, n_cells_max = 0;

    // ---- phase 1: every chare packs and "sends" what others need from its tile ----
    std::vector<std::vector<RemoteBuffer>> inbox((size_t)nchares);
    for (int64_t c = 0; c < nchares; ++c) {
        int32_t idx[ORC_MAX_ND] = {0, 0, 0};
        chare_index(c, idx);
        orc_region chare;
        orc_decomp_chare_region_global(&dc, idx, &chare);
        int64_t cst[ORC_MAX_ND];
        tile_strides(chare, cst);
        const int cap = 4096;
        std::vector<int32_t> targets((size_t)cap * nd), which(cap);
        std::vector<orc_region> regs(cap);
        int ns = orc_send_remote_inputs(&r_out, K, inputs.data(), idx, &dc, in_dc.data(), cap,
                                        targets.data(), regs.data(), which.data());
        if (ns < 0)
            return -4;
        for (int m = 0; m < ns; ++m) {
            RemoteBuffer rb;
            rb.input_index = which[m];
            rb.region = regs[m];
            int64_t counts[ORC_MAX_ND], sstart[ORC_MAX_ND], sstep[ORC_MAX_ND], dstart[ORC_MAX_ND],
                dstep[ORC_MAX_ND], dstr[ORC_MAX_ND];
            int64_t total = 1;
            for (int d = 0; d < nd; ++d) {
                counts[d] = rsize(regs[m], d);
                total *= counts[d];
            }
            int64_t sdim = 1;
            for (int d = nd - 1; d >= 0; --d) {
                dstr[d] = sdim;
                sdim *= counts[d];
                sstart[d] = regs[m].start[d] - chare.start[d];
                sstep[d] = regs[m].step[d];
                dstart[d] = 0;
                dstep[d] = 1;
            }
            rb.data.resize((size_t)total * esz);
            orc_copy_region(nd, esz, rb.data.data(), dstr, dstart, dstep, tiles[c], cst, sstart, sstep,
                            counts);
            n_msgs++;
            n_bytes += total * esz;
            inbox[(size_t)chare_flat(&targets[(size_t)m * nd])].push_back(std::move(rb));
        }
    }

    // ---- phases 2 and 3 per chare: fragments -> aligned cells -> kernels -> SET_REGION copy ----
    std::vector<int> rc_of((size_t)nchares, 0);
    std::vector<int64_t> kern_of((size_t)nchares, 0), cells_of((size_t)nchares, 0);
    std::vector<std::vector<char>> results((size_t)nchares);
    std::vector<orc_region> myouts((size_t)nchares);
    std::vector<char> has_out((size_t)nchares, 0);
    run_blocks(nchares, threads, [&](int64_t c0, int64_t c1) {
        for (int64_t c = c0; c < c1; ++c) {
            int32_t idx[ORC_MAX_ND] = {0, 0, 0};
            chare_index(c, idx);
            orc_region chare, myout;
            orc_decomp_chare_region_global(&dc, idx, &chare);
            if (!orc_region_intersect(&r_out, &chare, &myout))
                continue;
            has_out[(size_t)c] = 1;
            myouts[(size_t)c] = myout;
            std::vector<orc_region> my_inputs(K);
            int expected = 0;
            if (orc_local_inputs(&r_out, K, inputs.data(), idx, &dc, in_dc.data(), my_inputs.data(),
                                 &expected) < 0) {
                rc_of[(size_t)c] = -5;
                continue;
            }
            if (expected != (int)inbox[(size_t)c].size()) {
                rc_of[(size_t)c] = -6; // planner inconsistency: sends do not match expectations
                continue;
            }
            int64_t cst[ORC_MAX_ND];
            tile_strides(chare, cst);
            std::vector<orc_fragment> frags;
            std::vector<const char*> bases;
            std::vector<int32_t> begin(K + 1, 0);
            for (int k = 0; k < K; ++k) {
                begin[k] = (int32_t)frags.size();
                orc_region local;
                if (orc_region_intersect(&my_inputs[k], &chare, &local)) {
                    orc_fragment f;
                    std::memset(&f, 0, sizeof f);
                    f.region = local;
                    int64_t off = 0;
                    for (int d = 0; d < nd; ++d) {
                        f.src_strides[d] = cst[d];
                        off += (int64_t)(local.start[d] - chare.start[d]) * cst[d];
                    }
                    frags.push_back(f);
                    bases.push_back(static_cast<const char*>(tiles[c]) + off * esz);
                }
                for (const RemoteBuffer& rb : inbox[(size_t)c])
                    if (rb.input_index == k) {
                        orc_fragment f;
                        std::memset(&f, 0, sizeof f);
                        f.region = rb.region; // packed: strides all 0
                        frags.push_back(f);
                        bases.push_back(rb.data.data());
                    }
            }
            begin[K] = (int32_t)frags.size();
            const int cap = 1024;
            std::vector<int32_t> of((size_t)cap * K);
            std::vector<int64_t> oo((size_t)cap * K), osz((size_t)cap * K * ORC_MAX_ND),
                ost((size_t)cap * K * ORC_MAX_ND);
            std::vector<orc_region> cells((size_t)cap * K);
            int M = orc_align_fragments(nd, K, begin.data(), frags.data(), my_inputs.data(), cap,
                                        of.data(), oo.data(), osz.data(), ost.data(), cells.data());
            if (M < 0) {
                rc_of[(size_t)c] = -7;
                continue;
            }
            cells_of[(size_t)c] = M;
            // packed result buffer of this chare's part of the assigned region
            int64_t rsz[ORC_MAX_ND], rst[ORC_MAX_ND], total = 1;
            for (int d = 0; d < nd; ++d)
                rsz[d] = rsize(myout, d);
            for (int d = nd - 1; d >= 0; --d) {
                rst[d] = total;
                total *= rsz[d];
            }
            results[(size_t)c].assign((size_t)total * esz, 0);
            for (int m = 0; m < M; ++m) {
                std::vector<orc_memref> in(K);
                for (int k = 0; k < K; ++k) {
                    const size_t at = (size_t)k * M + m;
                    orc_memref& mr = in[k];
                    std::memset(&mr, 0, sizeof mr);
                    char* ptr = const_cast<char*>(bases[of[at]]) + oo[at] * esz;
                    mr.allocated = mr.aligned = ptr;
                    for (int d = 0; d < nd; ++d) {
                        mr.sizes[d] = osz[at * ORC_MAX_ND + d];
                        mr.strides[d] = ost[at * ORC_MAX_ND + d];
                    }
                }
                // where the cell lands in the result buffer: its corner mapped from operand 0's
                // index space to the assigned region (src/execute_node.cpp:1492-1506)
                orc_region corner;
                orc_region_map(&cells[(size_t)0 * M + m], &my_inputs[0], &myout, &corner);
                int64_t off = 0;
                for (int d = 0; d < nd; ++d)
                    off += ((int64_t)(corner.start[d] - myout.start[d]) / myout.step[d]) * rst[d];
                orc_memref out;
                std::memset(&out, 0, sizeof out);
                out.allocated = out.aligned = results[(size_t)c].data() + off * esz;
                for (int d = 0; d < nd; ++d) {
                    out.sizes[d] = in[0].sizes[d];
                    out.strides[d] = rst[d];
                }
                int rc = orc_eval_group(ast, dtype, nd, K, in.data(), 0, nullptr, 1, &out);
                if (rc) {
                    rc_of[(size_t)c] = rc;
                    break;
                }
                kern_of[(size_t)c]++;
            }
        }
    });
    for (int64_t c = 0; c < nchares; ++c) {
        if (rc_of[(size_t)c])
            return rc_of[(size_t)c];
        n_kernels += kern_of[(size_t)c];
        n_cells_max = std::max(n_cells_max, cells_of[(size_t)c]);
    }
    // SET_REGION: packed result buffer -> strided part of the tile, one element at a time
    run_blocks(nchares, threads, [&](int64_t c0, int64_t c1) {
        for (int64_t c = c0; c < c1; ++c) {
            if (!has_out[(size_t)c])
                continue;
            int32_t idx[ORC_MAX_ND] = {0, 0, 0};
            chare_index(c, idx);
            orc_region chare;
            orc_decomp_chare_region_global(&dc, idx, &chare);
            const orc_region& myout = myouts[(size_t)c];
            int64_t cst[ORC_MAX_ND], counts[ORC_MAX_ND], sstr[ORC_MAX_ND], sstart[ORC_MAX_ND],
                sstep[ORC_MAX_ND], dstart[ORC_MAX_ND], dstep[ORC_MAX_ND];
            tile_strides(chare, cst);
            int64_t sdim = 1;
            for (int d = nd - 1; d >= 0; --d) {
                counts[d] = rsize(myout, d);
                sstr[d] = sdim;
                sdim *= counts[d];
                sstart[d] = 0;
                sstep[d] = 1;
                dstart[d] = myout.start[d] - chare.start[d];
                dstep[d] = myout.step[d];
            }
            orc_copy_region(nd, esz, tiles[c], cst, dstart, dstep, results[(size_t)c].data(), sstr,
                            sstart, sstep, counts);
        }
    });
    if (stats) {
        stats[0] = n_msgs;
        stats[1] = n_bytes;
        stats[2] = n_kernels;
        stats[3] = n_cells_max;
    }
    return 0;
}
