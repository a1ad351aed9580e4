// Register-window source for same-array unit-step stencils (the Jacobi-style SET_REGION groups),
// optionally with operands of other arrays read at the element's own position (source terms) or,
// in the whole-array kernel, at shifted positions too (a window per array).
//
// Every lane owns RZ x RY output rows of one 16-byte column pair inside ONE tile. It first issues
// all the 128-bit loads of its window (the rows and planes its shifted operands touch, aligned
// pairs only), then evaluates the group from registers and writes 128-bit results. There is no
// LDS staging, no barrier and no loop-carried wait: on this part a grid that covers the array
// once with many independent loads per lane streams faster than a marched or persistent form.
// Neighbour tiles are read in place: the 27 tile pointers around the workgroup's tile are
// workgroup-uniform, and a lane picks among them with selects only for the directions a given
// load can cross. Workgroups are ordered tile by tile (x fastest, then y, then z inside a tile)
// and dealt to the 8 XCDs in contiguous runs, so the planes a tile re-reads stay in one L2.
#include "codegen.h"

#include <algorithm>
#include <sstream>

namespace cnh {

int direct_shape(const GroupProgram& p, const DirectConfig& cfg, DirectShape& sh, std::string& err) {
    sh = DirectShape();
    if (p.ndims != 2 && p.ndims != 3) {
        err = "register-window stencil needs rank 2 or 3";
        return -18;
    }
    const int nroots = (int)p.out_roots.size();
    if (nroots < 1 || nroots > 2) {
        err = "register-window stencil needs one or two SET_REGION roots";
        return -18;
    }
    for (int j = 0; j < nroots; ++j)
        if (!p.out_is_set_region[(size_t)j] || p.out_region[(size_t)j].is_global || p.out_reduce[(size_t)j] ||
            p.out_target[(size_t)j] != p.out_target[0]) {
            err = "register-window stencil needs SET_REGION roots on one array";
            return -18;
        }
    sh.nroots = nroots;
    // A lane works on pairs of elements: 16-byte accesses for 8-byte types, 8-byte accesses for
    // 4-byte types (half the width per access, still one coalesced run per wavefront).
    const cnh_region& ro = p.out_region[0];
    const int nd = p.ndims, pad = CNH_MAX_ND - nd;
    for (int d = 0; d < nd; ++d) {
        if (ro.step[d] != 1 && ro.step[d] != 2) {
            err = "assigned region has a step other than 1 or 2";
            return -18;
        }
        sh.lat[pad + d] = ro.step[d] - 1;
        sh.lattice = sh.lattice || ro.step[d] == 2;
    }
    sh.lattice = sh.lattice || nroots == 2;
    for (int j = 1; j < nroots; ++j) {
        const cnh_region& rj = p.out_region[(size_t)j];
        bool apart = false;
        for (int d = 0; d < nd; ++d) {
            if (rj.step[d] != ro.step[d]) {
                err = "the roots' regions differ in step";
                return -18;
            }
            apart = apart || (ro.step[d] == 2 && ((rj.start[d] - ro.start[d]) & 1) != 0);
        }
        if (!apart) {
            err = "the roots' lattices can meet";
            return -18;
        }
    }
    if (p.load_leaf.empty()) {
        err = "no array operand";
        return -18;
    }
    // the SET_REGION root a leaf use works for: the first output at or after its root position
    auto owner_of = [&](const LeafUse& u) {
        for (int j = 0; j < nroots; ++j)
            if (p.out_roots[(size_t)j] >= u.root)
                return j;
        return nroots - 1;
    };
    const size_t NLd = p.load_leaf.size();
    sh.shifts.assign(NLd, {0, 0, 0});
    sh.shifts2.assign(NLd, {0, 0, 0});
    sh.other.assign(NLd, -1);
    // every use of a load by one root must sit at the same offset from that root's lattice
    std::vector<std::array<int, 3>> rel[2] = {std::vector<std::array<int, 3>>(NLd, {0, 0, 0}),
                                               std::vector<std::array<int, 3>>(NLd, {0, 0, 0})};
    std::vector<int> seen[2] = {std::vector<int>(NLd, 0), std::vector<int>(NLd, 0)};
    for (const LeafUse& u : p.leaves) {
        if (!u.has_region) {
            err = "operand without a region";
            return -18;
        }
        const int j = owner_of(u);
        const cnh_region& rr = p.out_region[(size_t)j];
        std::array<int, 3> off = {0, 0, 0};
        for (int d = 0; d < nd; ++d) {
            if (u.region.step[d] != rr.step[d] ||
                (u.region.stop[d] - u.region.start[d] + rr.step[d] - 1) / rr.step[d] !=
                    (rr.stop[d] - rr.start[d] + rr.step[d] - 1) / rr.step[d]) {
                err = "operand region differs from the assigned one in step or extent";
                return -18;
            }
            off[(size_t)(pad + d)] = u.region.start[d] - rr.start[d];
        }
        if (seen[j][(size_t)u.load] && rel[j][(size_t)u.load] != off) {
            err = "one load is used at two offsets";
            return -18;
        }
        seen[j][(size_t)u.load] = 1;
        rel[j][(size_t)u.load] = off;
    }
    auto shifted_at = [&](int j, size_t l) {
        return seen[j][l] && (rel[j][l][0] != 0 || rel[j][l][1] != 0 || rel[j][l][2] != 0);
    };
    // The window array: an array read at positions other than the element's own -- the assigned
    // one if it is among them (its sweep then goes into a second buffer), else the first such
    // array; the assigned array when there is none. Further arrays read at shifted positions get
    // windows of their own in the whole-array kernel (other_shifted).
    sh.window_name = p.out_target[0];
    bool found_shifted = false, target_shifted = false;
    for (size_t l = 0; l < NLd; ++l) {
        const LeafUse& u = p.leaves[p.load_leaf[l]];
        if (!shifted_at(0, l) && !shifted_at(1, l))
            continue;
        target_shifted = target_shifted || u.name == p.out_target[0];
        if (!found_shifted)
            sh.window_name = u.name;
        found_shifted = true;
    }
    if (target_shifted)
        sh.window_name = p.out_target[0];
    sh.masked = sh.window_name != p.out_target[0];
    if (sh.masked && sh.lattice) {
        err = "a lattice sweep reads its own array through the window";
        return -18;
    }
    bool reads_target = false;
    sh.inplace_safe = sh.lattice;
    for (size_t l = 0; l < NLd; ++l) {
        const LeafUse& u = p.leaves[p.load_leaf[l]];
        if (u.name != sh.window_name) {
            // another array (a source term, a weight): at the element's own position, or shifted
            // (a window of its own, whole-array kernel, one root, unit steps)
            if (shifted_at(0, l) || shifted_at(1, l)) {
                if (sh.lattice || nroots != 1) {
                    err = "a lattice sweep reads other arrays at the element's own position only";
                    return -18;
                }
                sh.other_shifted = true;
                for (int d = 0; d < 3; ++d) {
                    sh.shifts[l][(size_t)d] = rel[0][l][(size_t)d];
                    sh.halo[d] = std::max(sh.halo[d], std::abs(rel[0][l][(size_t)d]));
                }
            }
            size_t j = 0;
            while (j < sh.other_names.size() && sh.other_names[j] != u.name)
                ++j;
            if (j == sh.other_names.size()) {
                if ((int)j == kDirectMaxOther) {
                    err = "too many arrays";
                    return -18;
                }
                sh.other_names.push_back(u.name);
            }
            sh.other[l] = (int)j;
            continue;
        }
        reads_target = true;
        for (int j = 0; j < nroots; ++j) {
            if (!seen[j][l])
                continue;
            for (int d = 0; d < 3; ++d) {
                (j == 0 ? sh.shifts : sh.shifts2)[l][(size_t)d] = rel[j][l][(size_t)d];
                sh.halo[d] = std::max(sh.halo[d], std::abs(rel[j][l][(size_t)d]));
            }
            // in place: a shifted read must miss every assigned lattice in some stepped dimension
            if (sh.lattice && shifted_at(j, l)) {
                const cnh_region& rr = p.out_region[(size_t)j];
                for (int q = 0; q < nroots; ++q) {
                    const cnh_region& rq = p.out_region[(size_t)q];
                    bool misses = false;
                    for (int d = 0; d < nd; ++d)
                        misses = misses || (rq.step[d] == 2 &&
                                            ((rr.start[d] + rel[j][l][(size_t)(pad + d)] - rq.start[d]) & 1) != 0);
                    sh.inplace_safe = sh.inplace_safe && misses;
                }
            }
        }
    }
    if (!reads_target) {
        err = "no array is read through a window";
        return -18;
    }
    for (int d = 0; d < 3; ++d)
        if (sh.halo[d] > 2) {
            err = "halo wider than 2";
            return -18;
        }
    // measured on MI355X: 2 rows per lane for rank 2; 2 rows x 4 planes per lane for rank 3
    sh.tx = 64;
    sh.ry = 2;
    sh.rz = nd == 3 ? 4 : 1;
    if (cfg.tx > 0)
        sh.tx = cfg.tx;
    if (cfg.ry > 0)
        sh.ry = cfg.ry;
    if (cfg.rz > 0 && nd == 3)
        sh.rz = cfg.rz;
    if (sh.tx < 1 || sh.tx > 256 || (sh.tx & (sh.tx - 1)) || sh.ry < 1 || sh.ry > 16 || sh.rz < 1 ||
        sh.rz > 8) {
        err = "bad register-window geometry";
        return -18;
    }
    sh.ty = 256 / sh.tx;
    sh.tail_ok = false;
    if (!sh.masked && !sh.lattice && sh.nroots == 1 && sh.halo[2] >= 1)
        for (size_t l = 0; l < NLd; ++l)
            if (sh.other[l] < 0 && sh.shifts[l][0] == 0 && sh.shifts[l][1] == 0 && sh.shifts[l][2] >= 1)
                sh.tail_ok = true;
    const int hk = (sh.halo[2] + 1) / 2; // column pairs to each side
    const int window = (sh.rz + 2 * sh.halo[0]) * (sh.ry + 2 * sh.halo[1]) * (2 * hk + 1);
    if (window > 96) {
        err = "register window too large";
        return -18;
    }
    return 0;
}

std::string direct_source(const GroupProgram& p, const DirectConfig& cfg, std::string& err) {
    DirectShape sh;
    if (direct_shape(p, cfg, sh, err))
        return std::string();
    std::string pre;
    if (emit_variant_source(p, "prelude", pre, err) != 0)
        return std::string();
    const int H0 = sh.halo[0], H1 = sh.halo[1], H2 = sh.halo[2];
    const int HK = (H2 + 1) / 2;
    const int WZ = sh.rz + 2 * H0, WY = sh.ry + 2 * H1, WK = 2 * HK + 1;
    // Which window entries does some output of the lane read?
    std::vector<int> need((size_t)WZ * WY * WK, 0);
    auto at = [&](int z, int y, int k) -> int& { return need[((size_t)z * WY + y) * WK + k]; };
    auto floordiv2 = [](int v) { return v >= 0 ? v / 2 : -((-v + 1) / 2); };
    for (int rz = 0; rz < sh.rz; ++rz)
        for (int ry = 0; ry < sh.ry; ++ry) {
            if (!sh.masked)
                at(rz + H0, ry + H1, HK) = 1; // the element itself (kept outside the assigned region)
            for (int e = 0; e < 2; ++e) {
                for (size_t l = 0; l < sh.shifts.size(); ++l) {
                    if (sh.other_shifted && sh.other[l] >= 0)
                        continue;                 // read through its own array's window, below
                    const auto& s = sh.shifts[l];
                    at(rz + H0 + s[0], ry + H1 + s[1], HK + floordiv2(e + s[2])) = 1;
                }
                if (sh.nroots > 1)
                    for (const auto& s : sh.shifts2)
                        at(rz + H0 + s[0], ry + H1 + s[1], HK + floordiv2(e + s[2])) = 1;
            }
        }
    // the same per other array, when some of them are read at shifted positions
    const int NOTH0 = (int)sh.other_names.size();
    std::vector<int> oneed((size_t)std::max(1, NOTH0) * WZ * WY * WK, 0);
    auto oat = [&](int j, int z, int y, int k) -> int& { return oneed[(((size_t)j * WZ + z) * WY + y) * WK + k]; };
    if (sh.other_shifted)
        for (int rz = 0; rz < sh.rz; ++rz)
            for (int ry = 0; ry < sh.ry; ++ry)
                for (int e = 0; e < 2; ++e)
                    for (size_t l = 0; l < sh.shifts.size(); ++l)
                        if (sh.other[l] >= 0) {
                            const auto& sft = sh.shifts[l];
                            oat(sh.other[l], rz + H0 + sft[0], ry + H1 + sft[1], HK + floordiv2(e + sft[2])) = 1;
                        }
    std::ostringstream s;
    s << pre;
    s << "#define DR_TX " << sh.tx << "\n#define DR_TY " << sh.ty << "\n#define DR_RY " << sh.ry
      << "\n#define DR_RZ " << sh.rz << "\n#define DR_H0 " << H0 << "\n#define DR_H1 " << H1
      << "\n#define DR_H2 " << H2 << "\n#define DR_HK " << HK << "\n";
    s << "#define DR_WZ " << WZ << "\n#define DR_WY " << WY << "\n#define DR_WK " << WK << "\n";
    s << "__device__ constexpr int DR_SHIFT[NLA][3] = {";
    for (size_t l = 0; l < sh.shifts.size(); ++l)
        s << (l ? ", " : "") << "{" << sh.shifts[l][0] << ", " << sh.shifts[l][1] << ", "
          << sh.shifts[l][2] << "}";
    s << "};\n";
    s << "__device__ constexpr int DR_SHIFT2[NLA][3] = {";
    for (size_t l = 0; l < sh.shifts2.size(); ++l)
        s << (l ? ", " : "") << "{" << sh.shifts2[l][0] << ", " << sh.shifts2[l][1] << ", "
          << sh.shifts2[l][2] << "}";
    s << "};\n#define DR_NROOTS " << sh.nroots << "\n";
    const int NOTH = (int)sh.other_names.size();
    s << "#define DR_MASKED " << (sh.masked ? 1 : 0) << "\n";
    s << "#define DR_TAIL_OK " << (sh.tail_ok ? 1 : 0) << "\n";
    s << "#define DR_OSH " << (sh.other_shifted ? 1 : 0) << "\n";
    s << "#define DR_RED " << (cfg.reduce ? 1 : 0) << "\n";
    s << "#define DR_NOTH " << NOTH << "\n#define DR_NOTHA " << (NOTH > 0 ? NOTH : 1) << "\n";
    s << "__device__ constexpr int DR_OTHER[NLA] = {";
    for (size_t l = 0; l < sh.other.size(); ++l)
        s << (l ? ", " : "") << sh.other[l];
    s << "};\n";
    // Rows of the window whose first or last lane needs the pair beyond the wavefront's 128
    // columns. When they form a full block of 4 to 32 rows, one partial load per wavefront
    // fetches all of them (lane 2r + side for row r) and lanes 0 and 63 pick theirs by readlane.
    int bi0 = WZ, bi1 = -1, bj0 = WY, bj1 = -1, brows = 0;
    for (int z = 0; z < WZ; ++z)
        for (int y = 0; y < WY; ++y)
            if (at(z, y, 0) || at(z, y, WK - 1)) {
                bi0 = std::min(bi0, z);
                bi1 = std::max(bi1, z);
                bj0 = std::min(bj0, y);
                bj1 = std::max(bj1, y);
                ++brows;
            }
    // (with two rows, rank 2, the row-by-row form measured 0.7 % faster: 184.0 against 185.3 us)
    const bool gather = brows >= 4 && brows == (bi1 - bi0 + 1) * (bj1 - bj0 + 1) && brows <= 32 && HK == 1;
    s << "#define DR_EDGE_GATHER " << (gather ? 1 : 0) << "\n#define DR_BI0 " << (gather ? bi0 : 0)
      << "\n#define DR_BJ0 " << (gather ? bj0 : 0) << "\n#define DR_BNJ " << (gather ? bj1 - bj0 + 1 : 1)
      << "\n#define DR_NB " << (gather ? brows : 0) << "\n";
    s << "__device__ constexpr bool DR_NEED[DR_WZ][DR_WY][DR_WK] = {";
    for (int z = 0; z < WZ; ++z) {
        s << (z ? ", " : "") << "{";
        for (int y = 0; y < WY; ++y) {
            s << (y ? ", " : "") << "{";
            for (int k = 0; k < WK; ++k)
                s << (k ? ", " : "") << (at(z, y, k) ? "true" : "false");
            s << "}";
        }
        s << "}";
    }
    s << "};\n";
    s << "__device__ constexpr bool DR_ONEED[DR_NOTHA][DR_WZ][DR_WY][DR_WK] = {";
    for (int j = 0; j < std::max(1, NOTH0); ++j) {
        s << (j ? ", " : "") << "{";
        for (int z = 0; z < WZ; ++z) {
            s << (z ? ", " : "") << "{";
            for (int y = 0; y < WY; ++y) {
                s << (y ? ", " : "") << "{";
                for (int k = 0; k < WK; ++k)
                    s << (k ? ", " : "") << (oat(j, z, y, k) ? "true" : "false");
                s << "}";
            }
            s << "}";
        }
        s << "}";
    }
    s << "};\n";
    s << R"(
// n / d for 0 <= n < 2^31 as a multiply and a shift; the host fills m and s.
struct FDiv { unsigned d, m, s; };
__device__ __forceinline__ int fdiv(int n, const FDiv& f) {
    return (int)(((unsigned long long)(unsigned)n * f.m) >> f.s);
}
struct DirectArgs {
    const T* const* cur;   // tile table of the current contents (row-major tile grid)
    T* const* dst;         // tile table of the new contents
    int tile;              // tile edge
    int shape[3];          // array extents (leading dims padded with 1)
    int grid[3];           // tiles per dimension
    int rs[3], re[3];      // assigned region
    int tb[3];             // workgroups per tile along z, y, x
    int sg[3];             // tiles per ordering group along z, y, x
    int nblocks;
    int nblocks8;          // nblocks / 8 when that is exact, else 0
    int stagger;           // rotation of the order inside group g by (g % 8) * stagger workgroups
    FDiv per_group;        // workgroups per ordering group
    FDiv ggrid1, ggrid2;   // ordering groups along y and x
    FDiv grow, gcol;       // workgroups per group along x and y
    FDiv tbz, tby, tbx;    // = tb[0], tb[1], tb[2]
    const T* const* oth[4]; // tile tables of the other arrays read at the element's own position
    int py, pz;            // elements between rows and between planes inside every tile when the
                           // tiles are views into one larger row-major block; 0: a tile is
                           // contiguous over its own extents
    T* slots;              // reducing launches: one partial per launched wavefront
};
typedef T P2 __attribute__((ext_vector_type(2)));
typedef int I2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int floordiv2(int v) { return v >= 0 ? v / 2 : -((-v + 1) / 2); }

// One pair of results. A sweep in place of the window array writes every pair whole (elements
// outside the assigned region carry their old values in `v`); a launch whose window array is
// another one (DR_MASKED) writes assigned elements only and leaves the rest of the target alone.
template <bool NTS>
__device__ __forceinline__ void store_pair(P2* out, P2 v, bool in0, bool in1) {
    if (!DR_MASKED || (in0 && in1)) {
        if (NTS) __builtin_nontemporal_store(v, out); else *out = v;
    } else {
        T* one = reinterpret_cast<T*>(out);
        if (in0) one[0] = v[0];
        if (in1) one[1] = v[1];
    }
}

// A build that runs the lanes of a wavefront as coroutines on a host (bounds checking of this
// source) supplies its own lane exchange and readfirstlane.
#ifndef DR_HOST_BUILD
// Value of the same register in the previous / next lane of the wavefront (whole-wave shift by
// one lane; the first / last lane keeps its own value and is patched by the caller).
template <int CTRL, typename V>
__device__ __forceinline__ V lane_shift(V v) {
    if constexpr (sizeof(V) == 8) {
        I2 a = __builtin_bit_cast(I2, v), r;
        r[0] = __builtin_amdgcn_update_dpp(a[0], a[0], CTRL, 0xf, 0xf, false);
        r[1] = __builtin_amdgcn_update_dpp(a[1], a[1], CTRL, 0xf, 0xf, false);
        return __builtin_bit_cast(V, r);
    } else {
        const int a = __builtin_bit_cast(int, v);
        return __builtin_bit_cast(V, __builtin_amdgcn_update_dpp(a, a, CTRL, 0xf, 0xf, false));
    }
}
// The value a given lane holds, as a wavefront-uniform value.
template <typename V>
__device__ __forceinline__ V from_lane(V v, int src) {
    if constexpr (sizeof(V) == 8) {
        I2 a = __builtin_bit_cast(I2, v), r;
        r[0] = __builtin_amdgcn_readlane(a[0], src);
        r[1] = __builtin_amdgcn_readlane(a[1], src);
        return __builtin_bit_cast(V, r);
    } else {
        return __builtin_bit_cast(V, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src));
    }
}
__device__ __forceinline__ T from_prev_lane(T v) { return lane_shift<0x138>(v); }
__device__ __forceinline__ T from_next_lane(T v) { return lane_shift<0x130>(v); }
__device__ __forceinline__ int wave_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
#endif

// Sum of a value over the 64 lanes of a wavefront in a fixed tree (all lanes active); lane 0
// holds the result. MAXV: the maximum instead.
template <bool MAXV, typename V>
__device__ __forceinline__ V wave_combine(V v) {
#ifndef DR_HOST_BUILD
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        V o;
        if constexpr (sizeof(V) == 8) {
            I2 a = __builtin_bit_cast(I2, v), r;
            r[0] = __shfl_down(a[0], off, 64);
            r[1] = __shfl_down(a[1], off, 64);
            o = __builtin_bit_cast(V, r);
        } else {
            o = __builtin_bit_cast(V, __shfl_down(__builtin_bit_cast(int, v), off, 64));
        }
        v = MAXV ? (o > v ? o : v) : v + o;
    }
#endif
    return v;
}

// Where a workgroup works: tile, tile extents, origin, and the patch inside the tile.
struct Place {
    int t, t0, t1, t2;           // tile index and coordinates
    int bx, by, bz;              // workgroup inside the tile
    int tz0, ty0, tx0;           // tile origin
    int w0, w1, w2;              // tile extents
};
// Consecutive workgroup ids go round the 8 XCDs; give every XCD one contiguous run instead.
__device__ __forceinline__ int xcd_order(const DirectArgs& a, int b) {
    return a.nblocks8 ? (b & 7) * a.nblocks8 + (b >> 3) : b;
}
__device__ __forceinline__ Place locate(const DirectArgs& a, int blk) {
    // Workgroups are ordered group by group (a group is sg^3 neighbouring tiles, so that what
    // the tiles of a group re-read from each other stays in one L2), and inside a group x
    // fastest, then y, then z across the whole group.
    const int g = fdiv(blk, a.per_group);
    // Groups that run at the same time start at different places of their tiles, so that they do
    // not walk through the same address offsets in step.
    int w = blk - g * (int)a.per_group.d + (g & 7) * a.stagger;
    if (w >= (int)a.per_group.d) w -= (int)a.per_group.d;
    const int gq = fdiv(g, a.ggrid2), g2 = g - gq * (int)a.ggrid2.d;
    const int g0 = fdiv(gq, a.ggrid1), g1 = gq - g0 * (int)a.ggrid1.d;
    const int wq = fdiv(w, a.grow), bxx = w - wq * (int)a.grow.d;
    const int bzz = fdiv(wq, a.gcol), byy = wq - bzz * (int)a.gcol.d;
    const int ix = fdiv(bxx, a.tbx), iy = fdiv(byy, a.tby), iz = fdiv(bzz, a.tbz);
    Place p;
    p.bx = bxx - ix * a.tb[2]; p.by = byy - iy * a.tb[1]; p.bz = bzz - iz * a.tb[0];
    p.t0 = g0 * a.sg[0] + iz; p.t1 = g1 * a.sg[1] + iy; p.t2 = g2 * a.sg[2] + ix;
    p.t = (p.t0 * a.grid[1] + p.t1) * a.grid[2] + p.t2;
    p.tz0 = p.t0 * a.tile; p.ty0 = p.t1 * a.tile; p.tx0 = p.t2 * a.tile;
    p.w0 = min(a.tile, a.shape[0] - p.tz0); p.w1 = min(a.tile, a.shape[1] - p.ty0);
    p.w2 = min(a.tile, a.shape[2] - p.tx0);
    return p;
}

// A wavefront takes the fast path when it is one run of 64 column pairs of one row group, its
// rows and planes plus halo lie inside the tile, and all its rows and planes are assigned. Only
// the x direction then needs care: the pairs to the left and right of a lane are its neighbour
// lanes' centre pairs, and the two end lanes read theirs from the tile or its x neighbour.
#define DR_WAVE_ROWS (DR_TX % 64 == 0)
__device__ __forceinline__ bool wave_is_fast(const DirectArgs& a, const Place& p, int lz0, int ly0,
                                             int x0) {
    return DR_WAVE_ROWS && DR_HK == 1 && x0 + 128 <= p.w2 &&
           ly0 - DR_H1 >= 0 && ly0 + DR_RY + DR_H1 <= p.w1 &&
           lz0 - DR_H0 >= 0 && lz0 + DR_RZ + DR_H0 <= p.w0 &&
           p.ty0 + ly0 >= a.rs[1] && p.ty0 + ly0 + DR_RY <= a.re[1] &&
           p.tz0 + lz0 >= a.rs[0] && p.tz0 + lz0 + DR_RZ <= a.re[0];
}

// RED: 0 = plain sweep; 1 = also the sum over the assigned elements of (new - old)^2; 2 = also the
// maximum of |new - old|. A reducing launch leaves one partial per launched wavefront in
// a.slots[4 * workgroup + wavefront] (0 from wavefronts that have nothing to do), added up
// afterwards in index order: the result never depends on scheduling.
template <bool NTS, int RED>
__device__ __forceinline__ void direct_fast(const DirectArgs& a, const T* s) {
    T* const my_slot = RED ? a.slots + ((size_t)blockIdx.x * 4 + (threadIdx.x >> 6)) : nullptr;
    const Place p = locate(a, xcd_order(a, (int)blockIdx.x));
    const int tid = (int)threadIdx.x;
    const int wv = wave_uniform(tid >> 6);              // wavefront inside the workgroup
    const int lane = tid & 63;
    const int lz0 = p.bz * DR_RZ;
    const int ly0 = (p.by * DR_TY + (wv * 64) / DR_TX) * DR_RY;
    const int x0 = (p.bx * DR_TX + (wv * 64) % DR_TX) * 2;   // first column of the wavefront
    // (both exits are taken by whole wavefronts: DR_TX is a multiple of 64 on this path)
    if (lz0 >= p.w0 || ly0 >= p.w1 || x0 >= p.w2 || !wave_is_fast(a, p, lz0, ly0, x0)) {
        if (RED && lane == 0) *my_slot = (T)0;
        return;
    }
    const int w1 = p.w1, w2 = p.w2;
    const int lx = x0 + 2 * lane;
    const T* const own = a.cur[p.t];
    // row and plane strides of this tile and of its x neighbours (their rows are as long as
    // they are wide unless all tiles are views with common pitches)
    const int PY = a.py ? a.py : w2, PZ = a.py ? a.pz : w1 * w2;
    const int oz = lz0 - DR_H0, oy = ly0 - DR_H1;                    // window origin (plane, row)
    const int origin = oz * PZ + oy * PY;
    const T* const pc = own + origin + lx;
    // where the end lanes find the pair before column x0 and the pair after column x0+127
    const T* lp = own + origin + x0;      // fallback: an address that exists (value unused)
    int lpy = PY, lpz = PZ;
    if (x0 >= 2) lp = own + origin + (x0 - 2);
    else if (p.t2 > 0) {
        lpy = a.py ? a.py : a.tile; lpz = a.py ? a.pz : w1 * a.tile;
        lp = a.cur[p.t - 1] + oz * lpz + oy * lpy + (a.tile - 2);
    }
    const T* rp = own + origin + (x0 + 126);
    int rpy = PY, rpz = PZ;
    if (x0 + 130 <= w2) rp = own + origin + (x0 + 128);
    else if (p.t2 + 1 < a.grid[2]) {
        const int rw = min(a.tile, a.shape[2] - p.tx0 - a.tile);
        rpy = a.py ? a.py : rw; rpz = a.py ? a.pz : w1 * rw;
        rp = a.cur[p.t + 1] + oz * rpz + oy * rpy;
    }
    const bool first = lane == 0, last = lane == 63;

    // All loads first. The pairs beyond the two ends of the wavefront are fetched by one load when
    // the rows that need them form a block (the usual case); otherwise the two end lanes fetch
    // theirs row by row while every other lane re-reads its own centre pair (a cache hit), one
    // more full-wave load per row. Either way the wavefront waits for memory once.
    P2 win[DR_WZ][DR_WY][DR_WK];
    P2 beyond[DR_WZ][DR_WY];
#pragma unroll
    for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
        for (int j = 0; j < DR_WY; ++j)
            if (DR_NEED[i][j][0] || DR_NEED[i][j][DR_HK] || DR_NEED[i][j][DR_WK - 1])
                win[i][j][DR_HK] = *reinterpret_cast<const P2*>(pc + i * PZ + j * PY);
    P2 edge = (P2){(T)0, (T)0};
    if (DR_EDGE_GATHER) {
        // one load for all of them: lane 2r holds the pair left of row r, lane 2r + 1 the pair
        // right of it (r counts the rows of the block in row-major order)
        if (lane < 2 * DR_NB) {
            const int r = lane >> 1, i = DR_BI0 + r / DR_BNJ, j = DR_BJ0 + r % DR_BNJ;
            const T* src = (lane & 1) ? rp + i * rpz + j * rpy : lp + i * lpz + j * lpy;
            edge = *reinterpret_cast<const P2*>(src);
        }
    } else {
#pragma unroll
        for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
            for (int j = 0; j < DR_WY; ++j)
                if (DR_NEED[i][j][0] || DR_NEED[i][j][DR_WK - 1]) {
                    const T* src = pc + i * PZ + j * PY;
                    src = first ? lp + i * lpz + j * lpy : src;
                    src = last ? rp + i * rpz + j * rpy : src;
                    beyond[i][j] = *reinterpret_cast<const P2*>(src);
                }
    }
    P2 ov[DR_NOTHA][DR_RZ][DR_RY];
#pragma unroll
    for (int j = 0; j < DR_NOTH; ++j) {
        const T* const ot = a.oth[j][p.t] + (lz0 * PZ + ly0 * PY + lx);
#pragma unroll
        for (int rz = 0; rz < DR_RZ; ++rz)
#pragma unroll
            for (int ry = 0; ry < DR_RY; ++ry)
                ov[j][rz][ry] = *reinterpret_cast<const P2*>(ot + rz * PZ + ry * PY);
    }
#pragma unroll
    for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
        for (int j = 0; j < DR_WY; ++j) {
            const int r = (i - DR_BI0) * DR_BNJ + (j - DR_BJ0);   // row of the gathered block
            if (DR_NEED[i][j][0]) {
                P2 sh, far = beyond[i][j];
                sh[0] = from_prev_lane(win[i][j][DR_HK][0]);
                sh[1] = from_prev_lane(win[i][j][DR_HK][1]);
                if (DR_EDGE_GATHER) {
                    far[0] = from_lane(edge[0], 2 * r);
                    far[1] = from_lane(edge[1], 2 * r);
                }
                win[i][j][0] = first ? far : sh;
            }
            if (DR_NEED[i][j][DR_WK - 1]) {
                P2 sh, far = beyond[i][j];
                sh[0] = from_next_lane(win[i][j][DR_HK][0]);
                sh[1] = from_next_lane(win[i][j][DR_HK][1]);
                if (DR_EDGE_GATHER) {
                    far[0] = from_lane(edge[0], 2 * r + 1);
                    far[1] = from_lane(edge[1], 2 * r + 1);
                }
                win[i][j][DR_WK - 1] = last ? far : sh;
            }
        }
    T* const out_tile = a.dst[p.t];
    T acc = (T)0;
#pragma unroll
    for (int rz = 0; rz < DR_RZ; ++rz)
#pragma unroll
        for (int ry = 0; ry < DR_RY; ++ry) {
            P2 res;
            bool in_e[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                T l[NLA], o[NOA];
#pragma unroll
                for (int q = 0; q < NL; ++q) {
                    const int xx = e + DR_SHIFT[q][2];
                    l[q] = DR_OTHER[q] >= 0
                               ? ov[DR_OTHER[q] >= 0 ? DR_OTHER[q] : 0][rz][ry][e]
                               : win[rz + DR_H0 + DR_SHIFT[q][0]][ry + DR_H1 + DR_SHIFT[q][1]]
                                    [DR_HK + floordiv2(xx)][xx & 1];
                }
                group_eval(l, s, o);
                const int gx = p.tx0 + lx + e;
                in_e[e] = gx >= a.rs[2] && gx < a.re[2];
                res[e] = (DR_MASKED || in_e[e]) ? o[0] : win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                if (RED) {
                    T d = o[0] - win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                    d = in_e[e] ? d : (T)0;
                    if (RED == 1) acc = acc + d * d;
                    else { d = d < (T)0 ? (T)0 - d : d; acc = d > acc ? d : acc; }
                }
            }
            P2* out = reinterpret_cast<P2*>(out_tile + ((lz0 + rz) * PZ + (ly0 + ry) * PY + lx));
            store_pair<NTS>(out, res, in_e[0], in_e[1]);
        }
    if (RED) {
        acc = wave_combine<RED == 2, T>(acc);
        if (lane == 0) *my_slot = acc;
    }
}

// Everything the fast path leaves (or, with skip_fast = 0, everything): windows that touch
// neighbour tiles in y or z, partial tiles, rows and planes outside the assigned region,
// workgroups narrower than a wavefront. With a list, workgroup i does position list[i] of the
// order (the host lists the workgroups on the y and z faces of the tiles); without, all of them.
template <bool NTS, int RED>
__device__ __forceinline__ void direct_rest(const DirectArgs& a, const T* s, int skip_fast,
                                            const int* list, int first_block) {
    T* const my_slot = RED ? a.slots + ((size_t)blockIdx.x * 4 + (threadIdx.x >> 6)) : nullptr;
    const int me = (int)blockIdx.x - first_block;   // this workgroup's number among those doing the rest
    const Place p = locate(a, list ? list[me] : xcd_order(a, me));
    const int t = p.t, t0 = p.t0, t1 = p.t1, t2 = p.t2;
    const int tz0 = p.tz0, ty0 = p.ty0, tx0 = p.tx0, w0 = p.w0, w1 = p.w1, w2 = p.w2;
    // extents of the next tiles (the previous ones are always full)
    const int w0n = min(a.tile, a.shape[0] - tz0 - a.tile), w1n = min(a.tile, a.shape[1] - ty0 - a.tile),
              w2n = min(a.tile, a.shape[2] - tx0 - a.tile);
    const int lz0 = p.bz * DR_RZ;
    const int tid = (int)threadIdx.x;
    if (lz0 >= w0) {                                   // the whole workgroup
        if (RED && (tid & 63) == 0) *my_slot = (T)0;
        return;
    }
    if (skip_fast && DR_WAVE_ROWS) {
        const int wv = wave_uniform(tid >> 6);
        const int wy0 = (p.by * DR_TY + (wv * 64) / DR_TX) * DR_RY;
        const int wx0 = (p.bx * DR_TX + (wv * 64) % DR_TX) * 2;
        if (wy0 < w1 && wx0 < w2 && wave_is_fast(a, p, lz0, wy0, wx0)) {   // the whole wavefront
            if (RED && (tid & 63) == 0) *my_slot = (T)0;
            return;
        }
    }
    int lx = (p.bx * DR_TX + tid % DR_TX) * 2;
    int ly0 = (p.by * DR_TY + tid / DR_TX) * DR_RY;
    // Lanes beyond the tile have nothing to do. A plain sweep lets them go; a reducing one keeps
    // every lane of the wavefront to the end (the lane exchange of the final sum needs all 64):
    // such a lane works on the tile's first pair instead, stores nothing and adds nothing.
    const bool idle = lx >= w2 || ly0 >= w1;
    if (!RED && idle) return;
    if (idle) { lx = 0; ly0 = 0; }

    // ---- the 27 tile pointers around this tile (uniform); missing neighbours fall back to own ----
    const T* nb[3][3][3];
#pragma unroll
    for (int dz = -1; dz <= 1; ++dz)
#pragma unroll
        for (int dy = -1; dy <= 1; ++dy)
#pragma unroll
            for (int dx = -1; dx <= 1; ++dx) {
                const int z = t0 + dz, y = t1 + dy, x = t2 + dx;
                const bool ok = z >= 0 && z < a.grid[0] && y >= 0 && y < a.grid[1] && x >= 0 &&
                                x < a.grid[2];
                const int ti = ok ? (z * a.grid[1] + y) * a.grid[2] + x : t;
                nb[dz + 1][dy + 1][dx + 1] = a.cur[ti];
            }
    T* const out_tile = a.dst[t];

    // A window entry in a halo position (before/after the lane's own rows, planes, column pair)
    // can leave the tile in exactly that direction; entries in own positions never do, because
    // the tile edge is a multiple of the rows and planes a lane owns. So the tile of an entry is
    // one of 8 pointers whose table indices are compile-time constants, chosen with selects.
    // ---- column resolution per pair offset k (per lane) ----
    bool xc[DR_WK];                        // entry lies in the x-neighbour
    int xl[DR_WK], xw[DR_WK];              // local column, row length of the tile read
#pragma unroll
    for (int k = 0; k < DR_WK; ++k) {
        int c = lx + 2 * (k - DR_HK);
        bool cross = false;
        int wd = w2;
        if (k < DR_HK && c < 0) {
            if (t2 > 0) { cross = true; c += a.tile; wd = a.tile; } else c = 0;
        } else if (k > DR_HK && c >= w2) {
            if (t2 + 1 < a.grid[2]) { cross = true; c = min(c - w2, w2n - 2); wd = w2n; } else c = w2 - 2;
        }
        xc[k] = cross; xl[k] = c; xw[k] = wd;
    }
    // ---- row resolution per window row (per lane) ----
    bool yc[DR_WY];
    int yl[DR_WY], yh[DR_WY];
#pragma unroll
    for (int j = 0; j < DR_WY; ++j) {
        int c = ly0 + j - DR_H1;
        bool cross = false;
        int ht = w1;
        if (j < DR_H1 && c < 0) {
            if (t1 > 0) { cross = true; c += a.tile; ht = a.tile; } else c = 0;
        } else if (c >= w1) {
            if (j >= DR_H1 + DR_RY && t1 + 1 < a.grid[1]) { cross = true; c = min(c - w1, w1n - 1); ht = w1n; }
            else c = w1 - 1;
        }
        yc[j] = cross; yl[j] = c; yh[j] = ht;
    }

    // ---- issue every load of the window ----
    P2 win[DR_WZ][DR_WY][DR_WK];
#pragma unroll
    for (int i = 0; i < DR_WZ; ++i) {
        int cz = lz0 + i - DR_H0;      // uniform
        bool zc = false;
        if (i < DR_H0 && cz < 0) {
            if (t0 > 0) { zc = true; cz += a.tile; } else cz = 0;
        } else if (cz >= w0) {
            if (i >= DR_H0 + DR_RZ && t0 + 1 < a.grid[0]) { zc = true; cz = min(cz - w0, w0n - 1); }
            else cz = w0 - 1;
        }
        constexpr int one = 1;
        const int DZ = i < DR_H0 ? -1 : (i >= DR_H0 + DR_RZ ? 1 : 0);
#pragma unroll
        for (int j = 0; j < DR_WY; ++j) {
            const int DY = j < DR_H1 ? -1 : (j >= DR_H1 + DR_RY ? 1 : 0);
#pragma unroll
            for (int k = 0; k < DR_WK; ++k)
                if (DR_NEED[i][j][k]) {
                    const int DX = k < DR_HK ? -1 : (k > DR_HK ? 1 : 0);
                    // DZ, DY, DX are constants after unrolling: every nb[][][] index below is static
                    const T* q00 = zc ? nb[one + DZ][one][one] : nb[one][one][one];
                    const T* q01 = zc ? nb[one + DZ][one][one + DX] : nb[one][one][one + DX];
                    const T* q10 = zc ? nb[one + DZ][one + DY][one] : nb[one][one + DY][one];
                    const T* q11 = zc ? nb[one + DZ][one + DY][one + DX] : nb[one][one + DY][one + DX];
                    const T* r0 = xc[k] ? q01 : q00;
                    const T* r1 = xc[k] ? q11 : q10;
                    const T* base = yc[j] ? r1 : r0;
                    // row and plane strides of the tile read: its own extents, or the common pitches
                    const int rowlen = a.py ? a.py : xw[k];
                    const int planelen = a.py ? a.pz : yh[j] * xw[k];
                    const int off = cz * planelen + yl[j] * rowlen + xl[k];
                    win[i][j][k] = *reinterpret_cast<const P2*>(base + off);
                }
        }
    }

    // ---- the other arrays, at the lane's own rows and planes (clamped into the tile: what a
    // row or plane beyond the tile would read is never used) ----
    const int OPY = a.py ? a.py : w2, OPZ = a.py ? a.pz : w1 * w2;   // strides of this tile
    P2 ov[DR_NOTHA][DR_RZ][DR_RY];
#pragma unroll
    for (int j = 0; j < DR_NOTH; ++j) {
        const T* const ot = a.oth[j][t];
#pragma unroll
        for (int rz = 0; rz < DR_RZ; ++rz)
#pragma unroll
            for (int ry = 0; ry < DR_RY; ++ry)
                ov[j][rz][ry] = *reinterpret_cast<const P2*>(
                    ot + (min(lz0 + rz, w0 - 1) * OPZ + min(ly0 + ry, w1 - 1) * OPY + lx));
    }

    // ---- evaluate and store ----
    T acc = (T)0;
#pragma unroll
    for (int rz = 0; rz < DR_RZ; ++rz) {
        const int lz = lz0 + rz;
        if (lz < w0) {
            const int gz = tz0 + lz;
            const bool zin = gz >= a.rs[0] && gz < a.re[0];
#pragma unroll
            for (int ry = 0; ry < DR_RY; ++ry) {
                const int ly = ly0 + ry;
                if (ly < w1) {
                    const int gy = ty0 + ly;
                    const bool yin = zin && gy >= a.rs[1] && gy < a.re[1];
                    P2 res;
                    bool in_e[2];
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const int gx = tx0 + lx + e;
                        // evaluated for every element and selected afterwards: window entries an
                        // unassigned element would read exist (clamped), and straight-line code
                        // keeps all loads ahead of the arithmetic
                        const bool in_region = yin && gx >= a.rs[2] && gx < a.re[2];
                        T l[NLA], o[NOA];
#pragma unroll
                        for (int q = 0; q < NL; ++q) {
                            const int xx = e + DR_SHIFT[q][2];
                            l[q] = DR_OTHER[q] >= 0
                                       ? ov[DR_OTHER[q] >= 0 ? DR_OTHER[q] : 0][rz][ry][e]
                                       : win[rz + DR_H0 + DR_SHIFT[q][0]][ry + DR_H1 + DR_SHIFT[q][1]]
                                            [DR_HK + floordiv2(xx)][xx & 1];
                        }
                        group_eval(l, s, o);
                        in_e[e] = in_region;
                        res[e] = (DR_MASKED || in_region) ? o[0] : win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                        if (RED) {
                            T d = o[0] - win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                            d = (in_region && !idle) ? d : (T)0;
                            if (RED == 1) acc = acc + d * d;
                            else { d = d < (T)0 ? (T)0 - d : d; acc = d > acc ? d : acc; }
                        }
                    }
                    if (!RED || !idle) {
                        P2* out = reinterpret_cast<P2*>(out_tile + (lz * OPZ + ly * OPY + lx));
                        store_pair<NTS>(out, res, in_e[0], in_e[1]);
                    }
                }
            }
        }
    }
    if (RED) {
        acc = wave_combine<RED == 2, T>(acc);
        if ((tid & 63) == 0) *my_slot = acc;
    }
}

// ---- the whole array as one row-major block ----
// When every tile of every array of the launch is a view into one block (an executor that keeps all
// partitions of an array on one device may store it that way), tiles need no pointers and no
// neighbour logic: a wavefront works on 128 columns of DR_RY rows in DR_RZ planes of the ARRAY,
// window coordinates are clamped into the array (what a clamped entry holds is only ever used by
// elements outside the assigned region, which keep their old value), and the only faces left are
// the array's own. Workgroups are ordered in blocks of ob[] workgroups (x fastest inside a block,
// then y, then z) and the 8 XCDs get contiguous runs of that order, so that the planes and rows a
// block re-reads stay in one L2.
struct FlatArgs {
    const T* cur;          // current contents of the window array
    T* dst;                // new contents of the assigned array
    const T* oth[4];       // other arrays read at the element's own position
    int shape[3];          // array extents (leading dims padded with 1)
    int rs[3], re[3];      // assigned region
    int py, pz;            // elements between rows and between planes
    int nb[3];             // workgroups along z, y, x
    int ob[3];             // ordering block, in workgroups along z, y, x
    int nblocks8;          // launched workgroups / 8 (the launch is padded to a multiple of 8)
    FDiv per_block;        // workgroups per ordering block
    FDiv gb1, gb2;         // ordering blocks along y and x
    FDiv obx, oby;         // = ob[2], ob[1]
    T* slots;              // reducing launches: one partial per launched wavefront
    int sub8;              // ragged grids: workgroups per ordering block / 8, else 0
    FDiv fsub;             // = sub8
    int lat[3];            // step - 1 of every region per dimension (0: unit step, 1: every other point)
    int nroots;            // 1, or 2: a second assigned lattice [rs2, re2) with the same steps
    int rs2[3], re2[3];
    int tail;              // 1 or 2: columns beyond the last wavefront of a row, copied by its last lane
    int unused;
};

// Rows of odd length, odd pitches or a block that does not start on a 16-byte boundary (UA): pairs
// are then only element-aligned. They still move as one access each (the hardware takes 128-bit
// accesses at any 4-byte boundary); the pair that holds the last element of an odd row is read one
// element to the left and shifted, and written as a single element, so that nothing outside the row
// is touched.
typedef P2 P2A __attribute__((aligned(sizeof(T))));
template <bool UA>
__device__ __forceinline__ P2 load_pair(const T* row, int c, int S2) {
    if (!UA) return *reinterpret_cast<const P2*>(row + c);
    const bool whole = c + 1 < S2;
    const P2 u = *reinterpret_cast<const P2A*>(row + (whole ? c : S2 - 2));
    return whole ? u : (P2){u[1], u[1]};
}
template <bool NTS, bool UA>
__device__ __forceinline__ void store_pair_flat(T* out, P2 v, bool in0, bool in1, bool has1) {
    if (!UA) {
        store_pair<NTS>(reinterpret_cast<P2*>(out), v, in0, in1);
        return;
    }
    const bool w0 = !DR_MASKED || in0, w1 = has1 && (!DR_MASKED || in1);
    if (w0 && w1) {
        if (NTS) __builtin_nontemporal_store(v, reinterpret_cast<P2A*>(out)); else *reinterpret_cast<P2A*>(out) = v;
    } else {
        if (w0) out[0] = v[0];
        if (w1) out[1] = v[1];
    }
}

// RED as above.
template <bool NTS, int RED, bool UA>
__device__ __forceinline__ void direct_flat(const FlatArgs& a, const T* s) {
    T* const my_slot = RED ? a.slots + ((size_t)blockIdx.x * 4 + (threadIdx.x >> 6)) : nullptr;
    int blk = (int)blockIdx.x;
    if (a.sub8) {
        // Ragged grids pad their last ordering blocks with workgroups that do nothing, so whole
        // blocks per XCD would leave most of the work to a few XCDs: here every ordering block is
        // cut into eight contiguous runs, one per XCD, and all XCDs walk the blocks together.
        const int xcd = blk & 7, j = blk >> 3;
        const int gq = fdiv(j, a.fsub);
        blk = gq * (int)a.per_block.d + xcd * a.sub8 + (j - gq * a.sub8);
    } else if (a.nblocks8) {
        blk = (blk & 7) * a.nblocks8 + (blk >> 3);
    }
    const int g = fdiv(blk, a.per_block), w = blk - g * (int)a.per_block.d;
    const int gq = fdiv(g, a.gb2), g2 = g - gq * (int)a.gb2.d;
    const int g0 = fdiv(gq, a.gb1), g1 = gq - g0 * (int)a.gb1.d;
    const int wq = fdiv(w, a.obx), wx = w - wq * (int)a.obx.d;
    const int wz = fdiv(wq, a.oby), wy = wq - wz * (int)a.oby.d;
    const int bz = g0 * a.ob[0] + wz, by = g1 * a.ob[1] + wy, bx = g2 * a.ob[2] + wx;
    if (bz >= a.nb[0] || by >= a.nb[1] || bx >= a.nb[2]) {          // padding of a ragged block
        if (RED && (threadIdx.x & 63) == 0) *my_slot = (T)0;
        return;
    }
    const int tid = (int)threadIdx.x;
    const int wv = wave_uniform(tid >> 6);
    const int lane = tid & 63;
    const int S0 = a.shape[0], S1 = a.shape[1], S2 = a.shape[2];
    const int z0 = bz * DR_RZ, y0 = (by * 4 + wv) * DR_RY, x0 = bx * 128;
    if (y0 >= S1) {                                                  // wavefront-uniform
        if (RED && lane == 0) *my_slot = (T)0;
        return;
    }
    const int PY = a.py, PZ = a.pz;
    const int lx = x0 + 2 * lane;
    const bool live = lx < S2;                  // a live lane owns a pair, or the last element of an odd row
    const bool live1 = lx + 1 < S2;
    const int lastc = (S2 - 1) & ~1;            // column of the last pair (even S2) or last element (odd)
    const int cx = min(lx, lastc);              // idle lanes re-read the end of the row
    const bool first = lane == 0, last = lane == 63;
    // clamped planes and rows of the window (wavefront-uniform)
    int zo[DR_WZ], yo[DR_WY];
#pragma unroll
    for (int i = 0; i < DR_WZ; ++i) zo[i] = min(max(z0 - DR_H0 + i, 0), S0 - 1) * PZ;
#pragma unroll
    for (int j = 0; j < DR_WY; ++j) yo[j] = min(max(y0 - DR_H1 + j, 0), S1 - 1) * PY;
    const T* const cur = a.cur;

    // All loads first: the centre pairs, then the pairs beyond the two ends of the wavefront.
    P2 win[DR_WZ][DR_WY][DR_WK];
    P2 beyond[DR_WZ][DR_WY];
#pragma unroll
    for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
        for (int j = 0; j < DR_WY; ++j)
            if (DR_NEED[i][j][0] || DR_NEED[i][j][DR_HK] || DR_NEED[i][j][DR_WK - 1])
                win[i][j][DR_HK] = load_pair<UA>(cur + (zo[i] + yo[j]), cx, S2);
    const int xl = max(x0 - 2, 0), xr = min(x0 + 128, lastc);    // columns of the two far pairs
    P2 edge = (P2){(T)0, (T)0};
    if (DR_HK == 1) {
        if (DR_EDGE_GATHER) {
            // one load for all of them: lane 2r holds the pair left of row r of the block of rows
            // that need one, lane 2r + 1 the pair right of it
            if (lane < 2 * DR_NB) {
                const int r = lane >> 1, i = DR_BI0 + r / DR_BNJ, j = DR_BJ0 + r % DR_BNJ;
                const int zz = min(max(z0 - DR_H0 + i, 0), S0 - 1), yy = min(max(y0 - DR_H1 + j, 0), S1 - 1);
                edge = load_pair<UA>(cur + (zz * PZ + yy * PY), (lane & 1) ? xr : xl, S2);
            }
        } else {
#pragma unroll
            for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
                for (int j = 0; j < DR_WY; ++j)
                    if (DR_NEED[i][j][0] || DR_NEED[i][j][DR_WK - 1]) {
                        const int c = first ? xl : (last ? xr : cx);
                        beyond[i][j] = load_pair<UA>(cur + (zo[i] + yo[j]), c, S2);
                    }
        }
    }
    P2 ov[DR_NOTHA][DR_RZ][DR_RY];
    if (!DR_OSH) {
#pragma unroll
        for (int j = 0; j < DR_NOTH; ++j)
#pragma unroll
            for (int rz = 0; rz < DR_RZ; ++rz)
#pragma unroll
                for (int ry = 0; ry < DR_RY; ++ry)
                    ov[j][rz][ry] = load_pair<UA>(a.oth[j] + (zo[rz + DR_H0] + yo[ry + DR_H1]), cx, S2);
    }
    // Other arrays read at shifted positions: a window per array, the same clamped rows and planes,
    // the left and right pairs by lane exchange, the pairs beyond the wavefront's ends by one more
    // load per row in which the first and the last lane fetch theirs.
    P2 wo[DR_NOTHA][DR_WZ][DR_WY][DR_WK];      // unused (and gone from the code) unless DR_OSH
    if (DR_OSH) {
#pragma unroll
        for (int j = 0; j < DR_NOTH; ++j)
#pragma unroll
            for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
                for (int jj = 0; jj < DR_WY; ++jj) {
                    const bool side0 = DR_HK == 1 && DR_ONEED[j][i][jj][0];
                    const bool side1 = DR_HK == 1 && DR_ONEED[j][i][jj][DR_WK - 1];
                    if (DR_ONEED[j][i][jj][DR_HK] || side0 || side1)
                        wo[j][i][jj][DR_HK] =
                            load_pair<UA>(a.oth[j] + (zo[i] + yo[jj]), cx, S2);
                    if (side0 || side1) {
                        const P2 mid = wo[j][i][jj][DR_HK];
                        const P2 far = load_pair<UA>(a.oth[j] + (zo[i] + yo[jj]), first ? xl : (last ? xr : cx), S2);
                        if (side0) {
                            P2 sh;
                            sh[0] = from_prev_lane(mid[0]);
                            sh[1] = from_prev_lane(mid[1]);
                            wo[j][i][jj][0] = first ? far : sh;
                        }
                        if (side1) {
                            P2 sh;
                            sh[0] = from_next_lane(mid[0]);
                            sh[1] = from_next_lane(mid[1]);
                            wo[j][i][jj][DR_WK - 1] = last ? far : sh;
                        }
                    }
                }
    }
    if (DR_HK == 1) {
#pragma unroll
        for (int i = 0; i < DR_WZ; ++i)
#pragma unroll
            for (int j = 0; j < DR_WY; ++j) {
                const int r = (i - DR_BI0) * DR_BNJ + (j - DR_BJ0);   // row of the gathered block
                if (DR_NEED[i][j][0]) {
                    P2 sh, far = beyond[i][j];
                    sh[0] = from_prev_lane(win[i][j][DR_HK][0]);
                    sh[1] = from_prev_lane(win[i][j][DR_HK][1]);
                    if (DR_EDGE_GATHER) {
                        far[0] = from_lane(edge[0], 2 * r);
                        far[1] = from_lane(edge[1], 2 * r);
                    }
                    win[i][j][0] = first ? far : sh;
                }
                if (DR_NEED[i][j][DR_WK - 1]) {
                    P2 sh, far = beyond[i][j];
                    sh[0] = from_next_lane(win[i][j][DR_HK][0]);
                    sh[1] = from_next_lane(win[i][j][DR_HK][1]);
                    if (DR_EDGE_GATHER) {
                        far[0] = from_lane(edge[0], 2 * r + 1);
                        far[1] = from_lane(edge[1], 2 * r + 1);
                    }
                    win[i][j][DR_WK - 1] = last ? far : sh;
                }
            }
    }
    T* const dst = a.dst;
    // A sweep in place (a lattice whose shifted reads never meet an assigned point) leaves rows
    // without assigned points alone; one into a second buffer writes every element of it.
    const bool inplace = a.cur == a.dst;
    T acc = (T)0;
#pragma unroll
    for (int rz = 0; rz < DR_RZ; ++rz) {
        const int z = z0 + rz;
        const bool zin = z >= a.rs[0] && z < a.re[0] && ((z - a.rs[0]) & a.lat[0]) == 0;
        const bool zin2 = DR_NROOTS > 1 && a.nroots > 1 && z >= a.rs2[0] && z < a.re2[0] && ((z - a.rs2[0]) & a.lat[0]) == 0;
#pragma unroll
        for (int ry = 0; ry < DR_RY; ++ry) {
            const int y = y0 + ry;
            const bool yin = zin && y >= a.rs[1] && y < a.re[1] && ((y - a.rs[1]) & a.lat[1]) == 0;
            const bool yin2 = zin2 && y >= a.rs2[1] && y < a.re2[1] && ((y - a.rs2[1]) & a.lat[1]) == 0;
            P2 res;
            bool in_e[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                T l[NLA], o[NOA];
#pragma unroll
                for (int q = 0; q < NL; ++q) {
                    const int xx = e + DR_SHIFT[q][2];
                    const int oj = DR_OTHER[q] >= 0 ? DR_OTHER[q] : 0;
                    l[q] = DR_OTHER[q] >= 0
                               ? (DR_OSH ? wo[oj][rz + DR_H0 + DR_SHIFT[q][0]][ry + DR_H1 + DR_SHIFT[q][1]]
                                             [DR_HK + floordiv2(xx)][xx & 1]
                                         : ov[oj][rz][ry][e])
                               : win[rz + DR_H0 + DR_SHIFT[q][0]][ry + DR_H1 + DR_SHIFT[q][1]]
                                    [DR_HK + floordiv2(xx)][xx & 1];
                }
                group_eval(l, s, o);
                T second = o[0];
                if (DR_NROOTS > 1) {
                    // the second root reads its operands at its own offsets (a load both roots use
                    // sits at another offset from each lattice)
                    T l2[NLA], o2[NOA];
#pragma unroll
                    for (int q = 0; q < NL; ++q) {
                        const int xx = e + DR_SHIFT2[q][2];
                        l2[q] = DR_OTHER[q] >= 0
                                    ? ov[DR_OTHER[q] >= 0 ? DR_OTHER[q] : 0][rz][ry][e]
                                    : win[rz + DR_H0 + DR_SHIFT2[q][0]][ry + DR_H1 + DR_SHIFT2[q][1]]
                                         [DR_HK + floordiv2(xx)][xx & 1];
                    }
                    group_eval(l2, s, o2);
                    second = o2[NO > 1 ? 1 : 0];
                }
                const int gx = lx + e;
                const bool in1 = yin && gx >= a.rs[2] && gx < a.re[2] && ((gx - a.rs[2]) & a.lat[2]) == 0;
                const bool in2 = yin2 && gx >= a.rs2[2] && gx < a.re2[2] && ((gx - a.rs2[2]) & a.lat[2]) == 0;
                in_e[e] = in1 || in2;
                const T mine = in2 ? second : o[0];
                res[e] = (DR_MASKED || in_e[e]) ? mine : win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                if (RED) {
                    // assigned elements of live lanes only (rows and planes beyond the array are
                    // never assigned: the region lies inside it)
                    T d = o[0] - win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                    d = (in_e[e] && live) ? d : (T)0;
                    if (RED == 1) acc = acc + d * d;
                    else { d = d < (T)0 ? (T)0 - d : d; acc = d > acc ? d : acc; }
                }
            }
            // rows and planes beyond the array (a ragged last workgroup) and idle lanes store nothing
            if (live && z < S0 && y < S1 && (!inplace || yin || yin2))
                store_pair_flat<NTS, UA>(dst + (z * PZ + y * PY + lx), res, in_e[0], in_e[1], live1);
            // An array of 128 k + 1 or 128 k + 2 columns whose last columns no statement assigns
            // (the boundary of a 2^k + 1 grid) launches k wavefronts per row: the last lane of the
            // last one holds those columns as its right-hand neighbours and copies them over.
            if (DR_TAIL_OK && a.tail && last && bx == a.nb[2] - 1 && !inplace && z < S0 && y < S1) {
                const P2 far = win[rz + DR_H0][ry + DR_H1][DR_WK - 1];
                T* const beyond_row = dst + (z * PZ + y * PY + x0 + 128);
                beyond_row[0] = far[0];
                if (a.tail > 1) beyond_row[1] = far[1];
            }
        }
    }
    if (RED) {
        acc = wave_combine<RED == 2, T>(acc);
        if (lane == 0) *my_slot = acc;
    }
}
#if DR_RED
// The reducing forms only (built on demand under a variant name of their own).
#define FLAT_RED_ENTRY(NAME, NTS, RED, UA)                                                        \
extern "C" __global__ __launch_bounds__(256) void NAME(FlatArgs a, Scal sc) {                     \
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);                                                                \
    direct_flat<NTS, RED, UA>(a, s);                                                              \
}
FLAT_RED_ENTRY(grp_direct_flat_red1, false, 1, false)
FLAT_RED_ENTRY(grp_direct_flat_red1_nts, true, 1, false)
FLAT_RED_ENTRY(grp_direct_flat_red2, false, 2, false)
FLAT_RED_ENTRY(grp_direct_flat_red2_nts, true, 2, false)
FLAT_RED_ENTRY(grp_direct_flatu_red1, false, 1, true)
FLAT_RED_ENTRY(grp_direct_flatu_red1_nts, true, 1, true)
FLAT_RED_ENTRY(grp_direct_flatu_red2, false, 2, true)
FLAT_RED_ENTRY(grp_direct_flatu_red2_nts, true, 2, true)
// Tiles with buffers of their own: the lean part and the listed face workgroups in one launch.
#define BOTH_RED_ENTRY(NAME, NTS, RED)                                                            \
extern "C" __global__ __launch_bounds__(256) void NAME(DirectArgs a, Scal sc, const int* list) {  \
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);                                                                \
    if ((int)blockIdx.x < a.nblocks) direct_fast<NTS, RED>(a, s);                                 \
    else direct_rest<NTS, RED>(a, s, 1, list, a.nblocks);                                         \
}
BOTH_RED_ENTRY(grp_direct_both_red1, false, 1)
BOTH_RED_ENTRY(grp_direct_both_red1_nts, true, 1)
BOTH_RED_ENTRY(grp_direct_both_red2, false, 2)
BOTH_RED_ENTRY(grp_direct_both_red2_nts, true, 2)
#else
extern "C" __global__ __launch_bounds__(256) void grp_direct_flat(FlatArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_flat<false, 0, false>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_flat_nts(FlatArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_flat<true, 0, false>(a, s);
}
// the same for blocks whose pairs are only element-aligned (odd rows or pitches)
extern "C" __global__ __launch_bounds__(256) void grp_direct_flatu(FlatArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_flat<false, 0, true>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_flatu_nts(FlatArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_flat<true, 0, true>(a, s);
}

// nts: the written stream is not read back soon, store it non-temporally.
extern "C" __global__ __launch_bounds__(256) void grp_direct_fast(DirectArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_fast<false, 0>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_fast_nts(DirectArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_fast<true, 0>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_rest(DirectArgs a, Scal sc, int skip_fast,
                                                                  const int* list) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_rest<false, 0>(a, s, skip_fast, list, 0);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_rest_nts(DirectArgs a, Scal sc, int skip_fast,
                                                                      const int* list) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    direct_rest<true, 0>(a, s, skip_fast, list, 0);
}
// Both in one launch: the first a.nblocks workgroups do the lean part, the ones after them what
// the lean part leaves (those on `list`, or all positions again when there is no list). One
// launch and no gap between the two, and the second part fills the tail of the first.
extern "C" __global__ __launch_bounds__(256) void grp_direct_both(DirectArgs a, Scal sc, const int* list) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    if ((int)blockIdx.x < a.nblocks) direct_fast<false, 0>(a, s);
    else direct_rest<false, 0>(a, s, 1, list, a.nblocks);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_both_nts(DirectArgs a, Scal sc, const int* list) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    if ((int)blockIdx.x < a.nblocks) direct_fast<true, 0>(a, s);
    else direct_rest<true, 0>(a, s, 1, list, a.nblocks);
}
#endif
)";
    return s.str();
}

} // namespace cnh
