// Register-window source for same-array unit-step stencils (the Jacobi-style SET_REGION groups).
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
    if (p.out_roots.size() != 1 || !p.out_is_set_region[0] || p.out_region[0].is_global) {
        err = "register-window stencil needs a single SET_REGION root";
        return -18;
    }
    if (p.dtype != CNH_F64 && p.dtype != CNH_I64) {
        err = "register-window stencil is built for 8-byte elements";
        return -18;
    }
    const cnh_region& ro = p.out_region[0];
    const int nd = p.ndims, pad = CNH_MAX_ND - nd;
    for (int d = 0; d < nd; ++d)
        if (ro.step[d] != 1) {
            err = "assigned region is strided";
            return -18;
        }
    if (p.load_leaf.empty()) {
        err = "no array operand";
        return -18;
    }
    sh.shifts.assign(p.load_leaf.size(), {0, 0, 0});
    for (size_t l = 0; l < p.load_leaf.size(); ++l) {
        const LeafUse& u = p.leaves[p.load_leaf[l]];
        if (u.name != p.out_target[0]) {
            err = "operand is not the assigned array";
            return -18;
        }
        if (!u.has_region) {
            err = "operand without a region";
            return -18;
        }
        for (int d = 0; d < nd; ++d) {
            if (u.region.step[d] != 1 ||
                u.region.stop[d] - u.region.start[d] != ro.stop[d] - ro.start[d]) {
                err = "operand region is strided or of a different extent";
                return -18;
            }
            int s = u.region.start[d] - ro.start[d];
            sh.shifts[l][pad + d] = s;
            sh.halo[pad + d] = std::max(sh.halo[pad + d], std::abs(s));
        }
    }
    for (int d = 0; d < 3; ++d)
        if (sh.halo[d] > 2) {
            err = "halo wider than 2";
            return -18;
        }
    // measured on MI355X: 8 rows per lane for rank 2; 2 rows x 4 planes per lane for rank 3
    sh.tx = 64;
    sh.ry = nd == 3 ? 2 : 8;
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
            at(rz + H0, ry + H1, HK) = 1; // the element itself (kept outside the assigned region)
            for (int e = 0; e < 2; ++e)
                for (const auto& s : sh.shifts)
                    at(rz + H0 + s[0], ry + H1 + s[1], HK + floordiv2(e + s[2])) = 1;
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
    s << R"(
struct DirectArgs {
    const T* const* cur;   // tile table of the current contents (row-major tile grid)
    T* const* dst;         // tile table of the new contents
    int tile;              // tile edge
    int shape[3];          // array extents (leading dims padded with 1)
    int grid[3];           // tiles per dimension
    int rs[3], re[3];      // assigned region
    int tb[3];             // workgroups per tile along z, y, x
    int nblocks;
};
typedef T P2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int xcd_remap(int b, int n) {
    return (n % 8 == 0) ? (b % 8) * (n / 8) + b / 8 : b;
}
__device__ __forceinline__ int floordiv2(int v) { return v >= 0 ? v / 2 : -((-v + 1) / 2); }

template <bool NTS>
__device__ __forceinline__ void direct_run(const DirectArgs& a, const T* s) {
    // ---- which tile, which patch of it (all workgroup-uniform) ----
    const int per_tile = a.tb[0] * a.tb[1] * a.tb[2];
    const int blk = xcd_remap((int)blockIdx.x, a.nblocks);
    const int t = blk / per_tile, w = blk - t * per_tile;
    const int t2 = t % a.grid[2], t1 = (t / a.grid[2]) % a.grid[1], t0 = t / (a.grid[2] * a.grid[1]);
    const int bx = w % a.tb[2], by = (w / a.tb[2]) % a.tb[1], bz = w / (a.tb[2] * a.tb[1]);
    const int tz0 = t0 * a.tile, ty0 = t1 * a.tile, tx0 = t2 * a.tile;   // tile origin
    const int w0 = min(a.tile, a.shape[0] - tz0), w1 = min(a.tile, a.shape[1] - ty0),
              w2 = min(a.tile, a.shape[2] - tx0);                         // tile extents
    // extents of the next tiles (the previous ones are always full)
    const int w0n = min(a.tile, a.shape[0] - tz0 - a.tile), w1n = min(a.tile, a.shape[1] - ty0 - a.tile),
              w2n = min(a.tile, a.shape[2] - tx0 - a.tile);
    const int lz0 = bz * DR_RZ;
    if (lz0 >= w0) return;
    const int tid = (int)threadIdx.x;
    const int lx = (bx * DR_TX + tid % DR_TX) * 2;
    const int ly0 = (by * DR_TY + tid / DR_TX) * DR_RY;
    if (lx >= w2 || ly0 >= w1) return;

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
                    const int off = (cz * yh[j] + yl[j]) * xw[k] + xl[k];
                    win[i][j][k] = *reinterpret_cast<const P2*>(base + off);
                }
        }
    }

    // ---- evaluate and store ----
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
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const int gx = tx0 + lx + e;
                        if (yin && gx >= a.rs[2] && gx < a.re[2]) {
                            T l[NLA], o[NOA];
#pragma unroll
                            for (int q = 0; q < NL; ++q) {
                                const int xx = e + DR_SHIFT[q][2];
                                l[q] = win[rz + DR_H0 + DR_SHIFT[q][0]][ry + DR_H1 + DR_SHIFT[q][1]]
                                          [DR_HK + floordiv2(xx)][xx & 1];
                            }
                            group_eval(l, s, o);
                            res[e] = o[0];
                        } else {
                            res[e] = win[rz + DR_H0][ry + DR_H1][DR_HK][e];
                        }
                    }
                    P2* out = reinterpret_cast<P2*>(out_tile + ((lz * w1 + ly) * w2 + lx));
                    if (NTS) __builtin_nontemporal_store(res, out); else *out = res;
                }
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(256) void grp_direct(DirectArgs a, Scal sc) {
    T s[NSA]; load_scalars(sc, s);
    direct_run<false>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_direct_nts(DirectArgs a, Scal sc) {
    T s[NSA]; load_scalars(sc, s);
    direct_run<true>(a, s);
}
)";
    return s.str();
}

} // namespace cnh
