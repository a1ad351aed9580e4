// Sliding-window source for same-array unit-step stencils (the Jacobi-style SET_REGION groups).
//
// One workgroup owns a column of the array: a patch of the trailing dimensions, marched along the
// leading dimension. Planes are staged once through an LDS ring of 2*H0+2 slots with 128-bit
// loads, every shifted operand is then an LDS read, and the new plane is written with 128-bit
// stores into the destination tiles. Loads run PD planes ahead of the plane being computed and
// wait in registers, so several planes per workgroup are in flight towards HBM; the one spare
// ring slot lets a single barrier per plane separate the writer of plane z+H0+1 from the readers
// of plane z. Neighbour tiles are addressed in place through the tile table, so no halo is
// packed, sent or unpacked.
#include "codegen.h"

#include <algorithm>
#include <sstream>

namespace cnh {

int slide_shape(const GroupProgram& p, const SlideConfig& cfg, SlideShape& sh, std::string& err) {
    sh = SlideShape();
    sh.march2d = cfg.march2d != 0;
    if (p.ndims != 2 && p.ndims != 3) {
        err = "sliding window needs rank 2 or 3";
        return -18;
    }
    if (p.out_roots.size() != 1 || !p.out_is_set_region[0] || p.out_region[0].is_global) {
        err = "sliding window needs a single SET_REGION root";
        return -18;
    }
    if (p.dtype != CNH_F64 && p.dtype != CNH_I64) {
        err = "sliding window is built for 8-byte elements";
        return -18;
    }
    const cnh_region& ro = p.out_region[0];
    const int nd = p.ndims;
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
            sh.shifts[l][sh.kdim(nd, d)] = s;
            sh.halo[sh.kdim(nd, d)] = std::max(sh.halo[sh.kdim(nd, d)], std::abs(s));
        }
    }
    for (int d = 0; d < 3; ++d)
        if (sh.halo[d] > 2) {
            err = "halo wider than 2";
            return -18;
        }
    if (nd == 2 && sh.march2d) { // (y, x): a 1 x 512 strip marched down the rows
        sh.bx = 512;
        sh.ry = 1;
        sh.zc = 64;
        sh.pd = 4;
    } else if (nd == 2) { // one 32 x 128 patch per workgroup, no march
        sh.bx = 128;
        sh.ry = 8;
        sh.zc = 1;
        sh.pd = 1;
    } else { // (z, y, x): a 16 x 64 patch marched along z
        sh.bx = 64;
        sh.ry = 2;
        sh.zc = 32;
        sh.pd = 2;
    }
    if (cfg.bx > 0)
        sh.bx = cfg.bx;
    if (cfg.ry > 0)
        sh.ry = cfg.ry;
    if (cfg.zc > 0)
        sh.zc = cfg.zc;
    if (cfg.pd > 0)
        sh.pd = cfg.pd;
    if (sh.bx < 2 || sh.bx > 512 || (sh.bx & (sh.bx - 1))) {
        err = "bad sliding-window width";
        return -18;
    }
    sh.ty = 256 / (sh.bx / 2);
    if (sh.ry < 1 || sh.ry > 16 || sh.zc < 1 || sh.pd < 1 || sh.pd > 8 ||
        (sh.zc > 1 && sh.zc % sh.pd != 0) || (sh.zc == 1 && sh.pd != 1)) {
        err = "bad sliding-window geometry";
        return -18;
    }
    const int ring = sh.zc == 1 ? 1 : 2 * sh.halo[0] + 2;
    const int px = sh.bx + 2 * ((sh.halo[2] + 1) & ~1);
    const int py = sh.ty * sh.ry + 2 * sh.halo[1];
    if ((size_t)ring * py * px * 8 > 64 * 1024) {
        err = "sliding-window patch does not fit in LDS";
        return -18;
    }
    return 0;
}

std::string slide_source(const GroupProgram& p, const SlideConfig& cfg, std::string& err) {
    SlideShape sh;
    if (slide_shape(p, cfg, sh, err))
        return std::string();
    std::string pre;
    if (emit_variant_source(p, "prelude", pre, err) != 0)
        return std::string();
    std::ostringstream s;
    s << pre;
    const int hx_even = (sh.halo[2] + 1) & ~1;
    s << "#define SL_BX " << sh.bx << "\n#define SL_TY " << sh.ty << "\n#define SL_RY " << sh.ry
      << "\n#define SL_ZC " << sh.zc << "\n#define SL_PD " << sh.pd << "\n#define SL_H0 "
      << sh.halo[0] << "\n#define SL_H1 " << sh.halo[1] << "\n#define SL_H2 " << sh.halo[2]
      << "\n#define SL_HXE " << hx_even << "\n";
    s << "__device__ constexpr int SL_SHIFT[NLA][3] = {";
    for (size_t l = 0; l < sh.shifts.size(); ++l)
        s << (l ? ", " : "") << "{" << sh.shifts[l][0] << ", " << sh.shifts[l][1] << ", "
          << sh.shifts[l][2] << "}";
    s << "};\n";
    s << R"(
#define SL_BY (SL_TY * SL_RY)
#define SL_PY (SL_BY + 2 * SL_H1)
#define SL_PX (SL_BX + 2 * SL_HXE)
#define SL_R (SL_ZC == 1 ? 1 : 2 * SL_H0 + 2)
#define SL_PLANE (SL_PY * SL_PX)
#define SL_PAIRS (SL_PY * (SL_PX / 2))
#define SL_LOADS ((SL_PAIRS + 255) / 256)

struct SlideArgs {
    const T* const* cur;   // tile table of the current contents
    T* const* dst;         // tile table of the new contents
    int shift;             // log2(tile edge)
    int shape[3];          // array extents in kernel dimensions (unused ones are 1)
    int grid[3];           // tiles per dimension
    int rs[3], re[3];      // assigned region
    int nbx, nby, nzc;     // workgroup grid
    int nblocks;
};
typedef T P2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int xcd_remap(int b, int n) {
    return (n % 8 == 0) ? (b % 8) * (n / 8) + b / 8 : b;
}

// Trailing-dimension part of a tile address; fixed for a lane while it marches.
struct Col { int t12; int rowoff; int plane; bool ok; };

__device__ __forceinline__ Col make_col(const SlideArgs& a, int gy, int gx, bool extra) {
    Col c;
    c.ok = extra && gy >= 0 && gy < a.shape[1] && gx >= 0 && gx < a.shape[2];
    const int cy = c.ok ? gy : 0, cx = c.ok ? gx : 0;
    const int t1 = cy >> a.shift, t2 = cx >> a.shift;
    const int lo1 = t1 << a.shift, lo2 = t2 << a.shift;
    const int w1 = min(lo1 + (1 << a.shift), a.shape[1]) - lo1;
    const int w2 = min(lo2 + (1 << a.shift), a.shape[2]) - lo2;
    c.t12 = t1 * a.grid[2] + t2;
    c.rowoff = (cy - lo1) * w2 + (cx - lo2);
    c.plane = w1 * w2;
    return c;
}

template <bool VEC, bool NT>
__device__ __forceinline__ void slide_run(const SlideArgs& a, const T* s) {
    __shared__ T lds[SL_R * SL_PLANE];
    const int blk = xcd_remap((int)blockIdx.x, a.nblocks);
    const int bx = blk % a.nbx;
    const int by = (blk / a.nbx) % a.nby;
    const int zc = blk / (a.nbx * a.nby);
    const int x0 = bx * SL_BX, y0 = by * SL_BY;
    const int z_begin = zc * SL_ZC;
    const int z_end = min(z_begin + SL_ZC, a.shape[0]);
    const int tid = (int)threadIdx.x;
    const int g12 = a.grid[1] * a.grid[2];

    // ---- staging lanes: pair index -> (py, px) of the patch ----
    Col lc[SL_LOADS], lc1[SL_LOADS];
    int lidx[SL_LOADS];
    const T* lbase[SL_LOADS];
    const T* lbase1[SL_LOADS];
#pragma unroll
    for (int i = 0; i < SL_LOADS; ++i) {
        const int pi = tid + i * 256;
        const int py = pi / (SL_PX / 2);
        const int px = (pi - py * (SL_PX / 2)) * 2;
        const bool in_patch = pi < SL_PAIRS;
        lidx[i] = py * SL_PX + px;
        lc[i] = make_col(a, y0 - SL_H1 + py, x0 - SL_HXE + px, in_patch);
        if (!VEC) lc1[i] = make_col(a, y0 - SL_H1 + py, x0 - SL_HXE + px + 1, in_patch);
        lbase[i] = nullptr;
        lbase1[i] = nullptr;
    }
    int l_t0 = -1; // tile index along the march that lbase[] belongs to (uniform)
    P2 pre[SL_PD][SL_LOADS];

    auto gload = [&](int gz, int slot) {
        const int t0 = gz >> a.shift;
        const int lz = gz - (t0 << a.shift);
        if (t0 != l_t0) {
            l_t0 = t0;
#pragma unroll
            for (int i = 0; i < SL_LOADS; ++i) {
                if (lc[i].ok) lbase[i] = a.cur[t0 * g12 + lc[i].t12];
                if (!VEC) { if (lc1[i].ok) lbase1[i] = a.cur[t0 * g12 + lc1[i].t12]; }
            }
        }
#pragma unroll
        for (int i = 0; i < SL_LOADS; ++i) {
            if (VEC) {
                if (lc[i].ok) {
                    const P2* src = reinterpret_cast<const P2*>(lbase[i] + (lz * lc[i].plane + lc[i].rowoff));
                    pre[slot][i] = NT ? __builtin_nontemporal_load(src) : *src;
                }
            } else {
                pre[slot][i][0] = lc[i].ok ? lbase[i][lz * lc[i].plane + lc[i].rowoff] : (T)0;
                pre[slot][i][1] = lc1[i].ok ? lbase1[i][lz * lc1[i].plane + lc1[i].rowoff] : (T)0;
            }
        }
    };
    auto lstore = [&](int gz, int slot) {
        T* plane = lds + (gz % SL_R) * SL_PLANE;
#pragma unroll
        for (int i = 0; i < SL_LOADS; ++i) {
            if (VEC) {
                if (lc[i].ok) *reinterpret_cast<P2*>(plane + lidx[i]) = pre[slot][i];
            } else {
                if (lc[i].ok) plane[lidx[i]] = pre[slot][i][0];
                if (lc1[i].ok) plane[lidx[i] + 1] = pre[slot][i][1];
            }
        }
    };

    // ---- output lanes ----
    const int txi = tid % (SL_BX / 2), tyi = tid / (SL_BX / 2);
    Col oc[SL_RY], oc1[SL_RY];
    T* obase[SL_RY];
    T* obase1[SL_RY];
    unsigned inmask = 0; // bit (2*r + e): element lies inside the assigned region in y and x
#pragma unroll
    for (int r = 0; r < SL_RY; ++r) {
        const int gy = y0 + tyi * SL_RY + r, gx = x0 + 2 * txi;
        oc[r] = make_col(a, gy, gx, true);
        if (!VEC) oc1[r] = make_col(a, gy, gx + 1, true);
        obase[r] = nullptr;
        obase1[r] = nullptr;
        const bool yin = gy >= a.rs[1] && gy < a.re[1];
#pragma unroll
        for (int e = 0; e < 2; ++e)
            if (yin && gx + e >= a.rs[2] && gx + e < a.re[2]) inmask |= 1u << (2 * r + e);
    }
    int o_t0 = -1;
    const int obase_idx = (SL_H1 + tyi * SL_RY) * SL_PX + SL_HXE + 2 * txi;

    auto compute = [&](int gz) {
        const int t0 = gz >> a.shift;
        const int lz = gz - (t0 << a.shift);
        if (t0 != o_t0) {
            o_t0 = t0;
#pragma unroll
            for (int r = 0; r < SL_RY; ++r) {
                if (oc[r].ok) obase[r] = a.dst[t0 * g12 + oc[r].t12];
                if (!VEC) { if (oc1[r].ok) obase1[r] = a.dst[t0 * g12 + oc1[r].t12]; }
            }
        }
        const bool zin = gz >= a.rs[0] && gz < a.re[0];
        const T* centre = lds + (gz % SL_R) * SL_PLANE;
#pragma unroll
        for (int r = 0; r < SL_RY; ++r) {
            if (oc[r].ok) {
                T res[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int at = obase_idx + r * SL_PX + e;
                    if (zin && ((inmask >> (2 * r + e)) & 1u)) {
                        T l[NLA], o[NOA];
#pragma unroll
                        for (int q = 0; q < NL; ++q)
                            l[q] = lds[((gz + SL_SHIFT[q][0] + SL_R) % SL_R) * SL_PLANE + at +
                                       SL_SHIFT[q][1] * SL_PX + SL_SHIFT[q][2]];
                        group_eval(l, s, o);
                        res[e] = o[0];
                    } else {
                        res[e] = centre[at];
                    }
                }
                T* out = obase[r] + (lz * oc[r].plane + oc[r].rowoff);
                if (VEC) {
                    P2 v; v[0] = res[0]; v[1] = res[1];
                    if (NT) __builtin_nontemporal_store(v, reinterpret_cast<P2*>(out));
                    else *reinterpret_cast<P2*>(out) = v;
                } else {
                    out[0] = res[0];
                    if (oc1[r].ok) obase1[r][lz * oc1[r].plane + oc1[r].rowoff] = res[1];
                }
            }
        }
    };

    // Plane p is needed by the steps z with |p - z| <= H0 of this workgroup.
    const int last_plane = min(z_end - 1 + SL_H0, a.shape[0] - 1);

    // prologue: planes z_begin-H0 .. z_begin+H0 go straight to LDS, the next PD-1 wait in registers
    for (int p = z_begin - SL_H0; p <= z_begin + SL_H0; ++p)
        if (p >= 0 && p <= last_plane) { gload(p, 0); lstore(p, 0); }
#pragma unroll
    for (int m = 1; m < SL_PD; ++m) {
        const int p = z_begin + SL_H0 + m;
        if (p <= last_plane) gload(p, (SL_H0 + m) % SL_PD);
    }
    __syncthreads();

    for (int zb = z_begin; zb < z_end; zb += SL_PD) {
#pragma unroll
        for (int j = 0; j < SL_PD; ++j) {
            const int gz = zb + j;
            if (gz < z_end) {
                // z_begin is a multiple of PD, so the register slot of a plane is static here
                const int far = gz + SL_H0 + SL_PD;   // issued now, stored PD-1 steps later
                const int near = gz + SL_H0 + 1;      // stored now, read by the next step
                if (far <= last_plane) gload(far, (j + SL_H0) % SL_PD);
                compute(gz);
                if (near <= last_plane) lstore(near, (j + SL_H0 + 1) % SL_PD);
                __syncthreads();
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(256) void grp_slide_v(SlideArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    slide_run<true, false>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_slide_vn(SlideArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    slide_run<true, true>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_slide_s(SlideArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    slide_run<false, false>(a, s);
}
)";
    return s.str();
}

} // namespace cnh
