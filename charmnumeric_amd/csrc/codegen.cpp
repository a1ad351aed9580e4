// AST -> HIP source for one fused group (host-only).
#include "codegen.h"

#include <cmath>
#include <cstring>
#include <map>
#include <sstream>

namespace cnh {

const char* dtype_ctype(int dtype) {
    switch (dtype) {
    case CNH_F32: return "float";
    case CNH_F64: return "double";
    case CNH_I32: return "int";
    case CNH_I64: return "long long";
    }
    return "void";
}

namespace {

bool is_int(int dt) { return dt == CNH_I32 || dt == CNH_I64; }

std::string fmt(const char* f, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof buf, f, ap);
    va_end(ap);
    return buf;
}

// Literal of a scalar leaf in the group's element type. Integers are cast through int64,
// floats through double (src/jit.cpp:108-116 upstream).
std::string literal(int dtype, double c) {
    if (is_int(dtype)) {
        long long v = 0;
        if (std::isfinite(c) && c > -9.2233720368547758e18 && c < 9.2233720368547758e18)
            v = (long long)c;
        if (dtype == CNH_I32)
            v = (long long)(int32_t)(uint32_t)(uint64_t)v;
        if (v == (-9223372036854775807LL - 1))
            return "((T)(-9223372036854775807LL - 1))";
        return fmt("((T)(%lldLL))", v);
    }
    if (dtype == CNH_F32) {
        float f = (float)c;
        if (std::isnan(f))
            return "((T)__builtin_nanf(\"\"))";
        if (std::isinf(f))
            return f > 0 ? "((T)__builtin_inff())" : "((T)(-__builtin_inff()))";
        return fmt("((T)(%af))", (double)f);
    }
    if (std::isnan(c))
        return "((T)__builtin_nan(\"\"))";
    if (std::isinf(c))
        return c > 0 ? "((T)__builtin_inf())" : "((T)(-__builtin_inf()))";
    return fmt("((T)(%a))", c);
}

// Small multiples of a quarter (0, +-1, 0.5, 2.5, -1 for a negation, ...) stay in the source, where
// the compiler can fold them; any other literal (a time step, a coefficient computed on the host)
// becomes a launch parameter, so that a loop whose literal changes every step keeps one code object
// instead of compiling a kernel per value.
bool literal_stays_in_source(int dtype, double c) {
    if (!std::isfinite(c))
        return true;
    if (std::fabs(c) > 16.0)
        return false;
    const double q = c * 4.0;
    return q == std::floor(q) || is_int(dtype);
}

} // namespace
void literal_value(int dtype, double c, void* out) {
    if (is_int(dtype)) {
        long long v = 0;
        if (std::isfinite(c) && c > -9.2233720368547758e18 && c < 9.2233720368547758e18)
            v = (long long)c;
        if (dtype == CNH_I32) {
            const int32_t w = (int32_t)(uint32_t)(uint64_t)v;
            std::memcpy(out, &w, 4);
        } else {
            std::memcpy(out, &v, 8);
        }
    } else if (dtype == CNH_F32) {
        const float f = (float)c;
        std::memcpy(out, &f, 4);
    } else {
        std::memcpy(out, &c, 8);
    }
}
namespace {

struct Value {
    std::string expr;
    bool scalar = false;
    bool valid = false;
};

std::string leaf_key(const cnh_ast_node& root, int oi, const cnh_ast_node& op) {
    // Same identity rule as the upstream leafUseKey (src/jit.cpp:265-284): name, rank, region.
    std::string key = fmt("%d|%d", op.result_name, op.ndims);
    if (!root.has_operand_region[oi])
        return key + "|null";
    const cnh_region& r = root.operand_regions[oi];
    if (r.is_global)
        return key + "|global";
    for (int d = 0; d < op.ndims && d < CNH_MAX_ND; ++d)
        key += fmt("|%d:%d:%d", r.start[d], r.stop[d], r.step[d]);
    return key;
}

std::string binop(int dtype, int opc, const std::string& a, const std::string& b) {
    if (is_int(dtype)) {
        switch (opc) {
        case CNH_OP_ADD: return "(T)((UT)" + a + " + (UT)" + b + ")";
        case CNH_OP_SUB: return "(T)((UT)" + a + " - (UT)" + b + ")";
        case CNH_OP_MUL: return "(T)((UT)" + a + " * (UT)" + b + ")";
        default: return "cn_idiv(" + a + ", " + b + ")";
        }
    }
    const char* sym = opc == CNH_OP_ADD ? "+" : opc == CNH_OP_SUB ? "-" : opc == CNH_OP_MUL ? "*" : "/";
    return a + " " + sym + " " + b;
}

} // namespace

int build_group_program(const cnh_ast* ast, int dtype, int ndims, GroupProgram& p,
                        std::string& err) {
    if (!ast || !ast->nodes || !ast->roots || ast->n_roots <= 0) {
        err = "empty AST";
        return -2;
    }
    if (ndims < 1 || ndims > CNH_MAX_ND) {
        err = fmt("ndims %d not in 1..3", ndims);
        return -2;
    }
    if (dtype < 0 || dtype > 3) {
        err = fmt("unknown dtype %d", dtype);
        return -2;
    }
    for (int r = 0; r < ast->n_roots; ++r)
        if (ast->roots[r] < 0 || ast->roots[r] >= ast->n_nodes) {
            err = "root index out of range";
            return -2;
        }
    p = GroupProgram();
    p.dtype = dtype;
    p.ndims = ndims;

    std::map<int, int> internal;
    for (int r = 0; r < ast->n_roots; ++r)
        internal[ast->nodes[ast->roots[r]].result_name] = 1;

    std::map<std::string, int> load_by_key;
    std::map<int, int> bcast_by_name;
    std::map<int, Value> values; // result_name -> expression

    for (int r = 0; r < ast->n_roots; ++r) {
        const cnh_ast_node& root = ast->nodes[ast->roots[r]];
        if (root.n_operands < 0 || root.n_operands > 2) {
            err = "operand count out of range";
            return -2;
        }
        for (int oi = 0; oi < root.n_operands; ++oi) {
            int on = root.operands[oi];
            if (on < 0)
                continue;
            if (on >= ast->n_nodes) {
                err = "operand index out of range";
                return -2;
            }
            const cnh_ast_node& op = ast->nodes[on];
            if (internal.count(op.result_name))
                continue;
            if (root.opcode == CNH_OP_SET_REGION && oi == 0)
                continue;
            if (op.opcode != CNH_OP_NOOP && op.opcode != CNH_OP_CREATE)
                continue;
            if (op.is_scalar) {
                auto seen = values.find(op.result_name);
                if (seen != values.end() && seen->second.scalar)
                    continue;                  // the same literal node under another root
                Value v;
                if (literal_stays_in_source(dtype, op.scalar)) {
                    v.expr = literal(dtype, op.scalar);
                } else {
                    v.expr = fmt("s[NS + %d]", (int)p.lit_values.size());
                    p.lit_values.push_back(op.scalar);
                }
                v.scalar = true;
                v.valid = true;
                values[op.result_name] = v;
            } else if (op.is_broadcast) {
                if (!bcast_by_name.count(op.result_name)) {
                    bcast_by_name[op.result_name] = (int)p.bcast_nodes.size();
                    p.bcast_nodes.push_back(on);
                    p.bcast_names.push_back(op.result_name);
                }
                Value v;
                v.expr = fmt("s[%d]", bcast_by_name[op.result_name]);
                v.scalar = true;
                v.valid = true;
                values[op.result_name] = v;
            } else {
                std::string key = leaf_key(root, oi, op);
                LeafUse u;
                u.node = on;
                u.root = r;
                u.operand = oi;
                u.name = op.result_name;
                u.has_region = root.has_operand_region[oi] && !root.operand_regions[oi].is_global;
                u.region = root.operand_regions[oi];
                auto it = load_by_key.find(key);
                if (it == load_by_key.end()) {
                    u.load = (int)p.load_leaf.size();
                    load_by_key[key] = u.load;
                    p.load_leaf.push_back((int)p.leaves.size());
                } else {
                    u.load = it->second;
                    p.load_leaf[u.load] = (int)p.leaves.size(); // the later argument wins
                }
                p.leaves.push_back(u);
            }
        }
    }

    auto lookup = [&](const cnh_ast_node& root, int oi) -> Value {
        Value none;
        if (oi >= root.n_operands || root.operands[oi] < 0)
            return none;
        const cnh_ast_node& op = ast->nodes[root.operands[oi]];
        std::string key = leaf_key(root, oi, op);
        if (root.has_operand_region[oi]) {
            auto it = load_by_key.find(key);
            if (it != load_by_key.end()) {
                Value v;
                v.expr = fmt("l[%d]", it->second);
                v.valid = true;
                return v;
            }
        }
        auto it = values.find(op.result_name);
        if (it != values.end())
            return it->second;
        auto it2 = load_by_key.find(key);
        if (it2 != load_by_key.end()) {
            Value v;
            v.expr = fmt("l[%d]", it2->second);
            v.valid = true;
            return v;
        }
        return none;
    };

    int n_tmp = 0;
    std::ostringstream body;
    for (int r = 0; r < ast->n_roots; ++r) {
        const cnh_ast_node& root = ast->nodes[ast->roots[r]];
        int opc = root.opcode;
        if (opc == CNH_OP_NOOP || opc == CNH_OP_CREATE)
            continue;
        Value res;
        if (opc == CNH_OP_SET_REGION) {
            res = lookup(root, 1);
            if (!res.valid) {
                err = "SET_REGION without a usable right-hand side";
                return -10;
            }
        } else if (opc == CNH_OP_SCALAR_OF) {
            res = lookup(root, 0);
            if (!res.valid || !res.scalar || root.is_temp) {
                err = "SCALAR_OF is an output that takes a value formed from scalars alone";
                return -12;
            }
        } else if (opc == CNH_OP_COPY || opc == CNH_OP_SUM_OF || opc == CNH_OP_MAXABS_OF) {
            res = lookup(root, 0);
            if (!res.valid || res.scalar) {
                err = "COPY and the reducing roots need an array operand";
                return -12;
            }
            if (opc != CNH_OP_COPY && (root.is_temp || dtype != CNH_F64)) {
                err = "a reducing root is an fp64 output of its group";
                return -12;
            }
        } else if (opc >= CNH_OP_ADD && opc <= CNH_OP_DIV) {
            Value a = lookup(root, 0), b = lookup(root, 1);
            if (!a.valid || !b.valid) {
                err = "binary op with an unresolved operand";
                return -11;
            }
            std::string name = fmt("t%d", n_tmp++);
            body << "    const T " << name << " = " << binop(dtype, opc, a.expr, b.expr) << ";\n";
            res.expr = name;
            res.scalar = a.scalar && b.scalar;
            res.valid = true;
        } else if (opc == CNH_OP_TANH || opc == CNH_OP_EXP) {
            if (is_int(dtype)) {
                err = "tanh/exp have no integer form";
                return -21;
            }
            Value a = lookup(root, 0);
            if (!a.valid || a.scalar) {
                err = "unary op needs an array operand";
                return -12;
            }
            std::string name = fmt("t%d", n_tmp++);
            const char* fn = opc == CNH_OP_TANH ? "cn_tanh" : "cn_exp";
            body << "    const T " << name << " = " << fn << "(" << a.expr << ");\n";
            res.expr = name;
            res.valid = true;
            p.uses_transcendental = true;
        } else {
            err = fmt("opcode %d cannot be part of a fused group", opc);
            return -13;
        }
        values[root.result_name] = res;
    }

    for (int r = 0; r < ast->n_roots; ++r) {
        const cnh_ast_node& root = ast->nodes[ast->roots[r]];
        if (root.opcode == CNH_OP_NOOP || root.opcode == CNH_OP_CREATE || root.is_temp)
            continue;
        auto it = values.find(root.result_name);
        if (it == values.end() || !it->second.valid) {
            err = "output root without a value";
            return -15;
        }
        p.out_roots.push_back(r);
        p.out_names.push_back(root.result_name);
        bool sr = root.opcode == CNH_OP_SET_REGION;
        p.out_is_set_region.push_back(sr ? 1 : 0);
        p.out_reduce.push_back(root.opcode == CNH_OP_SUM_OF ? 1 : root.opcode == CNH_OP_MAXABS_OF ? 2
                               : root.opcode == CNH_OP_SCALAR_OF ? 3 : 0);
        int target = root.result_name;
        if (sr && root.n_operands > 0 && root.operands[0] >= 0)
            target = ast->nodes[root.operands[0]].result_name;
        p.out_target.push_back(target);
        p.out_region.push_back(root.region);
        p.out_expr.push_back(it->second.expr);
    }
    for (size_t j = 0; j < p.out_expr.size(); ++j)
        body << "    o[" << j << "] = " << p.out_expr[j] << ";\n";
    p.body = body.str();
    return 0;
}

namespace {

// Text shared by every variant: element type, scalar block, helpers and the group body.
std::string prelude(const GroupProgram& p) {
    int NL = (int)p.load_leaf.size(), NS = (int)p.bcast_nodes.size(), NO = (int)p.out_roots.size();
    std::ostringstream s;
    s << "// generated by libcnhip for one fused group; dtype " << dtype_ctype(p.dtype) << ", rank "
      << p.ndims << "\n";
    s << "typedef " << dtype_ctype(p.dtype) << " T;\n";
    s << "typedef unsigned " << (p.dtype == CNH_I64 ? "long long" : "int") << " UT;\n";
    s << "typedef long long i64;\n";
    s << "#define NL " << NL << "\n#define NS " << NS << "\n#define NO " << NO << "\n";
    const int NLIT = (int)p.lit_values.size();
    s << "#define NLA " << (NL > 0 ? NL : 1) << "\n#define NSA " << (NS > 0 ? NS : 1)
      << "\n#define NOA " << (NO > 0 ? NO : 1) << "\n";
    // literal scalars handed over with the launch: s[NS .. NS + NLIT) of the scalar values
    s << "#define NLIT " << NLIT << "\n#define NLITA " << (NLIT > 0 ? NLIT : 1) << "\n#define NSV "
      << (NS + NLIT > 0 ? NS + NLIT : 1) << "\n";
    s << "struct Scal { const T* p[NSA]; T v[NSA]; T c[NLITA]; };\n";
    if (is_int(p.dtype)) {
        // Truncating signed division; x/0 -> 0 and MIN/-1 -> MIN are fixed here because the
        // upstream operation (arith.divsi) leaves both undefined.
        s << "__device__ __forceinline__ T cn_idiv(T a, T b) {\n"
             "    if (b == 0) return 0;\n"
             "    if (b == -1) return (T)((UT)0 - (UT)a);\n"
             "    return a / b;\n}\n";
    } else if (p.dtype == CNH_F64) {
        // exp/tanh must give what the host C library gives (upstream lowers math.exp/tanh to
        // libm calls), so the group carries its own restatement instead of the device library's.
        if (p.body.find("cn_exp(") != std::string::npos || p.body.find("cn_tanh(") != std::string::npos)
            s << libm_f64_text()
              << "__device__ __forceinline__ T cn_exp(T x) { return cn_exp_f64(x); }\n"
                 "__device__ __forceinline__ T cn_tanh(T x) { return cn_tanh_f64(x); }\n";
    } else {
        if (p.body.find("cn_exp(") != std::string::npos || p.body.find("cn_tanh(") != std::string::npos)
            s << libm_f32_text()
              << "__device__ __forceinline__ T cn_exp(T x) { return cn_exp_f32(x); }\n"
                 "__device__ __forceinline__ T cn_tanh(T x) { return cn_tanh_f32(x); }\n";
    }
    // A code object may be built for ONE entry point (CNH_ONLY_NAME set ahead of this text): every
    // other entry point returns at once and costs the compiler nothing. The comparison of two
    // constant strings is folded at compile time.
    s << "#ifdef CNH_ONLY_NAME\n"
         "#define CNH_ENTRY_GUARD if (__builtin_strcmp(__func__, CNH_ONLY_NAME) != 0) return;\n"
         "#else\n#define CNH_ENTRY_GUARD\n#endif\n";
    s << "__device__ __forceinline__ void load_scalars(const Scal& sc, T* s) {\n"
         "#pragma unroll\n"
         "    for (int i = 0; i < NS; ++i) s[i] = sc.p[i] ? *sc.p[i] : sc.v[i];\n"
         "#pragma unroll\n"
         "    for (int i = 0; i < NLIT; ++i) s[NS + i] = sc.c[i];\n}\n";
    s << "__device__ __forceinline__ void group_eval(const T* l, const T* s, T* o) {\n"
      << "    (void)l; (void)s;\n"
      << p.body << "}\n";
    s << "template <typename S> __device__ __forceinline__ int find_seg(const S* segs, int n, i64 "
         "blk) {\n"
         "    int lo = 0, hi = n - 1;\n"
         "    while (lo < hi) { int mid = (lo + hi + 1) >> 1; if (segs[mid].blk0 <= blk) lo = mid; "
         "else hi = mid - 1; }\n"
         "    return lo;\n}\n";
    return s.str();
}

std::string flat_source(const GroupProgram& p) {
    int vec = 16 / dtype_size(p.dtype);
    std::ostringstream s;
    s << prelude(p);
    s << "#define VECW " << vec << "\n";
    // Outputs that are reduced instead of stored: a mask over the output list, and the statement
    // that folds one element's values into the lane's running results.
    unsigned mask = 0, once_mask = 0;
    int nred = 0;
    std::ostringstream fold, init;
    for (size_t j = 0; j < p.out_reduce.size(); ++j) {
        if (!p.out_reduce[j])
            continue;
        mask |= 1u << j;
        if (p.out_reduce[j] == 3) {
            once_mask |= 1u << j;
            continue;
        }
        if (p.out_reduce[j] == 1)
            fold << " racc[" << nred << "] += o[" << j << "];";
        else
            fold << " { const T a_ = o[" << j << "] < 0 ? -o[" << j << "] : o[" << j << "]; racc[" << nred
                 << "] = a_ > racc[" << nred << "] ? a_ : racc[" << nred << "]; }";
        ++nred;
    }
    s << "#define RED_MASK " << mask << "u\n#define ONCE_MASK " << once_mask << "u\n#define NR " << nred
      << "\n#define NRA " << (nred ? nred : 1) << "\n";
    s << "#define RED_FOLD(o, racc) do {" << fold.str() << " } while (0)\n";
    std::ostringstream comb;
    {
        int q = 0;
        for (size_t j = 0; j < p.out_reduce.size(); ++j) {
            if (!p.out_reduce[j] || p.out_reduce[j] == 3)
                continue;
            if (p.out_reduce[j] == 1)
                comb << " racc[" << q << "] += other[" << q << "];";
            else
                comb << " racc[" << q << "] = other[" << q << "] > racc[" << q << "] ? other[" << q
                     << "] : racc[" << q << "];";
            ++q;
        }
    }
    s << "#define RED_COMBINE(racc, other) do {" << comb.str() << " } while (0)\n";
    s << R"(
// Contiguous segments: every memref of a partition is dense and has the same element count.
// One 128-bit vector per lane and a grid that covers the data once: on this part the plain form
// streams faster than unrolled or persistent ones. NT selects non-temporal loads and stores for
// launches whose traffic exceeds what the last-level cache could keep anyway.
// Outputs in RED_MASK are not stored: every lane folds its elements' values into racc[], the
// wavefront combines the lanes in a fixed order, the workgroup its four wavefronts in order, and
// one partial per workgroup and reduction goes to ro.slots[q][blockIdx.x] for a later launch to fold.
struct Seg { i64 n; i64 blk0; const T* in[NLA]; T* out[NOA]; };
typedef T TV __attribute__((ext_vector_type(VECW)));
#define OUT_STORED(j) (((RED_MASK >> (j)) & 1u) == 0u)

// Outputs in ONCE_MASK (CNH_OP_SCALAR_OF) hold a value formed from the launch's scalars alone: the
// first lane of the launch stores it once, at element 0 of the first segment's output.
__device__ __forceinline__ void store_once(T* const* out, const T* s) {
    if (ONCE_MASK != 0u && blockIdx.x == 0 && threadIdx.x == 0) {
        T l[NLA], o[NOA];
#pragma unroll
        for (int k = 0; k < NLA; ++k) l[k] = 0;
        group_eval(l, s, o);
#pragma unroll
        for (int j = 0; j < NO; ++j)
            if ((ONCE_MASK >> j) & 1u) out[j][0] = o[j];
    }
}

// Workgroups of one wavefront where nothing is reduced (a plain triad over 2^24 doubles streams at
// 0.86 of the HBM peak with 64 lanes a workgroup, 0.84 with 128, 0.82 with 256 to 1024); reducing
// launches keep 256 lanes, whose four wavefronts share one partial.
#if NR > 0
#define FLAT_WG 256
#else
#define FLAT_WG 64
#endif
template <bool NT, int WG>
__device__ __forceinline__ void flat_vec(const Seg& sg, i64 blk, const T* s, T* racc) {
    (void)racc;
    const i64 i = (blk * WG + threadIdx.x) * VECW;
    const i64 n = sg.n;
    if (i + VECW <= n) {
        TV lv[NLA];
#pragma unroll
        for (int k = 0; k < NL; ++k) {
            const TV* src = reinterpret_cast<const TV*>(sg.in[k] + i);
            lv[k] = NT ? __builtin_nontemporal_load(src) : *src;
        }
        TV ov[NOA];
#pragma unroll
        for (int e = 0; e < VECW; ++e) {
            T l[NLA], o[NOA];
#pragma unroll
            for (int k = 0; k < NL; ++k) l[k] = lv[k][e];
            group_eval(l, s, o);
            RED_FOLD(o, racc);
#pragma unroll
            for (int j = 0; j < NO; ++j) ov[j][e] = o[j];
        }
#pragma unroll
        for (int j = 0; j < NO; ++j) {
            if (OUT_STORED(j)) {
                TV* dst = reinterpret_cast<TV*>(sg.out[j] + i);
                if (NT) __builtin_nontemporal_store(ov[j], dst); else *dst = ov[j];
            }
        }
    } else {
        for (i64 x = i; x < n; ++x) {
            T l[NLA], o[NOA];
#pragma unroll
            for (int k = 0; k < NL; ++k) l[k] = sg.in[k][x];
            group_eval(l, s, o);
            RED_FOLD(o, racc);
#pragma unroll
            for (int j = 0; j < NO; ++j)
                if (OUT_STORED(j)) sg.out[j][x] = o[j];
        }
    }
}

// Pointers that are not 16-byte aligned: one element per lane.
template <int WG>
__device__ __forceinline__ void flat_scalar(const Seg& sg, i64 blk, const T* s, T* racc) {
    (void)racc;
#pragma unroll
    for (int u = 0; u < VECW; ++u) {
        const i64 i = (blk * VECW + u) * WG + threadIdx.x;
        if (i < sg.n) {
            T l[NLA], o[NOA];
#pragma unroll
            for (int k = 0; k < NL; ++k) l[k] = sg.in[k][i];
            group_eval(l, s, o);
            RED_FOLD(o, racc);
#pragma unroll
            for (int j = 0; j < NO; ++j)
                if (OUT_STORED(j)) sg.out[j][i] = o[j];
        }
    }
}

#if NR > 0
struct RedOut { T* slots[NRA]; };
__device__ __forceinline__ void red_finish(T* racc, const RedOut& ro) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        T other[NRA];
#pragma unroll
        for (int q = 0; q < NR; ++q) other[q] = __shfl_xor(racc[q], m, 64);
        RED_COMBINE(racc, other);
    }
    // the four wavefronts of the workgroup, in order, then one partial per workgroup and reduction
    __shared__ T red_lds[4][NRA];
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
        for (int q = 0; q < NR; ++q) red_lds[threadIdx.x >> 6][q] = racc[q];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            T other[NRA];
#pragma unroll
            for (int q = 0; q < NR; ++q) other[q] = red_lds[w][q];
            RED_COMBINE(racc, other);
        }
#pragma unroll
        for (int q = 0; q < NR; ++q)
            ro.slots[q][(i64)blockIdx.x] = racc[q];
    }
}
#define RED_PARAM , RedOut ro
#define RED_BEGIN T racc[NRA]; for (int q = 0; q < NRA; ++q) racc[q] = 0;
#define RED_END red_finish(racc, ro);
#else
#define RED_PARAM
#define RED_BEGIN T* racc = nullptr;
#define RED_END
#endif

// Run-time scalars that are given as partial sums (what a reducing launch left behind): scalar i is
// the sum of n[i] values at sc.p[i], taken by every workgroup in the same fixed order (lane-strided
// running sums, butterfly over the wavefront, the four wavefronts left to right), so all workgroups
// compute with the same bits; workgroup 0 also stores it at out[i] when that is not null.
struct Fold { T* out[NSA]; int n[NSA]; };
__device__ __forceinline__ void load_scalars_folding(const Scal& sc, const Fold& fd, T* s) {
    __shared__ T fold_lds[4];
#pragma unroll
    for (int i = 0; i < NLIT; ++i) s[NS + i] = sc.c[i];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        if (sc.p[i] == nullptr) {
            s[i] = sc.v[i];
        } else if (fd.n[i] <= 1) {
            s[i] = *sc.p[i];
        } else {
            T v = 0;
            for (int j = threadIdx.x; j < fd.n[i]; j += 256) v += sc.p[i][j];
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
            if ((threadIdx.x & 63) == 0) fold_lds[threadIdx.x >> 6] = v;
            __syncthreads();
            v = ((fold_lds[0] + fold_lds[1]) + fold_lds[2]) + fold_lds[3];
            __syncthreads();
            s[i] = v;
            if (fd.out[i] != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *fd.out[i] = v;
        }
    }
}

#define FLAT_ENTRY(NAME, CALL, CALL256)                                                          \
extern "C" __global__ __launch_bounds__(FLAT_WG) void grp_flat_##NAME(const Seg* segs, int nseg, \
                                                                  Scal sc RED_PARAM) {           \
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);                                                               \
    RED_BEGIN                                                                                    \
    const int k = find_seg(segs, nseg, (i64)blockIdx.x);                                         \
    const Seg& sg = segs[k];                                                                     \
    const i64 blk = (i64)blockIdx.x - sg.blk0;                                                   \
    CALL;                                                                                        \
    store_once(segs[0].out, s);                                                                  \
    RED_END                                                                                      \
}                                                                                                \
extern "C" __global__ __launch_bounds__(FLAT_WG) void grp_flat1_##NAME(Seg sg, Scal sc RED_PARAM) { \
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);                                                               \
    RED_BEGIN                                                                                    \
    const i64 blk = (i64)blockIdx.x;                                                             \
    CALL;                                                                                        \
    store_once(sg.out, s);                                                                       \
    RED_END                                                                                      \
}                                                                                                \
extern "C" __global__ __launch_bounds__(256) void grp_flat1f_##NAME(Seg sg, Scal sc, Fold fd    \
                                                                    RED_PARAM) {                 \
    CNH_ENTRY_GUARD T s[NSV]; load_scalars_folding(sc, fd, s);                                                   \
    RED_BEGIN                                                                                    \
    const i64 blk = (i64)blockIdx.x;                                                             \
    CALL256;                                                                                     \
    store_once(sg.out, s);                                                                       \
    RED_END                                                                                      \
}
FLAT_ENTRY(v, (flat_vec<false, FLAT_WG>(sg, blk, s, racc)), (flat_vec<false, 256>(sg, blk, s, racc)))
FLAT_ENTRY(vn, (flat_vec<true, FLAT_WG>(sg, blk, s, racc)), (flat_vec<true, 256>(sg, blk, s, racc)))
FLAT_ENTRY(s, (flat_scalar<FLAT_WG>(sg, blk, s, racc)), (flat_scalar<256>(sg, blk, s, racc)))
)";
    return s.str();
}

std::string nd_source(const GroupProgram& p) {
    std::ostringstream s;
    s << prelude(p);
    s << R"(
// Strided cells: arbitrary memref descriptors (offset folded into the pointer), rank padded to 3.
struct Cell {
    i64 sizes[3]; i64 blk0; i64 nchunks;
    const T* in[NLA]; i64 istr[NLA][3];
    T* out[NOA]; i64 ostr[NOA][3];
};
// PER elements per lane, a workgroup's width apart: 4 for large launches (256 lanes a workgroup); 1
// for small ones (one wavefront a workgroup), which then spread over four times as many wavefronts (a 256 x 1024 gate statement with exp and tanh in fp64: 19.6 us
// with one wavefront per SIMD busy, latency-bound).
template <int ND_PER_THREAD, int WG>
__device__ __forceinline__ void nd_run(const Cell& c, i64 blk, const T* s) {
    const i64 outer = blk / c.nchunks;
    const i64 chunk = blk - outer * c.nchunks;
    const i64 i1 = outer % c.sizes[1];
    const i64 i0 = outer / c.sizes[1];
    const i64 x0 = chunk * (WG * ND_PER_THREAD) + threadIdx.x;
    T lv[NLA][ND_PER_THREAD];
#pragma unroll
    for (int u = 0; u < ND_PER_THREAD; ++u) {
        const i64 x = x0 + (i64)u * WG;
        if (x < c.sizes[2]) {
#pragma unroll
            for (int k = 0; k < NL; ++k)
                lv[k][u] = c.in[k][i0 * c.istr[k][0] + i1 * c.istr[k][1] + x * c.istr[k][2]];
        }
    }
#pragma unroll
    for (int u = 0; u < ND_PER_THREAD; ++u) {
        const i64 x = x0 + (i64)u * WG;
        if (x < c.sizes[2]) {
            T l[NLA], o[NOA];
#pragma unroll
            for (int k = 0; k < NL; ++k) l[k] = lv[k][u];
            group_eval(l, s, o);
#pragma unroll
            for (int j = 0; j < NO; ++j)
                c.out[j][i0 * c.ostr[j][0] + i1 * c.ostr[j][1] + x * c.ostr[j][2]] = o[j];
        }
    }
}

extern "C" __global__ __launch_bounds__(256) void grp_nd(const Cell* cells, int ncell, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    const int k = find_seg(cells, ncell, (i64)blockIdx.x);
    nd_run<4, 256>(cells[k], (i64)blockIdx.x - cells[k].blk0, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_nd1(Cell cell, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    nd_run<4, 256>(cell, (i64)blockIdx.x, s);
}
extern "C" __global__ __launch_bounds__(64) void grp_nd_p1(const Cell* cells, int ncell, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    const int k = find_seg(cells, ncell, (i64)blockIdx.x);
    nd_run<1, 64>(cells[k], (i64)blockIdx.x - cells[k].blk0, s);
}
extern "C" __global__ __launch_bounds__(64) void grp_nd1_p1(Cell cell, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    nd_run<1, 64>(cell, (i64)blockIdx.x, s);
}
)";
    return s.str();
}

// The product kernel with the group's statements in its epilogue: the text of gemm_kernel.inc in one of
// its three forms (1: two sets of 4 x 2 wavefronts sharing the K steps, for grids of one workgroup per
// CU; 2: one such set; 3: 2 x 2 wavefronts of 32 x 32; 64 x 64 tiles and buffer loads in all of them),
// with a workgroup's 64 columns taken as 64 / q from each of q column blocks of the product. When the
// sums are complete they go to global memory and to an LDS tile; then every lane of the workgroup
// takes elements (row, block column) of the tile's rows: loads that name a column block of the
// product come from the tile, the others from their memrefs, and the statements are those of the
// strided-cell kernel.
std::string product_source(const GroupProgram& p, int q, int form) {
    std::ostringstream s;
    s << prelude(p);
    s << "typedef long long cn_i64;\ntypedef int cn_i32;\n";
    s << "#define CN_EPILOGUE 1\n#define CN_EPI_Q " << q << "\n";
    s << R"(
struct Cell {
    i64 sizes[3]; i64 blk0; i64 nchunks;
    const T* in[NLA]; i64 istr[NLA][3];
    T* out[NOA]; i64 ostr[NOA][3];
};
// src[k]: which column block of the product load k is (-1: an array of its own, read through
// cell.in[k]); nblock: width of a column block
struct EpiArgs { Cell cell; Scal sc; int src[NLA]; int nblock; int unused; };
constexpr int BKT = 16;
constexpr bool FULL = true, BUF = true;
)";
    s << (form == 3 ? "constexpr int WM = 2, WN = 2, TM = 2, TN = 2, KS = 1;\n"
                    : form == 2 ? "constexpr int WM = 4, WN = 2, TM = 1, TN = 2, KS = 1;\n"
                                : "constexpr int WM = 4, WN = 2, TM = 1, TN = 2, KS = 2;\n");
    s << R"(

// Elements (row, block column) of the workgroup's tile a lane takes: e = lane, lane + LANES, ...
// The loads that do not come from the product are issued before the first K step when a lane has a
// single element (four column blocks): their latency then hides behind the whole product.
template <int BM, int CPB, int LANES>
struct CnEpi {
    static constexpr int EPL = BM * CPB / LANES;
    static_assert(EPL * LANES == BM * CPB, "the lanes divide the tile's elements evenly");
    static constexpr bool EARLY = EPL == 1;
    T pre[EARLY ? NLA : 1];
    __device__ __forceinline__ T load(const EpiArgs& epi, int k, int e, int m0, int n0) const {
        const Cell& c = epi.cell;
        const i64 i1 = m0 + e / CPB, x = n0 + e % CPB;
        return c.in[k][i1 * c.istr[k][1] + x * c.istr[k][2]];
    }
    __device__ __forceinline__ void prefetch(const EpiArgs& epi, int m0, int n0) {
        if (EARLY) {
#pragma unroll
            for (int k = 0; k < NL; ++k)
                if (epi.src[k] < 0)
                    pre[k] = load(epi, k, (int)threadIdx.x, m0, n0);
        }
    }
    // ct[g]: the tile of sums of wavefront set g. The product's value is set 0's sum plus set 1's.
    __device__ __forceinline__ void run(const EpiArgs& epi, double (*ct)[BM][WN * TN * 16 + 1], double* C, i64 ldc,
                                        int m0, int n0) const {
        T s[NSV]; load_scalars(epi.sc, s);
        const Cell& c = epi.cell;
#pragma unroll
        for (int u = 0; u < EPL; ++u) {
            const int e = (int)threadIdx.x + u * LANES;
            const int row = e / CPB, hc = e % CPB;
            const i64 i1 = m0 + row, x = n0 + hc;
            T v[CN_EPI_Q], l[NLA], o[NOA];
#pragma unroll
            for (int b = 0; b < CN_EPI_Q; ++b) {
                v[b] = ct[0][row][b * CPB + hc];
                if (KS > 1)
                    v[b] += ct[1][row][b * CPB + hc];
            }
#pragma unroll
            for (int k = 0; k < NL; ++k) {
                const int b = epi.src[k];
                if (b < 0) {
                    l[k] = EARLY ? pre[k] : load(epi, k, e, m0, n0);
                } else {
                    l[k] = v[0];
#pragma unroll
                    for (int w = 1; w < CN_EPI_Q; ++w)
                        l[k] = b == w ? v[w] : l[k];
                }
            }
            group_eval(l, s, o);
            // every store behind the arithmetic: a wait for a table lookup of exp in the middle of it
            // would otherwise also wait for the stores issued before it
#pragma unroll
            for (int b = 0; b < CN_EPI_Q; ++b)
                C[i1 * ldc + (i64)b * epi.nblock + x] = v[b];
#pragma unroll
            for (int j = 0; j < NO; ++j)
                c.out[j][i1 * c.ostr[j][1] + x * c.ostr[j][2]] = o[j];
        }
    }
};
#define CN_GEMM_HEAD(...) extern "C" __global__ __launch_bounds__(WM * WN * 64 * KS) void grp_product(__VA_ARGS__)
#define CN_GEMM_MORE_ARGS , EpiArgs epi
)";
    s << gemm_kernel_text();
    return s.str();
}

std::string tiles_source(const GroupProgram& p) {
    std::ostringstream s;
    s << prelude(p);
    s << R"(
// Gather over tiled arrays resident on this device: every element of every destination tile is
// produced by one thread, which resolves each shifted/strided input coordinate to its owning
// tile (tile edge is a power of two) and reads it there. Rank padded to 3.
// py, pz: elements between rows and between planes inside every tile when the tiles are views
// into one larger row-major block; py = 0: a tile is contiguous over its own extents.
struct Tiled {
    int shift; int tile; int off[3]; int shape[3]; int glo[3]; int grid[3];
    const T* const* tiles;
    int py, pz;
};
// cs, w: origin and extents of the tile; bs, bw: what of it this launch visits. A ping-pong
// launch walks the whole tile (bs = 0, bw = w, in elements). An in-place launch (TilesArgs.lattice)
// walks the points of the assigned region's lattice that fall into the tile: bs = index of the
// first such point along each dimension, bw = how many.
// rsh: a workgroup covers 2^rsh consecutive rows with 256 >> rsh lanes each (short rows, e.g. the
// 128-wide tiles of rank-3 arrays, would otherwise leave most lanes idle); 0 = one row.
struct DTile { i64 blk0; int cs[3]; int w[3]; int nchunks; int rsh; int bs[3]; int bw[3]; T* dst; const T* cur; int py, pz; };
struct LeafReg { int arr; int start[3]; int step[3]; };
struct TilesArgs {
    int out_off[3];
    int rs[3], re[3], rst[3];   // assigned region in the target's own coordinates
    int lattice;                // 1: a DTile's bs/bw count points of the region's lattice (in place)
    LeafReg leaf[NLA];
};
#define TL_PER_THREAD 4

__device__ __forceinline__ T tiled_read(const Tiled& a, int g0, int g1, int g2) {
    const int t0 = g0 >> a.shift, t1 = g1 >> a.shift, t2 = g2 >> a.shift;
    const int lo0 = max(t0 << a.shift, a.off[0]);
    const int lo1 = max(t1 << a.shift, a.off[1]);
    const int lo2 = max(t2 << a.shift, a.off[2]);
    const int w1 = min((t1 + 1) << a.shift, a.off[1] + a.shape[1]) - lo1;
    const int w2 = min((t2 + 1) << a.shift, a.off[2] + a.shape[2]) - lo2;
    const int ti = ((t0 - a.glo[0]) * a.grid[1] + (t1 - a.glo[1])) * a.grid[2] + (t2 - a.glo[2]);
    const T* base = a.tiles[ti];
    const i64 s1 = a.py ? a.py : w2, s0 = a.py ? (i64)a.pz : (i64)w1 * w2;
    return base[(g0 - lo0) * s0 + (g1 - lo1) * s1 + (g2 - lo2)];
}

template <bool ROWS>
__device__ __forceinline__ void tiles_run(const Tiled* arrs, const DTile* dts, int ndt,
                                          const TilesArgs& ta, const T* s) {
    const int k = find_seg(dts, ndt, (i64)blockIdx.x);
    const DTile& dt = dts[k];
    const i64 blk = (i64)blockIdx.x - dt.blk0;
    const i64 group = blk / dt.nchunks;
    const int chunk = (int)(blk - group * dt.nchunks);
    int lanes = 256, lx = (int)threadIdx.x, i0, i1;
    if (ROWS) {
        // rows differ between the lanes of a workgroup: 32-bit arithmetic per lane
        lanes = 256 >> dt.rsh;
        lx = (int)threadIdx.x & (lanes - 1);
        const unsigned row = ((unsigned)group << dt.rsh) + ((unsigned)threadIdx.x >> (8 - dt.rsh));
        if (row >= (unsigned)dt.bw[0] * (unsigned)dt.bw[1]) return;
        const unsigned q = row / (unsigned)dt.bw[1];
        i0 = dt.bs[0] + (int)q;
        i1 = dt.bs[1] + (int)(row - q * (unsigned)dt.bw[1]);
    } else {
        i1 = dt.bs[1] + (int)(group % dt.bw[1]);
        i0 = dt.bs[0] + (int)(group / dt.bw[1]);
    }
    // in place: (i0, i1, i2) are indices into the region's lattice; otherwise tile coordinates
    const int a0 = ta.lattice ? ta.rs[0] + i0 * ta.rst[0] : dt.cs[0] + i0 - ta.out_off[0];
    const int a1 = ta.lattice ? ta.rs[1] + i1 * ta.rst[1] : dt.cs[1] + i1 - ta.out_off[1];
    const int l0 = a0 + ta.out_off[0] - dt.cs[0];
    const int l1 = a1 + ta.out_off[1] - dt.cs[1];
    const bool in01 = ta.lattice ||
                      (a0 >= ta.rs[0] && a0 < ta.re[0] && (a0 - ta.rs[0]) % ta.rst[0] == 0 &&
                       a1 >= ta.rs[1] && a1 < ta.re[1] && (a1 - ta.rs[1]) % ta.rst[1] == 0);
    const int k0 = ta.lattice ? i0 : (a0 - ta.rs[0]) / ta.rst[0];
    const int k1 = ta.lattice ? i1 : (a1 - ta.rs[1]) / ta.rst[1];
#pragma unroll
    for (int u = 0; u < TL_PER_THREAD; ++u) {
        const int j2 = chunk * (lanes * TL_PER_THREAD) + u * lanes + lx;
        if (j2 >= dt.bw[2]) continue;
        const int i2 = dt.bs[2] + j2;
        const int a2 = ta.lattice ? ta.rs[2] + i2 * ta.rst[2] : dt.cs[2] + i2 - ta.out_off[2];
        const int l2 = a2 + ta.out_off[2] - dt.cs[2];
        const i64 ds1 = dt.py ? dt.py : dt.w[2], ds0 = dt.py ? (i64)dt.pz : (i64)dt.w[1] * dt.w[2];
        const i64 di = l0 * ds0 + l1 * ds1 + l2;
        const bool inside = in01 && (ta.lattice || (a2 >= ta.rs[2] && a2 < ta.re[2] &&
                                                    (a2 - ta.rs[2]) % ta.rst[2] == 0));
        if (inside) {
            const int k2 = ta.lattice ? i2 : (a2 - ta.rs[2]) / ta.rst[2];
            T l[NLA], o[NOA];
#pragma unroll
            for (int q = 0; q < NL; ++q) {
                const LeafReg& lr = ta.leaf[q];
                const Tiled& a = arrs[lr.arr];
                l[q] = tiled_read(a, lr.start[0] + k0 * lr.step[0] + a.off[0],
                                  lr.start[1] + k1 * lr.step[1] + a.off[1],
                                  lr.start[2] + k2 * lr.step[2] + a.off[2]);
            }
            group_eval(l, s, o);
            dt.dst[di] = o[0];
        } else if (dt.cur != nullptr && dt.cur != dt.dst) {
            dt.dst[di] = dt.cur[di];
        }
    }
}

// ---- the same gather over arrays that are one row-major block each ----
// No tile table, no tile arithmetic: element (g0, g1, g2) of an array is base[g0 * pz + g1 * py + g2],
// so the part of an operand's address that belongs to a row is formed once per row and lane, and an
// element costs one multiply-add per operand. Every strided or shifted statement on arrays of rank
// 3, on rank-2 arrays with odd rows or ragged tile grids, and on single-tile arrays runs here.
struct BlockLeaf {
    const T* base; int py, pz; int start[3]; int step[3];
    int lim[3];                 // last index of the leaf's own region per dimension (scatter launches)
    int unused;
};
struct BlockArgs {
    T* dst; const T* cur;       // cur != dst: a sweep into a second buffer copies what it does not assign
    int shape[3]; int dpy, dpz; // the target (extents, elements between rows and planes)
    int rs[3], re[3], rst[3];   // assigned region
    int cnt[3];                 // points of its lattice per dimension
    int lattice;                // 1: in place, walk the lattice's points only
    int nchunks, rsh;           // chunks per row; 2^rsh rows share a workgroup
    int nroots;                 // scatter launches: the assigned lattices (same steps rst), else 0
    int nblk8;                  // launched workgroups / 8 (the launch is padded to a multiple of 8)
    int rrs[4][3], rcnt[4][3];  // first point and number of points of each of them
    int rmate[4];               // the lattice one element to the right on the same rows, stored with this
                                // one as a pair (-1: none; -2: this lattice is such a mate itself)
    BlockLeaf leaf[NLA];
};
// Consecutive workgroup ids go round the 8 XCDs: every XCD takes one contiguous eighth of the rows
// instead, so that the rows neighbouring workgroups both read (a stencil's, a restriction's, the
// coarse rows of a prolongation) are fetched into one L2 and not into two.
__device__ __forceinline__ unsigned block_order(const BlockArgs& a) {
    const unsigned b = blockIdx.x;
    return a.nblk8 ? (b & 7u) * (unsigned)a.nblk8 + (b >> 3) : b;
}
template <bool ROWS>
__device__ __forceinline__ void block_run(const BlockArgs& a, const T* s) {
    const int W0 = a.lattice ? a.cnt[0] : a.shape[0], W1 = a.lattice ? a.cnt[1] : a.shape[1];
    const int W2 = a.lattice ? a.cnt[2] : a.shape[2];
    const unsigned blk = block_order(a);
    const unsigned group = blk / (unsigned)a.nchunks;
    const int chunk = (int)(blk - group * (unsigned)a.nchunks);
    int lanes = 256, lx = (int)threadIdx.x;
    unsigned row = group;
    if (ROWS) {
        lanes = 256 >> a.rsh;
        lx = (int)threadIdx.x & (lanes - 1);
        row = (group << a.rsh) + ((unsigned)threadIdx.x >> (8 - a.rsh));
    }
    if (row >= (unsigned)W0 * (unsigned)W1) return;       // a ragged last group, or padding of the launch
    const int i0 = (int)(row / (unsigned)W1), i1 = (int)(row - (unsigned)i0 * (unsigned)W1);
    const int a0 = a.lattice ? a.rs[0] + i0 * a.rst[0] : i0;
    const int a1 = a.lattice ? a.rs[1] + i1 * a.rst[1] : i1;
    const bool in01 = a.lattice ||
                      (a0 >= a.rs[0] && a0 < a.re[0] && (a0 - a.rs[0]) % a.rst[0] == 0 &&
                       a1 >= a.rs[1] && a1 < a.re[1] && (a1 - a.rs[1]) % a.rst[1] == 0);
    const int k0 = a.lattice ? i0 : (in01 ? (a0 - a.rs[0]) / a.rst[0] : 0);
    const int k1 = a.lattice ? i1 : (in01 ? (a1 - a.rs[1]) / a.rst[1] : 0);
    i64 rowoff[NLA];
#pragma unroll
    for (int q = 0; q < NL; ++q) {
        const BlockLeaf& lf = a.leaf[q];
        rowoff[q] = (i64)(lf.start[0] + k0 * lf.step[0]) * lf.pz + (i64)(lf.start[1] + k1 * lf.step[1]) * lf.py +
                    lf.start[2];
    }
    const i64 drow = (i64)a0 * a.dpz + (i64)a1 * a.dpy;
#pragma unroll
    for (int u = 0; u < TL_PER_THREAD; ++u) {
        const int j2 = chunk * (lanes * TL_PER_THREAD) + u * lanes + lx;
        if (j2 >= W2) continue;
        const int a2 = a.lattice ? a.rs[2] + j2 * a.rst[2] : j2;
        const bool inside = in01 && (a.lattice || (a2 >= a.rs[2] && a2 < a.re[2] && (a2 - a.rs[2]) % a.rst[2] == 0));
        if (inside) {
            const int k2 = a.lattice ? j2 : (a2 - a.rs[2]) / a.rst[2];
            T l[NLA], o[NOA];
#pragma unroll
            for (int q = 0; q < NL; ++q)
                l[q] = a.leaf[q].base[rowoff[q] + (i64)k2 * a.leaf[q].step[2]];
            group_eval(l, s, o);
            a.dst[drow + a2] = o[0];
        } else if (a.cur != nullptr && a.cur != a.dst) {
            a.dst[drow + a2] = a.cur[drow + a2];
        }
    }
}
// The gather in place over unit steps along the rows (operands and target alike: shifted reads
// of several arrays, halos wider than the register-window kernels take): a lane moves pairs of
// neighbouring elements, as one 128-bit access each wherever that pair is (element-aligned), which
// halves the memory instructions per element. A row of odd length ends in a single element.
typedef T BP2 __attribute__((ext_vector_type(2)));
typedef BP2 BP2A __attribute__((aligned(sizeof(T))));
template <bool ROWS>
__device__ __forceinline__ void block_pairs(const BlockArgs& a, const T* s) {
    const int W0 = a.cnt[0], W1 = a.cnt[1], W2 = a.cnt[2];
    const unsigned blk = block_order(a);
    const unsigned group = blk / (unsigned)a.nchunks;
    const int chunk = (int)(blk - group * (unsigned)a.nchunks);
    int lanes = 256, lx = (int)threadIdx.x;
    unsigned row = group;
    if (ROWS) {
        lanes = 256 >> a.rsh;
        lx = (int)threadIdx.x & (lanes - 1);
        row = (group << a.rsh) + ((unsigned)threadIdx.x >> (8 - a.rsh));
    }
    if (row >= (unsigned)W0 * (unsigned)W1) return;
    const int k0 = (int)(row / (unsigned)W1), k1 = (int)(row - (unsigned)k0 * (unsigned)W1);
    const T* rowp[NLA];
#pragma unroll
    for (int q = 0; q < NL; ++q) {
        const BlockLeaf& lf = a.leaf[q];
        rowp[q] = lf.base + ((i64)(lf.start[0] + k0 * lf.step[0]) * lf.pz + (i64)(lf.start[1] + k1 * lf.step[1]) * lf.py +
                             lf.start[2]);
    }
    T* const drow = a.dst + ((i64)(a.rs[0] + k0 * a.rst[0]) * a.dpz + (i64)(a.rs[1] + k1 * a.rst[1]) * a.dpy + a.rs[2]);
#pragma unroll
    for (int u = 0; u < TL_PER_THREAD / 2; ++u) {
        const int k2 = 2 * (chunk * (lanes * (TL_PER_THREAD / 2)) + u * lanes + lx);
        if (k2 >= W2) continue;
        const bool two = k2 + 1 < W2;
        T l0[NLA], l1[NLA], o0[NOA], o1[NOA];
#pragma unroll
        for (int q = 0; q < NL; ++q) {
            if (two) {
                const BP2 v = *reinterpret_cast<const BP2A*>(rowp[q] + k2);
                l0[q] = v[0];
                l1[q] = v[1];
            } else {
                l0[q] = rowp[q][k2];
                l1[q] = l0[q];
            }
        }
        group_eval(l0, s, o0);
        group_eval(l1, s, o1);
        if (two)
            *reinterpret_cast<BP2A*>(drow + k2) = (BP2){o0[0], o1[0]};
        else
            drow[k2] = o0[0];
    }
}
extern "C" __global__ __launch_bounds__(256) void grp_block_pairs(BlockArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    block_pairs<false>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_block_pairs_rows(BlockArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    block_pairs<true>(a, s);
}
#if NO > 1 && NO <= 4
// Several statements that assign interleaved lattices of one array from other arrays (the four
// statements of a prolongation, examples/multigrid2d.py upstream) as one launch, in place: a lane
// takes one index (k0, k1, k2) of the lattices, evaluates every statement there and stores each
// result at its own lattice's point, rs_r + k * step. The lattices may differ in their number of
// points (cnt holds the largest per dimension): an index beyond a statement's own region reads that
// statement's operands at their last index instead, and stores nothing for it. Two lattices with a
// step of 2 along the rows whose points lie side by side on the same rows are stored as pairs.
template <bool ROWS>
__device__ __forceinline__ void block_scatter(const BlockArgs& a, const T* s) {
    const int W0 = a.cnt[0], W1 = a.cnt[1], W2 = a.cnt[2];
    const unsigned blk = block_order(a);
    const unsigned group = blk / (unsigned)a.nchunks;
    const int chunk = (int)(blk - group * (unsigned)a.nchunks);
    int lanes = 256, lx = (int)threadIdx.x;
    unsigned row = group;
    if (ROWS) {
        lanes = 256 >> a.rsh;
        lx = (int)threadIdx.x & (lanes - 1);
        row = (group << a.rsh) + ((unsigned)threadIdx.x >> (8 - a.rsh));
    }
    if (row >= (unsigned)W0 * (unsigned)W1) return;       // a ragged last group, or padding of the launch
    const int k0 = (int)(row / (unsigned)W1), k1 = (int)(row - (unsigned)k0 * (unsigned)W1);
    i64 rowoff[NLA];
#pragma unroll
    for (int q = 0; q < NL; ++q) {
        const BlockLeaf& lf = a.leaf[q];
        rowoff[q] = (i64)(lf.start[0] + min(k0, lf.lim[0]) * lf.step[0]) * lf.pz +
                    (i64)(lf.start[1] + min(k1, lf.lim[1]) * lf.step[1]) * lf.py + lf.start[2];
    }
    i64 drow[NO];
    bool rin[NO];
#pragma unroll
    for (int r = 0; r < NO; ++r) {
        rin[r] = k0 < a.rcnt[r][0] && k1 < a.rcnt[r][1];
        drow[r] = (i64)(a.rrs[r][0] + k0 * a.rst[0]) * a.dpz + (i64)(a.rrs[r][1] + k1 * a.rst[1]) * a.dpy + a.rrs[r][2];
    }
#pragma unroll
    for (int u = 0; u < TL_PER_THREAD; ++u) {
        const int k2 = chunk * (lanes * TL_PER_THREAD) + u * lanes + lx;
        if (k2 >= W2) continue;
        T l[NLA], o[NOA];
#pragma unroll
        for (int q = 0; q < NL; ++q)
            l[q] = a.leaf[q].base[rowoff[q] + (i64)min(k2, a.leaf[q].lim[2]) * a.leaf[q].step[2]];
        group_eval(l, s, o);
#pragma unroll
        for (int r = 0; r < NO; ++r) {
            const int m = a.rmate[r];
            if (!rin[r] || m == -2)
                continue;
            T* at = a.dst + drow[r] + (i64)k2 * a.rst[2];
            const bool own = k2 < a.rcnt[r][2];
            if (m < 0) {
                if (own)
                    at[0] = o[r];
                continue;
            }
            // two lattices side by side (the even and the odd columns of a prolongation's rows):
            // both values of a lane as one 128-bit store, wherever the pair lies
            T right = o[0];
            int rcount = a.rcnt[0][2];
#pragma unroll
            for (int w = 1; w < NO; ++w) {
                right = m == w ? o[w] : right;
                rcount = m == w ? a.rcnt[w][2] : rcount;
            }
            const bool other = k2 < rcount;
            if (own && other)
                *reinterpret_cast<BP2A*>(at) = (BP2){o[r], right};
            else if (own)
                at[0] = o[r];
            else if (other)
                at[1] = right;
        }
    }
}
extern "C" __global__ __launch_bounds__(256) void grp_scatter(BlockArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    block_scatter<false>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_scatter_rows(BlockArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    block_scatter<true>(a, s);
}
#endif
extern "C" __global__ __launch_bounds__(256) void grp_block(BlockArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    block_run<false>(a, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_block_rows(BlockArgs a, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    block_run<true>(a, s);
}

extern "C" __global__ __launch_bounds__(256) void grp_tiles(const Tiled* arrs, const DTile* dts,
                                                            int ndt, TilesArgs ta, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    tiles_run<false>(arrs, dts, ndt, ta, s);
}
extern "C" __global__ __launch_bounds__(256) void grp_tiles_rows(const Tiled* arrs, const DTile* dts,
                                                                 int ndt, TilesArgs ta, Scal sc) {
    CNH_ENTRY_GUARD T s[NSV]; load_scalars(sc, s);
    tiles_run<true>(arrs, dts, ndt, ta, s);
}
)";
    return s.str();
}

} // namespace

std::string slide_source(const GroupProgram& p, const SlideConfig& cfg, std::string& err); // codegen_slide.cpp

std::string direct_source(const GroupProgram& p, const DirectConfig& cfg, std::string& err); // codegen_direct.cpp

std::string DirectConfig::variant() const {
    char buf[64];
    snprintf(buf, sizeof buf, "direct%s@%d,%d,%d", reduce ? "r" : "", tx, ry, rz);
    return buf;
}

bool DirectConfig::parse(const std::string& variant, DirectConfig& out) {
    out = DirectConfig();
    if (variant == "direct")
        return true;
    if (variant == "directr") {
        out.reduce = true;
        return true;
    }
    if (sscanf(variant.c_str(), "directr@%d,%d,%d", &out.tx, &out.ry, &out.rz) == 3) {
        out.reduce = true;
        return true;
    }
    return sscanf(variant.c_str(), "direct@%d,%d,%d", &out.tx, &out.ry, &out.rz) == 3;
}

std::string SlideConfig::variant() const {
    char buf[96];
    snprintf(buf, sizeof buf, "slide@%d,%d,%d,%d,%d", march2d, bx, ry, zc, pd);
    return buf;
}

bool SlideConfig::parse(const std::string& variant, SlideConfig& out) {
    out = SlideConfig();
    if (variant == "slide")
        return true;
    return sscanf(variant.c_str(), "slide@%d,%d,%d,%d,%d", &out.march2d, &out.bx, &out.ry, &out.zc,
                  &out.pd) == 5;
}

int emit_variant_source(const GroupProgram& p, const std::string& variant, std::string& src,
                        std::string& err) {
    if (p.out_roots.empty()) {
        err = "group has no output root";
        return -16;
    }
    if (variant == "prelude") {
        src = prelude(p);
        return 0;
    }
    if (variant == "flat") {
        src = flat_source(p);
        return 0;
    }
    if (p.reductions() > 0) {
        err = "a group with reducing roots runs over dense, equally laid out operands only";
        return -17;
    }
    if (variant == "nd") {
        src = nd_source(p);
        return 0;
    }
    if (variant.compare(0, 7, "product") == 0) {
        // "product<q>" + form: "" two sets of eight wavefronts, "e" eight wavefronts, "f" four
        const int q = variant.size() >= 8 ? variant[7] - '0' : 0;
        const int form = variant.size() == 8 ? 1 : variant.size() == 9 && variant[8] == 'e' ? 2
                         : variant.size() == 9 && variant[8] == 'f' ? 3 : 0;
        if ((q != 1 && q != 2 && q != 4) || form == 0) {
            err = "the product variant is product<1|2|4>[e|f] (column blocks per product, form of the kernel)";
            return -2;
        }
        if (p.dtype != CNH_F64) {
            err = "statements in a product's epilogue are fp64 only";
            return -17;
        }
        src = product_source(p, q, form);
        return 0;
    }
    if (variant == "tiles") {
        // one output root, or up to four SET_REGION roots (the scatter kernels of this variant;
        // its other kernels store the first root only, and the launch never picks them then)
        if (p.out_roots.size() > 4) {
            err = "the tiled variant takes one to four output roots";
            return -17;
        }
        src = tiles_source(p);
        return 0;
    }
    if (variant.compare(0, 6, "direct") == 0) {
        DirectConfig cfg;
        if (!DirectConfig::parse(variant, cfg)) {
            err = "malformed register-window variant '" + variant + "'";
            return -2;
        }
        src = direct_source(p, cfg, err);
        return src.empty() ? -18 : 0;
    }
    if (variant.compare(0, 5, "slide") == 0) {
        SlideConfig cfg;
        if (!SlideConfig::parse(variant, cfg)) {
            err = "malformed sliding-window variant '" + variant + "'";
            return -2;
        }
        src = slide_source(p, cfg, err);
        return src.empty() ? -18 : 0;
    }
    err = "unknown kernel variant '" + variant + "'";
    return -2;
}

} // namespace cnh
