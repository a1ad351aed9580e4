// Fused-group kernels: hipRTC build, cache and launch.
// Stands in for ArrayDAGGroup::compile_node (src/dag_group_compile.cpp:6-56 upstream) and
// dispatch_kernel<N,T> (src/dispatch.hpp:137-265): same argument order (memref per leaf use,
// scalar per broadcast leaf, memref per non-temp root), but all partitions of a node go into
// one launch and broadcast scalars may stay on the device.
#include "codegen.h"

#include <hip/hiprtc.h>

#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

using namespace cnh;

// Code object of one generated source text. Kernels whose variants generate the same text (the
// same group at another place of an array: regions travel as launch arguments) share it, so a
// time loop over slabs compiles once. Code objects live as long as the library.
struct CodeObject {
    std::string src;
    std::vector<char> code;
    std::mutex mu;                 // guards mod and fns: code objects are shared between kernels
    hipModule_t mod = nullptr;
    std::map<std::string, hipFunction_t> fns;
};

struct KernelVariant {
    std::string src;
    std::shared_ptr<CodeObject> obj;
};

struct cnh_kernel {
    GroupProgram prog;
    uint64_t key = 0;
    int refs = 1;
    std::string ident;             // the AST it was compiled from, field by field (see ast_ident)
    std::mutex mu;                 // guards variants: a kernel found by key is shared between executors
    std::map<std::string, KernelVariant> variants;
    // whether and how the group fits the register-window kernels, worked out once per geometry
    // (every launch asks; the answer depends on the program and the three numbers only)
    bool shape_known = false;
    int shape_cfg[3] = {0, 0, 0}, shape_rc = 0;
    DirectShape shape;
};

namespace {

std::mutex g_kmu;
std::map<uint64_t, cnh_kernel*> g_kernels; // key -> kernel (key 0 = not cached)
std::multimap<uint64_t, std::shared_ptr<CodeObject>> g_code; // hash of the source text -> code object
std::mutex g_cmu;                                             // guards g_code

uint64_t text_hash(const std::string& t) {
    uint64_t h = 1469598103934665603ull;
    for (unsigned char c : t) {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

// Everything of an AST that decides the generated code, as bytes: what a cache key stands for.
std::string ast_ident(const cnh_ast* ast, int dtype, int ndims) {
    std::string out;
    auto put = [&](const void* p, size_t n) { out.append(static_cast<const char*>(p), n); };
    auto put_region = [&](const cnh_region& r) {
        const int32_t v[11] = {r.is_global, r.ndims,   r.start[0], r.start[1], r.start[2], r.stop[0],
                               r.stop[1],   r.stop[2], r.step[0],  r.step[1],  r.step[2]};
        put(v, sizeof v);
    };
    const int32_t head[4] = {dtype, ndims, ast->n_nodes, ast->n_roots};
    put(head, sizeof head);
    for (int i = 0; i < ast->n_nodes; ++i) {
        const cnh_ast_node& a = ast->nodes[i];
        const int32_t f[12] = {a.result_name, a.opcode,      a.is_temp,     a.is_scalar,
                               a.is_broadcast, a.ndims,      a.dtype,       a.n_operands,
                               a.operands[0], a.operands[1], a.has_operand_region[0], a.has_operand_region[1]};
        put(f, sizeof f);
        put(&a.scalar, sizeof a.scalar);
        put_region(a.operand_regions[0]);
        put_region(a.operand_regions[1]);
        put_region(a.region);
    }
    put(ast->roots, sizeof(int32_t) * (size_t)ast->n_roots);
    return out;
}

// Code objects on disk, across processes: off unless CHARMNUMERIC_KERNEL_CACHE names a directory.
// One file per code object, named by the hash of the generated text and holding that text in
// full (compared before the code is trusted) next to the compiler's version; written under a
// temporary name and renamed, so a reader never sees half a file. Any failure here just means
// compiling as usual.
std::string disk_cache_path(uint64_t h) {
    const char* dir = std::getenv("CHARMNUMERIC_KERNEL_CACHE");
    if (dir == nullptr || dir[0] == '\0')
        return std::string();
    int major = 0, minor = 0;
    hiprtcVersion(&major, &minor);
    char name[96];
    std::snprintf(name, sizeof name, "/cnh-gfx950-rtc%d.%d-%016llx.co", major, minor, (unsigned long long)h);
    return std::string(dir) + name;
}

bool disk_cache_load(uint64_t h, const std::string& src, std::vector<char>& code) {
    const std::string path = disk_cache_path(h);
    if (path.empty())
        return false;
    FILE* f = std::fopen(path.c_str(), "rb");
    if (f == nullptr)
        return false;
    bool ok = false;
    uint64_t head[3] = {0, 0, 0};   // magic, text bytes, code bytes
    if (std::fread(head, sizeof head, 1, f) == 1 && head[0] == 0x314f43484e43ull && head[1] == src.size() &&
        head[2] > 0 && head[2] < (1ull << 30)) {
        std::string text(head[1], '\0');
        code.resize(head[2]);
        ok = std::fread(&text[0], 1, text.size(), f) == text.size() && text == src &&
             std::fread(code.data(), 1, code.size(), f) == code.size();
    }
    std::fclose(f);
    return ok;
}

void disk_cache_store(uint64_t h, const std::string& src, const std::vector<char>& code) {
    const std::string path = disk_cache_path(h);
    if (path.empty())
        return;
    char tmp_tail[48];
    std::snprintf(tmp_tail, sizeof tmp_tail, ".tmp%ld", (long)getpid());
    const std::string tmp = path + tmp_tail;
    FILE* f = std::fopen(tmp.c_str(), "wb");
    if (f == nullptr)
        return;
    const uint64_t head[3] = {0x314f43484e43ull, src.size(), code.size()};
    const bool ok = std::fwrite(head, sizeof head, 1, f) == 1 &&
                    std::fwrite(src.data(), 1, src.size(), f) == src.size() &&
                    std::fwrite(code.data(), 1, code.size(), f) == code.size();
    if (std::fclose(f) != 0 || !ok || std::rename(tmp.c_str(), path.c_str()) != 0)
        std::remove(tmp.c_str());
}

int64_t g_disk_hits = 0;

int build_variant(cnh_kernel* k, const std::string& variant, KernelVariant** out) {
    std::lock_guard<std::mutex> kernel_lock(k->mu);
    auto it = k->variants.find(variant);
    if (it != k->variants.end() && it->second.obj) {
        *out = &it->second;
        return 0;
    }
    KernelVariant& v = k->variants[variant];
    if (v.src.empty()) {
        // "variant#entry": the variant's text built for that one entry point only
        const size_t hash_at = variant.find('#');
        const std::string base = variant.substr(0, hash_at);
        std::string err;
        int rc = emit_variant_source(k->prog, base, v.src, err);
        if (rc) {
            k->variants.erase(variant);
            return set_error(rc, "codegen(%s): %s", variant.c_str(), err.c_str());
        }
        if (hash_at != std::string::npos)
            v.src = "#define CNH_ONLY_NAME \"" + variant.substr(hash_at + 1) + "\"\n" + v.src;
    }
    const uint64_t h = text_hash(v.src);
    std::lock_guard<std::mutex> code_lock(g_cmu);
    {
        auto range = g_code.equal_range(h);
        for (auto c = range.first; c != range.second; ++c)
            if (c->second->src == v.src) {
                v.obj = c->second;
                *out = &v;
                return 0;
            }
    }
    {
        auto cached = std::make_shared<CodeObject>();
        if (disk_cache_load(h, v.src, cached->code)) {
            cached->src = v.src;
            g_code.emplace(h, cached);
            ++g_disk_hits;
            v.obj = cached;
            *out = &v;
            return 0;
        }
    }
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, v.src.c_str(), "cnh_group.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS)
        return set_error(-110, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    // No FMA contraction: the upstream group is a chain of separately rounded IEEE operations.
    const char* opts[] = {"--offload-arch=gfx950", "-O3",     "-ffp-contract=off",
                          "-Xclang",               "-target-feature", "-Xclang",
                          "-packed-fp32-ops",      "-std=c++17"};
    r = hiprtcCompileProgram(prog, (int)(sizeof opts / sizeof opts[0]), opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n)
            hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        return set_error(-111, "hiprtc compile failed (%s):\n%s", hiprtcGetErrorString(r),
                         log.c_str());
    }
    size_t cs = 0;
    hiprtcGetCodeSize(prog, &cs);
    auto obj = std::make_shared<CodeObject>();
    obj->src = v.src;
    obj->code.resize(cs);
    hiprtcGetCode(prog, obj->code.data());
    hiprtcDestroyProgram(&prog);
    disk_cache_store(h, obj->src, obj->code);
    g_code.emplace(h, obj);
    v.obj = obj;
    *out = &v;
    return 0;
}

int get_function(cnh_kernel* k, const std::string& variant, const char* name, hipFunction_t* fn) {
    KernelVariant* v = nullptr;
    // a launch builds the variant for the one entry point it needs (a variant has up to ten, each
    // a kernel of its own to optimise: 0.1-0.9 s instead of 0.35-3.2 s at first use)
    if (int rc = build_variant(k, variant + "#" + name, &v))
        return rc;
    CodeObject* c = v->obj.get();
    std::lock_guard<std::mutex> object_lock(c->mu);
    if (!c->mod)
        CNH_HIP(hipModuleLoadData(&c->mod, c->code.data()));
    auto it = c->fns.find(name);
    if (it == c->fns.end()) {
        hipFunction_t f;
        CNH_HIP(hipModuleGetFunction(&f, c->mod, name));
        it = c->fns.emplace(name, f).first;
    }
    *fn = it->second;
    return 0;
}

// Scal { const T* p[NSA]; T v[NSA]; T c[NLITA]; } as the generated code lays it out: broadcast
// scalars by pointer or by value, then the literal scalars the source takes as parameters.
int pack_scalars(const GroupProgram& p, int n_scalar, const void* const* scalars, int on_device,
                 std::vector<unsigned char>& buf) {
    int ns = (int)p.bcast_nodes.size();
    CNH_CHECK(n_scalar == ns, -4, "group expects %d broadcast scalars, got %d", ns, n_scalar);
    int nsa = ns > 0 ? ns : 1;
    int esz = dtype_size(p.dtype);
    const int nlit = (int)p.lit_values.size(), nlita = nlit > 0 ? nlit : 1;
    size_t bytes = (size_t)nsa * 8 + (size_t)nsa * esz + (size_t)nlita * esz;
    bytes = (bytes + 7) & ~size_t(7);
    buf.assign(bytes, 0);
    for (int i = 0; i < nlit; ++i)
        literal_value(p.dtype, p.lit_values[(size_t)i], &buf[(size_t)nsa * 8 + (size_t)(nsa + i) * esz]);
    for (int i = 0; i < ns; ++i) {
        CNH_CHECK(scalars && scalars[i], -4, "broadcast scalar %d is null", i);
        if (on_device) {
            const void* ptr = scalars[i];
            std::memcpy(&buf[(size_t)i * 8], &ptr, 8);
        } else {
            std::memcpy(&buf[(size_t)nsa * 8 + (size_t)i * esz], scalars[i], esz);
        }
    }
    return 0;
}

bool dense_memref(int nd, const cnh_memref& m) {
    int64_t expect = 1;
    for (int d = nd - 1; d >= 0; --d) {
        if (m.sizes[d] != 1 && m.strides[d] != expect)
            return false;
        expect *= m.sizes[d];
    }
    return true;
}

int launch(hipFunction_t fn, int64_t blocks, void** params, hipStream_t st, unsigned lanes = 256) {
    CNH_CHECK(blocks > 0 && blocks < (1ll << 31), -3, "launch of %lld workgroups is out of range",
              (long long)blocks);
    CNH_HIP(hipModuleLaunchKernel(fn, (unsigned)blocks, 1, 1, lanes, 1, 1, 0, st, params, nullptr));
    return 0;
}

} // namespace

extern "C" {

int cnh_compile_group(const cnh_ast* ast, int dtype, int ndims, uint64_t key, cnh_kernel** out) {
    CNH_CHECK(out != nullptr, -2, "cnh_compile_group: null output");
    CNH_CHECK(ast != nullptr && ast->nodes != nullptr && ast->roots != nullptr && ast->n_nodes > 0 &&
                  ast->n_roots > 0,
              -2, "cnh_compile_group: empty AST");
    std::string ident = ast_ident(ast, dtype, ndims);
    std::lock_guard<std::mutex> lk(g_kmu);
    if (key != 0) {
        auto it = g_kernels.find(key);
        if (it != g_kernels.end()) {
            if (it->second->ident == ident) {
                it->second->refs++;
                *out = it->second;
                return 0;
            }
            key = 0;   // two different groups under one key: this one is compiled and kept apart
        }
    }
    cnh_kernel* k = new cnh_kernel;
    k->ident = std::move(ident);
    std::string err;
    int rc = build_group_program(ast, dtype, ndims, k->prog, err);
    if (rc) {
        delete k;
        return set_error(rc, "cnh_compile_group: %s", err.c_str());
    }
    k->key = key;
    if (key != 0)
        g_kernels[key] = k; // found again by key while somebody holds it; gone with its last user
    *out = k;
    return 0;
}

int cnh_kernel_matches(const cnh_kernel* k, const cnh_ast* ast, int dtype, int ndims) {
    if (k == nullptr || ast == nullptr || ast->nodes == nullptr || ast->roots == nullptr)
        return 0;
    return k->ident == ast_ident(ast, dtype, ndims) ? 1 : 0;
}

int cnh_kernel_release(cnh_kernel* k) {
    if (!k)
        return 0;
    std::lock_guard<std::mutex> lk(g_kmu);
    if (--k->refs > 0)
        return 0;
    if (k->key != 0)
        g_kernels.erase(k->key);
    delete k;
    return 0;
}

int cnh_kernel_signature(const cnh_kernel* k, int* n_in, int* n_scalar, int* n_out) {
    CNH_CHECK(k != nullptr, -2, "null kernel");
    if (n_in)
        *n_in = (int)k->prog.leaves.size();
    if (n_scalar)
        *n_scalar = (int)k->prog.bcast_nodes.size();
    if (n_out)
        *n_out = (int)k->prog.out_roots.size();
    return 0;
}

int cnh_kernel_input(const cnh_kernel* k, int i, int* name, int* has_region, cnh_region* region) {
    CNH_CHECK(k != nullptr, -2, "null kernel");
    CNH_CHECK(i >= 0 && i < (int)k->prog.leaves.size(), -2, "input index %d out of range", i);
    const LeafUse& u = k->prog.leaves[i];
    if (name)
        *name = u.name;
    if (has_region)
        *has_region = u.has_region ? 1 : 0;
    if (region)
        *region = u.region;
    return 0;
}

int cnh_kernel_scalar(const cnh_kernel* k, int i, int* name) {
    CNH_CHECK(k != nullptr, -2, "null kernel");
    CNH_CHECK(i >= 0 && i < (int)k->prog.bcast_names.size(), -2, "scalar index %d out of range", i);
    if (name)
        *name = k->prog.bcast_names[i];
    return 0;
}

int cnh_kernel_output(const cnh_kernel* k, int i, int* result_name, int* target_name,
                      int* is_set_region, cnh_region* region) {
    CNH_CHECK(k != nullptr, -2, "null kernel");
    CNH_CHECK(i >= 0 && i < (int)k->prog.out_roots.size(), -2, "output index %d out of range", i);
    if (result_name)
        *result_name = k->prog.out_names[i];
    if (target_name)
        *target_name = k->prog.out_target[i];
    if (is_set_region)
        *is_set_region = k->prog.out_is_set_region[i];
    if (region)
        *region = k->prog.out_region[i];
    return 0;
}

int64_t cnh_kernel_source(cnh_kernel* k, const char* variant, char* buf, size_t cap) {
    CNH_CHECK(k != nullptr && variant != nullptr, -2, "null argument");
    KernelVariant& v = k->variants[variant];
    if (v.src.empty()) {
        std::string err;
        int rc = emit_variant_source(k->prog, variant, v.src, err);
        if (rc) {
            k->variants.erase(variant);
            return set_error(rc, "codegen(%s): %s", variant, err.c_str());
        }
    }
    if (buf && cap > 0) {
        size_t n = v.src.size() < cap - 1 ? v.src.size() : cap - 1;
        std::memcpy(buf, v.src.data(), n);
        buf[n] = '\0';
    }
    return (int64_t)v.src.size() + 1;
}

int cnh_kernel_variants_loaded(const cnh_kernel* k, const char* prefix) {
    CNH_CHECK(k != nullptr && prefix != nullptr, -2, "null argument");
    int n = 0;
    for (const auto& kv : k->variants)
        if (kv.second.obj && kv.first.compare(0, std::strlen(prefix), prefix) == 0)
            ++n;
    return n;
}

int cnh_kernel_lattice(const cnh_kernel* k) {
    if (k == nullptr)
        return 0;
    DirectShape sh;
    std::string why;
    if (direct_shape(k->prog, DirectConfig(), sh, why) != 0 || !sh.lattice)
        return 0;
    return sh.inplace_safe ? 2 : 1;
}

int cnh_kernel_build(cnh_kernel* k, const char* variant) {
    CNH_CHECK(k != nullptr && variant != nullptr, -2, "null argument");
    KernelVariant* v = nullptr;
    return build_variant(k, variant, &v);
}

} // extern "C"

// A launch streams past the caches (non-temporal loads and stores) when the arrays it touches
// exceed what the 256 MiB last-level cache can hold from one launch to the next; below that the
// next statement of a loop finds its operands there. Measured on MI355X with the arrays of a loop
// adding up to 144 .. 384 MiB: cached 3-7 % faster up to 288 MiB, non-temporal 10 % faster at 384.
int g_flat_nt_mib = 272;
// The same for sweeps, where it matters more: a Jacobi sweep between two 134 MB buffers (4097^2)
// takes 42 us with cached stores and 61.5 us with non-temporal ones; with a third array (402 MB in
// all) 79.9 against 69.7 us; at 303 MB and above non-temporal wins by 3-8 %.
int g_stencil_nt_mib = 272;
namespace {
// The memref launch. `sums` (or null): per run-time scalar, how many partial sums stand behind its
// address and where the folded value is to be stored.
int launch_group_impl(cnh_kernel* k, int ndims, int n_parts, int n_in, const cnh_memref* in,
                      int n_scalar, const void* const* scalars, int scalars_on_device,
                      const cnh_scalar_sum* sums, int n_out, const cnh_memref* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(k != nullptr, -2, "null kernel");
    const GroupProgram& p = k->prog;
    CNH_CHECK(ndims == p.ndims, -4, "kernel was compiled for rank %d, launched with %d", p.ndims,
              ndims);
    CNH_CHECK(n_in == (int)p.leaves.size(), -4, "group expects %d input memrefs, got %d",
              (int)p.leaves.size(), n_in);
    CNH_CHECK(n_out == (int)p.out_roots.size(), -4, "group expects %d output memrefs, got %d",
              (int)p.out_roots.size(), n_out);
    CNH_CHECK(n_parts >= 0, -2, "negative partition count");
    CNH_CHECK(n_out >= 1 && out != nullptr, -2, "a group needs at least one output memref");
    CNH_CHECK(n_in == 0 || in != nullptr, -2, "null input memrefs");
    std::vector<unsigned char> scal;
    if (int rc = pack_scalars(p, n_scalar, scalars, scalars_on_device, scal))
        return rc;

    const int NL = (int)p.load_leaf.size();
    const int NLA = NL > 0 ? NL : 1, NOA = n_out;
    const int esz = dtype_size(p.dtype);
    const int vec = 16 / esz;

    // Outputs that are reduced over the launch (CNH_OP_SUM_OF / CNH_OP_MAXABS_OF roots): their
    // memref names the one element the result goes to (partition 0's counts); `e0` is the first
    // output that is stored element by element, whose extents every other memref must match.
    const int n_red = p.folds();
    auto folds = [&](int o) { return p.out_reduce[(size_t)o] == 1 || p.out_reduce[(size_t)o] == 2; };
    int e0 = -1;
    for (int o = 0; o < n_out; ++o)
        if (!p.out_reduce[(size_t)o]) {
            e0 = o;
            break;
        }
    CNH_CHECK(e0 >= 0, -4, "a group needs an output that is stored element by element");
    CNH_CHECK(n_red <= kFoldMaxVectors, -4, "%d reducing roots in one group (at most %d)", n_red,
              kFoldMaxVectors);

    // Shapes must agree across all memrefs of a partition (identity indexing maps upstream).
    bool all_dense = true, all_aligned = true;
    std::vector<int> live;
    for (int q = 0; q < n_parts; ++q) {
        const cnh_memref* pi = in + (size_t)q * n_in;
        const cnh_memref* po = out + (size_t)q * n_out;
        int64_t total = 1;
        for (int d = 0; d < ndims; ++d) {
            CNH_CHECK(po[e0].sizes[d] >= 0, -4, "negative extent");
            total *= po[e0].sizes[d];
        }
        if (total == 0)
            continue;
        live.push_back(q);
        for (int i = 0; i < n_in + n_out; ++i) {
            const cnh_memref& m = i < n_in ? pi[i] : po[i - n_in];
            CNH_CHECK(m.aligned != nullptr, -4, "partition %d: memref %d has a null pointer", q, i);
            if (i >= n_in && p.out_reduce[(size_t)(i - n_in)])
                continue;
            for (int d = 0; d < ndims; ++d)
                CNH_CHECK(m.sizes[d] == po[e0].sizes[d], -4,
                          "partition %d: memref %d extent %lld differs from the output's %lld in "
                          "dim %d",
                          q, i, (long long)m.sizes[d], (long long)po[e0].sizes[d], d);
            if (!dense_memref(ndims, m))
                all_dense = false;
            uintptr_t addr = (uintptr_t)m.aligned + (uintptr_t)(m.offset * esz);
            if (addr & 15)
                all_aligned = false;
        }
    }
    if (live.empty())
        return 0;
    hipStream_t st = as_stream(s);
    auto base_ptr = [&](const cnh_memref& m) -> uint64_t {
        return (uint64_t)((uintptr_t)m.aligned + (uintptr_t)(m.offset * esz));
    };

    if (all_dense) {
        // the generated code's FLAT_WG: one wavefront per workgroup unless the launch reduces or
        // sums partials on the way in (those kernels share values between four wavefronts)
        const unsigned lanes = (n_red > 0 || sums != nullptr) ? 256 : 64;
        const int per_block = (int)lanes * vec;
        const size_t seg_words = 2 + NLA + NOA;
        std::vector<uint64_t> segs(seg_words * live.size(), 0);
        int64_t blocks = 0, total = 0;
        for (size_t j = 0; j < live.size(); ++j) {
            int q = live[j];
            const cnh_memref* pi = in + (size_t)q * n_in;
            const cnh_memref* po = out + (size_t)q * n_out;
            int64_t n = 1;
            for (int d = 0; d < ndims; ++d)
                n *= po[e0].sizes[d];
            uint64_t* sg = &segs[j * seg_words];
            sg[0] = (uint64_t)n;
            sg[1] = (uint64_t)blocks;
            for (int l = 0; l < NL; ++l)
                sg[2 + l] = base_ptr(pi[p.load_leaf[l]]);
            for (int o = 0; o < n_out; ++o)
                sg[2 + NLA + o] = base_ptr(po[o]);
            blocks += (n + per_block - 1) / per_block;
            total += n;
        }
        // Streams larger than the last-level cache bypass it; small operands (CG vectors) stay.
        const bool nontemporal = total * (int64_t)(NL + n_out) * esz >= ((int64_t)g_flat_nt_mib << 20);
        const char* suffix = !all_aligned ? "s" : nontemporal ? "vn" : "v";
        std::string name = std::string(live.size() == 1 ? "grp_flat1_" : "grp_flat_") + suffix;
        hipFunction_t fn;
        if (int rc = get_function(k, "flat", name.c_str(), &fn))
            return rc;
        // Reducing roots: one partial per workgroup and reduction. A reduction whose output memref
        // names more than one element keeps its partials there (the caller, or a later launch that
        // takes them as a summed scalar, folds them; entries past the last workgroup are left as
        // they are). The others go to the stream's workspace and are folded right after the launch.
        const int64_t nslots = blocks;
        void* red_slots[kFoldMaxVectors] = {nullptr, nullptr, nullptr, nullptr};
        int maximum[kFoldMaxVectors] = {0, 0, 0, 0}, n_fold = 0;
        double* fold_vec[kFoldMaxVectors] = {nullptr, nullptr, nullptr, nullptr};
        double* fold_out[kFoldMaxVectors] = {nullptr, nullptr, nullptr, nullptr};
        if (n_red > 0) {
            CNH_CHECK(p.dtype == CNH_F64, -27, "reducing roots need an fp64 group");
            const cnh_memref* po = out + (size_t)live[0] * n_out;
            int kept = 0, q = 0;
            for (int o = 0; o < n_out; ++o)
                if (folds(o)) {
                    int64_t room = 1;
                    for (int d = 0; d < ndims; ++d)
                        room *= po[o].sizes[d];
                    if (room > 1) {
                        CNH_CHECK(room >= nslots, -4, "output %d has room for %lld partial results, the launch "
                                  "leaves %lld", o, (long long)room, (long long)nslots);
                        red_slots[q] = reinterpret_cast<void*>((uintptr_t)base_ptr(po[o]));
                        ++kept;
                    }
                    ++q;
                }
            if (kept < n_red) {
                const int64_t stride = nslots + kFoldRuns;   // the fold keeps its run sums behind each vector
                void* ws = nullptr;
                if (int rc = reduce_workspace(st, (size_t)(stride * (n_red - kept)) * sizeof(double), &ws))
                    return rc;
                q = 0;
                for (int o = 0; o < n_out; ++o)
                    if (folds(o)) {
                        if (red_slots[q] == nullptr) {
                            red_slots[q] = static_cast<double*>(ws) + stride * n_fold;
                            maximum[n_fold] = p.out_reduce[(size_t)o] == 2;
                            fold_vec[n_fold] = static_cast<double*>(red_slots[q]);
                            fold_out[n_fold] = reinterpret_cast<double*>((uintptr_t)base_ptr(po[o]));
                            ++n_fold;
                        }
                        ++q;
                    }
            }
        }
        if (sums != nullptr) {
            CNH_CHECK(live.size() == 1, -28, "summed scalars go with launches over one partition");
            const int NS = (int)p.bcast_nodes.size(), NSA = NS > 0 ? NS : 1;
            // Fold { T* out[NSA]; int n[NSA]; } as the generated code lays it out
            std::vector<unsigned char> fold(((size_t)NSA * 12 + 7) & ~size_t(7), 0);
            for (int i = 0; i < NS; ++i) {
                CNH_CHECK(sums[i].count >= 1 && sums[i].count <= (1 << 20), -4,
                          "scalar %d: %lld partial sums", i, (long long)sums[i].count);
                const void* fo = sums[i].folded;
                const int32_t cnt = (int32_t)sums[i].count;
                std::memcpy(&fold[(size_t)i * 8], &fo, 8);
                std::memcpy(&fold[(size_t)NSA * 8 + (size_t)i * 4], &cnt, 4);
            }
            hipFunction_t ffn;
            if (int rc = get_function(k, "flat", (std::string("grp_flat1f_") + suffix).c_str(), &ffn))
                return rc;
            void* params[] = {segs.data(), scal.data(), fold.data(), red_slots};
            if (int rc = launch(ffn, blocks, params, st, 256))
                return rc;
        } else if (live.size() == 1) {
            void* params[] = {segs.data(), scal.data(), red_slots};
            if (int rc = launch(fn, blocks, params, st, lanes))
                return rc;
        } else {
            const void* dsegs = nullptr;
            if (int rc = desc_upload(segs.data(), segs.size() * 8, st, &dsegs))
                return rc;
            int nseg = (int)live.size();
            void* params[] = {&dsegs, &nseg, scal.data(), red_slots};
            if (int rc = launch(fn, blocks, params, st, lanes))
                return rc;
        }
        if (n_fold == 0)
            return 0;
        return reduce_slots_f64_many(n_fold, maximum, fold_vec, nslots, fold_out, st);
    }
    CNH_CHECK(sums == nullptr, -28, "summed scalars need dense, equally laid out operands");
    CNH_CHECK(p.reductions() == 0, -28, "a group with reducing or scalar roots needs dense, equally laid out operands");

    // Strided cells.
    const size_t cell_words = 5 + NLA + 3 * NLA + NOA + 3 * NOA;
    std::vector<int64_t> cells(cell_words * live.size(), 0);
    int64_t blocks = 0;
    const int pad = CNH_MAX_ND - ndims;
    // elements per lane: 4 for large launches, 1 when that still leaves few wavefronts per SIMD
    int64_t all_elems = 0;
    for (size_t j = 0; j < live.size(); ++j) {
        int64_t n = 1;
        for (int d = 0; d < ndims; ++d)
            n *= out[(size_t)live[j] * n_out].sizes[d];
        all_elems += n;
    }
    const int per_lane = all_elems <= (1ll << 21) ? 1 : 4;
    const unsigned nd_lanes = per_lane == 1 ? 64 : 256;      // as the generated entry points are built
    for (size_t j = 0; j < live.size(); ++j) {
        int q = live[j];
        const cnh_memref* pi = in + (size_t)q * n_in;
        const cnh_memref* po = out + (size_t)q * n_out;
        int64_t* c = &cells[j * cell_words];
        int64_t sz[3] = {1, 1, 1};
        for (int d = 0; d < ndims; ++d)
            sz[pad + d] = po[0].sizes[d];
        int64_t nchunks = (sz[2] + nd_lanes * per_lane - 1) / (nd_lanes * per_lane);
        c[0] = sz[0];
        c[1] = sz[1];
        c[2] = sz[2];
        c[3] = blocks;
        c[4] = nchunks;
        int64_t* cin = c + 5;
        int64_t* cistr = cin + NLA;
        int64_t* cout = cistr + 3 * NLA;
        int64_t* costr = cout + NOA;
        for (int l = 0; l < NL; ++l) {
            const cnh_memref& m = pi[p.load_leaf[l]];
            cin[l] = (int64_t)base_ptr(m);
            for (int d = 0; d < ndims; ++d)
                cistr[l * 3 + pad + d] = m.strides[d];
        }
        for (int o = 0; o < n_out; ++o) {
            cout[o] = (int64_t)base_ptr(po[o]);
            for (int d = 0; d < ndims; ++d)
                costr[o * 3 + pad + d] = po[o].strides[d];
        }
        blocks += sz[0] * sz[1] * nchunks;
    }
    hipFunction_t fn;
    if (live.size() == 1) {
        if (int rc = get_function(k, "nd", per_lane == 1 ? "grp_nd1_p1" : "grp_nd1", &fn))
            return rc;
        void* params[] = {cells.data(), scal.data()};
        return launch(fn, blocks, params, st, nd_lanes);
    }
    if (int rc = get_function(k, "nd", per_lane == 1 ? "grp_nd_p1" : "grp_nd", &fn))
        return rc;
    const void* dcells = nullptr;
    if (int rc = desc_upload(cells.data(), cells.size() * 8, st, &dcells))
        return rc;
    int ncell = (int)live.size();
    void* params[] = {&dcells, &ncell, scal.data()};
    return launch(fn, blocks, params, st, nd_lanes);
}

} // namespace

extern "C" {

int cnh_launch_group_batched(cnh_kernel* k, int ndims, int n_parts, int n_in, const cnh_memref* in,
                             int n_scalar, const void* const* scalars, int scalars_on_device,
                             int n_out, const cnh_memref* out, cnh_stream s) {
    return launch_group_impl(k, ndims, n_parts, n_in, in, n_scalar, scalars, scalars_on_device, nullptr,
                             n_out, out, s);
}

int cnh_launch_group_sums(cnh_kernel* k, int ndims, int n_in, const cnh_memref* in, int n_scalar,
                          const cnh_scalar_sum* scalars, int n_out, const cnh_memref* out, cnh_stream s) {
    CNH_CHECK(n_scalar == 0 || scalars != nullptr, -2, "null scalars");
    std::vector<const void*> ptrs((size_t)std::max(1, n_scalar), nullptr);
    for (int i = 0; i < n_scalar; ++i)
        ptrs[(size_t)i] = scalars[i].ptr;
    return launch_group_impl(k, ndims, 1, n_in, in, n_scalar, ptrs.data(), 1, scalars, n_out, out, s);
}

int cnh_launch_group(cnh_kernel* k, int ndims, int n_in, const cnh_memref* in, int n_scalar,
                     const void* const* scalars, int scalars_on_device, int n_out,
                     const cnh_memref* out, cnh_stream s) {
    return cnh_launch_group_batched(k, ndims, 1, n_in, in, n_scalar, scalars, scalars_on_device,
                                    n_out, out, s);
}

} // extern "C"

// ---------------------------------------------------------------------------------------------
// A product with the statements of a group in its epilogue.
// ---------------------------------------------------------------------------------------------
namespace {
struct GemmSegDev {
    const double* A;
    int64_t lda;
    const double* B;
    int64_t ldb;
    int32_t K, pad;
};
struct GemmChainDev {
    double* C;
    int64_t ldc;
    int32_t M, N, seg0, nseg, blk0, nbm;
};
static_assert(sizeof(GemmSegDev) == 40 && sizeof(GemmChainDev) == 40, "as gemm_kernel.inc lays them out");
} // namespace

namespace cnh {
int g_product_statements = 1;   // option "product_statements"
bool product_statements_on() { return g_product_statements != 0; }
} // namespace cnh

extern "C" int cnh_launch_product_group(cnh_kernel* k, const cnh_gemm_job* job, int n_blocks, int ndims, int n_in,
                                        const cnh_memref* in, const int32_t* in_block, int n_scalar,
                                        const void* const* scalars, int scalars_on_device, int n_out,
                                        const cnh_memref* out, cnh_stream s) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(k != nullptr && job != nullptr, -2, "null argument");
    const GroupProgram& p = k->prog;
    CNH_CHECK(ndims == p.ndims, -4, "kernel was compiled for rank %d, launched with %d", p.ndims, ndims);
    CNH_CHECK(n_in == (int)p.leaves.size(), -4, "group expects %d input memrefs, got %d", (int)p.leaves.size(),
              n_in);
    CNH_CHECK(n_out == (int)p.out_roots.size(), -4, "group expects %d output memrefs, got %d",
              (int)p.out_roots.size(), n_out);
    CNH_CHECK(n_out >= 1 && out != nullptr, -2, "a group needs at least one output memref");
    CNH_CHECK(n_in == 0 || (in != nullptr && in_block != nullptr), -2, "null input memrefs");
    CNH_CHECK(job->M >= 0 && job->N >= 0 && job->K >= 0 && job->A && job->B && job->C, -2,
              "product: bad extent or null pointer");
    CNH_CHECK(job->lda >= job->K && job->ldb >= job->N && job->ldc >= job->N, -2,
              "product: row stride shorter than the row");
    // what the fused kernel does not take is left to the caller's two launches
    CNH_CHECK(g_product_statements, -17, "statements in a product's epilogue are switched off");
    CNH_CHECK(p.dtype == CNH_F64 && p.reductions() == 0 && ndims >= 2, -17,
              "statements in a product's epilogue: fp64, rank 2 or 3, no reducing roots");
    CNH_CHECK(n_blocks == 1 || n_blocks == 2 || n_blocks == 4, -17, "%d column blocks (1, 2 or 4)", n_blocks);
    const int form = gemm_form(job->M, job->N, job->K, job->A, job->lda, job->B, job->ldb);
    CNH_CHECK(form != 0 && job->N % n_blocks == 0, -17,
              "product of %lld x %lld x %lld: extents no multiples of the 64 x 64 x 16 tile, or operands the "
              "buffer loads do not take", (long long)job->M, (long long)job->N, (long long)job->K);
    const int64_t nblock = job->N / n_blocks;
    const int NL = (int)p.load_leaf.size();
    const int NLA = NL > 0 ? NL : 1, NOA = n_out;
    const int pad = CNH_MAX_ND - ndims;
    // every memref of the group has the extents (1, ..., rows of the product, width of a column block)
    for (int i = 0; i < n_in + n_out; ++i) {
        const cnh_memref& m = i < n_in ? in[i] : out[i - n_in];
        if (i < n_in && in_block[i] >= 0) {
            CNH_CHECK(in_block[i] < n_blocks, -4, "input %d names column block %d of %d", i, in_block[i], n_blocks);
            continue;                       // taken from the tile of sums: its memref is not read
        }
        CNH_CHECK(m.aligned != nullptr, -4, "memref %d has a null pointer", i);
        for (int d = 0; d < ndims; ++d) {
            const int64_t want = d == ndims - 1 ? nblock : d == ndims - 2 ? job->M : 1;
            CNH_CHECK(m.sizes[d] == want, -17, "memref %d has extent %lld in dim %d, the product's blocks have %lld",
                      i, (long long)m.sizes[d], d, (long long)want);
        }
    }
    std::vector<unsigned char> scal;
    if (int rc = pack_scalars(p, n_scalar, scalars, scalars_on_device, scal))
        return rc;
    const int esz = 8;
    auto base_ptr = [&](const cnh_memref& m) -> int64_t {
        return (int64_t)((uintptr_t)m.aligned + (uintptr_t)(m.offset * esz));
    };
    // EpiArgs { Cell cell; Scal sc; int src[NLA]; int nblock; int unused; } as the generated text lays it out
    const size_t cell_words = 5 + NLA + 3 * NLA + NOA + 3 * NOA;
    const size_t tail_bytes = ((size_t)(NLA + 2) * 4 + 7) & ~size_t(7);
    std::vector<unsigned char> epi(cell_words * 8 + scal.size() + tail_bytes, 0);
    int64_t* c = reinterpret_cast<int64_t*>(epi.data());
    c[0] = 1;
    c[1] = job->M;
    c[2] = nblock;
    int64_t* cin = c + 5;
    int64_t* cistr = cin + NLA;
    int64_t* cout = cistr + 3 * NLA;
    int64_t* costr = cout + NOA;
    int32_t* src = reinterpret_cast<int32_t*>(epi.data() + cell_words * 8 + scal.size());
    for (int l = 0; l < NL; ++l) {
        const int leaf = p.load_leaf[l];
        src[l] = in_block[leaf] >= 0 ? in_block[leaf] : -1;
        if (src[l] >= 0)
            continue;
        cin[l] = base_ptr(in[leaf]);
        for (int d = 0; d < ndims; ++d)
            cistr[l * 3 + pad + d] = in[leaf].strides[d];
    }
    for (int o = 0; o < n_out; ++o) {
        cout[o] = base_ptr(out[o]);
        for (int d = 0; d < ndims; ++d)
            costr[o * 3 + pad + d] = out[o].strides[d];
    }
    std::memcpy(epi.data() + cell_words * 8, scal.data(), scal.size());
    src[NLA] = (int32_t)nblock;
    hipFunction_t fn;
    const std::string variant = "product" + std::to_string(n_blocks) + (form == 2 ? "e" : form == 3 ? "f" : "");
    if (int rc = get_function(k, variant, "grp_product", &fn))
        return rc;
    GemmChainDev ch{(double*)job->C, job->ldc, (int32_t)job->M, (int32_t)job->N, 0, 1, 0, (int32_t)(job->M / 64)};
    GemmSegDev sg{(const double*)job->A, job->lda, (const double*)job->B, job->ldb, (int32_t)job->K, 0};
    const void* no_table = nullptr;
    int nchains = 1, nblocks = (int)((job->M / 64) * (job->N / 64)), overwrite = 1;
    void* params[] = {&no_table, &nchains, &no_table, &nblocks, &ch, &sg, &overwrite, epi.data()};
    return launch(fn, nblocks, params, as_stream(s), form == 1 ? 1024 : form == 2 ? 512 : 256);
}

// ---------------------------------------------------------------------------------------------
// Tiled launch: all tiles of the target in one launch, neighbour tiles read in place.
// ---------------------------------------------------------------------------------------------
namespace {

struct TiledDev {
    int32_t shift, tile, off[3], shape[3], glo[3], grid[3];
    const void* tiles;
    int32_t py, pz;
};
static_assert(sizeof(TiledDev) == 72, "TiledDev layout must match the generated struct");

struct DTileDev {
    int64_t blk0;
    int32_t cs[3], w[3], nchunks, rsh;
    int32_t bs[3], bw[3];
    void* dst;
    const void* cur;
    int32_t py, pz;
};
static_assert(sizeof(DTileDev) == 88, "DTileDev layout must match the generated struct");

int check_tiled(const cnh_tiled* t, int nd, const char* what) {
    CNH_CHECK(t != nullptr, -2, "%s: null descriptor", what);
    CNH_CHECK(t->ndims == nd, -4, "%s: rank %d, expected %d", what, t->ndims, nd);
    CNH_CHECK(t->tile > 0 && (t->tile & (t->tile - 1)) == 0, -4,
              "%s: tile edge %d is not a power of two", what, t->tile);
    CNH_CHECK(t->tiles != nullptr, -4, "%s: null tile table", what);
    int64_t count = 1;
    for (int d = 0; d < nd; ++d) {
        CNH_CHECK(t->shape[d] > 0 && t->offset[d] >= 0, -4, "%s: bad shape/offset in dim %d", what, d);
        int glo = t->offset[d] / t->tile;
        int ghi = (t->offset[d] + t->shape[d] + t->tile - 1) / t->tile;
        CNH_CHECK(t->grid_lo[d] == glo && t->grid[d] == ghi - glo, -4,
                  "%s: tile grid in dim %d is [%d,+%d), decomposition implies [%d,+%d)", what, d,
                  t->grid_lo[d], t->grid[d], glo, ghi - glo);
        count *= t->grid[d];
    }
    for (int64_t i = 0; i < count; ++i)
        CNH_CHECK(t->tiles[i] != nullptr, -4, "%s: tile %lld has a null pointer", what, (long long)i);
    bool any = false, all = true;
    for (int d = 0; d < nd; ++d) {
        any = any || t->pitch[d] != 0;
        all = all && t->pitch[d] > 0;
    }
    CNH_CHECK(!any || (all && t->pitch[nd - 1] == 1), -4,
              "%s: pitches must be all zero, or positive with 1 along the last dimension", what);
    for (int d = 0; any && d < nd; ++d)
        CNH_CHECK(t->pitch[d] < (1ll << 31), -4, "%s: pitch of dim %d does not fit 31 bits", what, d);
    for (int d = 0; any && d + 1 < nd; ++d)
        CNH_CHECK(t->pitch[d] >= t->pitch[d + 1] * std::min(t->tile, t->shape[d + 1]), -4,
                  "%s: pitch %lld of dim %d is shorter than a tile's extent below it", what,
                  (long long)t->pitch[d], d);
    return 0;
}

// Is the array one row-major block starting at element 0 (tiles that are views into it, or a single
// tile)? pitch[0], pitch[1] receive the elements between planes and between rows of the
// rank-padded (z, y, x) view.
bool one_block_of(const cnh_tiled* t, int esz, int64_t* pitch) {
    const int nd = t->ndims;
    int64_t ntiles = 1;
    for (int d = 0; d < nd; ++d) {
        if (t->offset[d] != 0)
            return false;
        ntiles *= t->grid[d];
    }
    int64_t p[3] = {0, 0, 0};
    bool pitched = false;
    for (int d = 0; d < nd; ++d)
        pitched = pitched || t->pitch[d] != 0;
    if (pitched) {
        for (int d = 0; d < nd; ++d)
            p[d] = t->pitch[d];
        if (p[nd - 1] != 1)
            return false;
    } else {
        if (ntiles != 1)
            return false;
        int64_t run = 1;
        for (int d = nd - 1; d >= 0; --d) {
            p[d] = run;
            run *= t->shape[d];
        }
    }
    // every tile starts where its first element lies in the block
    const char* base = static_cast<const char*>(t->tiles[0]);
    int64_t idx[3] = {0, 0, 0};
    for (int64_t n = 0; n < ntiles; ++n) {
        int64_t off = 0;
        for (int d = 0; d < nd; ++d)
            off += idx[d] * t->tile * p[d];
        if (static_cast<const char*>(t->tiles[n]) != base + off * esz)
            return false;
        for (int d = nd - 1; d >= 0; --d) {
            if (++idx[d] < t->grid[d])
                break;
            idx[d] = 0;
        }
    }
    pitch[0] = nd >= 3 ? p[0] : 0;
    pitch[1] = nd >= 2 ? p[nd - 2] : 0;
    pitch[2] = 1;
    return true;
}

struct BlockLeafDev {
    const void* base;
    int32_t py, pz, start[3], step[3], lim[3], unused;
};
struct BlockHeadDev {
    void* dst;
    const void* cur;
    int32_t shape[3], dpy, dpz, rs[3], re[3], rst[3], cnt[3], lattice, nchunks, rsh;
    int32_t nroots, nblk8, rrs[4][3], rcnt[4][3], rmate[4];
};
static_assert(sizeof(BlockLeafDev) == 56 && sizeof(BlockHeadDev) == 216, "BlockArgs layout must match the generated struct");

bool is_pitched(const cnh_tiled* t) {
    for (int d = 0; d < t->ndims; ++d)
        if (t->pitch[d] != 0)
            return true;
    return false;
}

int make_tiled_dev(const cnh_tiled* t, hipStream_t st, TiledDev& d) {
    int nd = t->ndims, pad = CNH_MAX_ND - nd;
    std::memset(&d, 0, sizeof d);
    d.tile = t->tile;
    d.shift = 0;
    while ((1 << d.shift) < t->tile)
        d.shift++;
    int64_t count = 1;
    for (int i = 0; i < 3; ++i) {
        d.off[i] = 0;
        d.shape[i] = 1;
        d.glo[i] = 0;
        d.grid[i] = 1;
    }
    for (int i = 0; i < nd; ++i) {
        d.off[pad + i] = t->offset[i];
        d.shape[pad + i] = t->shape[i];
        d.glo[pad + i] = t->grid_lo[i];
        d.grid[pad + i] = t->grid[i];
        count *= t->grid[i];
    }
    const void* table = nullptr;
    if (int rc = desc_upload(t->tiles, (size_t)count * sizeof(void*), st, &table))
        return rc;
    d.tiles = table;
    // rank 1 has nothing between rows; rank 2 has no planes
    d.py = nd >= 2 ? (int32_t)t->pitch[nd - 2] : 0;
    d.pz = nd >= 3 ? (int32_t)t->pitch[0] : 0;
    return 0;
}

} // namespace

namespace {

struct SlideArgsDev {
    const void* cur;
    void* dst;
    int32_t shift, shape[3], grid[3], rs[3], re[3], nbx, nby, nzc, nblocks;
};
static_assert(sizeof(SlideArgsDev) == 88, "SlideArgsDev layout must match the generated struct");

bool g_slide_enabled = false;
SlideConfig g_slide_cfg;
bool slide_disabled() { return !g_slide_enabled; }

// Launches the sliding-window variant when the group is a unit-step stencil on the assigned
// array itself, the decomposition has no offset and the new contents go to a second buffer.
int try_launch_slide(cnh_kernel* k, const std::vector<const cnh_tiled*>& arrays,
                     const cnh_tiled* cur, const cnh_tiled* dst,
                     const std::vector<unsigned char>& scal, hipStream_t st, bool* handled) {
    *handled = false;
    const GroupProgram& p = k->prog;
    SlideShape sh;
    std::string why;
    if (slide_disabled() || slide_shape(p, g_slide_cfg, sh, why) != 0)
        return 0;
    if (!cur || arrays.size() != 1 || cur->tile < 2)
        return 0;
    const int nd = p.ndims;
    int64_t ntiles = 1;
    for (int d = 0; d < nd; ++d) {
        if (cur->offset[d] != 0 || dst->offset[d] != 0 || arrays[0]->offset[d] != 0 ||
            arrays[0]->shape[d] != cur->shape[d])
            return 0;
        ntiles *= cur->grid[d];
    }
    if (arrays[0]->tile != cur->tile || arrays[0]->tiles[0] != cur->tiles[0])
        return 0;
    {
        int64_t vol = 1; // in-tile offsets are 32-bit in the kernel
        for (int d = 0; d < nd; ++d)
            vol *= std::min(cur->tile, cur->shape[d]);
        if (vol >= (1ll << 31))
            return 0;
    }
    for (int64_t t = 0; t < ntiles; ++t)
        if (cur->tiles[t] == dst->tiles[t])
            return 0; // in place: a sweep would read values it has already written

    SlideArgsDev a;
    std::memset(&a, 0, sizeof a);
    a.shift = 0;
    while ((1 << a.shift) < cur->tile)
        a.shift++;
    for (int d = 0; d < 3; ++d) {
        a.shape[d] = 1;
        a.grid[d] = 1;
        a.rs[d] = 0;
        a.re[d] = 1;
    }
    bool vec = (cur->tile % 2) == 0;
    for (int d = 0; d < nd; ++d) {
        const int kd = sh.kdim(nd, d);
        a.shape[kd] = cur->shape[d];
        a.grid[kd] = cur->grid[d];
        a.rs[kd] = p.out_region[0].start[d];
        a.re[kd] = p.out_region[0].stop[d];
    }
    if (a.shape[2] % 2 != 0)
        vec = false;
    for (int64_t t = 0; t < ntiles; ++t)
        if (((uintptr_t)cur->tiles[t] & 15) || ((uintptr_t)dst->tiles[t] & 15))
            vec = false;
    a.nbx = (a.shape[2] + sh.bx - 1) / sh.bx;
    a.nby = (a.shape[1] + sh.ty * sh.ry - 1) / (sh.ty * sh.ry);
    a.nzc = (a.shape[0] + sh.zc - 1) / sh.zc;
    const int64_t blocks = (int64_t)a.nbx * a.nby * a.nzc;
    CNH_CHECK(blocks > 0 && blocks < (1ll << 31), -3, "stencil launch of %lld workgroups",
              (long long)blocks);
    a.nblocks = (int)blocks;
    const void* dcur = nullptr;
    const void* ddst = nullptr;
    if (int rc = desc_upload(cur->tiles, (size_t)ntiles * sizeof(void*), st, &dcur))
        return rc;
    if (int rc = desc_upload(dst->tiles, (size_t)ntiles * sizeof(void*), st, &ddst))
        return rc;
    a.cur = dcur;
    a.dst = const_cast<void*>(ddst);
    hipFunction_t fn;
    int64_t volume = 1;
    for (int d = 0; d < nd; ++d)
        volume *= cur->shape[d];
    const bool nontemporal = volume * 16 >= ((int64_t)g_stencil_nt_mib << 20); // read + write stream past the cache
    if (int rc = get_function(k, g_slide_cfg.variant(),
                              !vec ? "grp_slide_s" : nontemporal ? "grp_slide_vn" : "grp_slide_v", &fn))
        return rc;
    void* params[] = {&a, const_cast<unsigned char*>(scal.data())};
    if (int rc = launch(fn, blocks, params, st))
        return rc;
    *handled = true;
    return 0;
}

struct FDivDev {
    uint32_t d, m, s;
};
// n / d == (n * m) >> s for 0 <= n < 2^31: s = 31 + ceil(log2 d), m = ceil(2^s / d) < 2^32.
FDivDev fdiv_make(uint32_t d) {
    if (d == 0)
        d = 1;
    uint32_t L = 0;
    while ((1ull << L) < d)
        ++L;
    FDivDev f;
    f.d = d;
    f.s = 31 + L;
    f.m = (uint32_t)(((1ull << f.s) + d - 1) / d);
    return f;
}
struct DirectArgsDev {
    const void* cur;
    void* dst;
    int32_t tile, shape[3], grid[3], rs[3], re[3], tb[3], sg[3], nblocks, nblocks8, stagger;
    FDivDev per_group, ggrid1, ggrid2, grow, gcol, tbz, tby, tbx;
    const void* oth[kDirectMaxOther];
    int32_t py, pz;
    void* slots;
};
static_assert(sizeof(DirectArgsDev) == 16 + 4 * 22 + 12 * 8 + 8 * kDirectMaxOther + 8 + 8,
              "DirectArgsDev layout must match the generated struct");

struct FlatArgsDev {
    const void* cur;
    void* dst;
    const void* oth[kDirectMaxOther];
    int32_t shape[3], rs[3], re[3], py, pz, nb[3], ob[3], nblocks8;
    FDivDev per_block, gb1, gb2, obx, oby;
    void* slots;
    int32_t sub8;
    FDivDev fsub;
    int32_t lat[3], nroots, rs2[3], re2[3], tail, unused;
};
static_assert(sizeof(FlatArgsDev) == 16 + 8 * kDirectMaxOther + 4 * 18 + 12 * 5 + 4 + 8 + 16 + 40 + 8,
              "FlatArgsDev layout must match the generated struct");

// A launch that should also reduce what it changes: mode 1 = sum of (new - old)^2, 2 = max
// |new - old|, result to *out (device). `done` is set by the kernel path that took it.
struct RedReq {
    int mode = 0;
    void* out = nullptr;
    bool done = false;
};

int g_direct_flat = 1;          // arrays stored as one block take the whole-array kernel
int g_flat_tail = 1;            // ... and fold one or two unassigned last columns into the wavefront before them
int g_flat_ob[3] = {0, 0, 0};   // ordering block of that kernel in elements (z, y, x); 0 = default
int g_stencil_mode = 2; // 0 = general gather, 1 = LDS sliding window, 2 = register window
int g_direct_group = 0; // order workgroups by groups of neighbouring tiles (rank 3)
int g_direct_lean = -1;   // wavefront-level lean kernel: 1 on, 0 off, -1 by rank
int g_tiles_rows = 1;     // general gather: short rows share a workgroup
int g_tiles_block = 1;    // general gather: arrays that are one block each skip the tile logic
int g_block_pairs = 1;    // ... and unit-step statements among them move pairs of elements
int g_direct_stagger = 0; // concurrent groups start at different offsets of their tiles
int g_direct_merge = 1;   // lean part and the rest in one launch instead of two
DirectConfig g_direct_cfg;

// Launches the register-window variant under the same conditions as the sliding window, plus:
// every tile extent along the fastest dimension is even (128-bit accesses never straddle tiles).
int launch_direct(cnh_kernel* k, const DirectShape& sh, const std::vector<const cnh_tiled*>& arrays,
                  const cnh_tiled* const* others, int n_other, const cnh_tiled* cur,
                  const cnh_tiled* dst, const std::vector<unsigned char>& scal, hipStream_t st,
                  bool* handled, RedReq* red);

int try_launch_direct(cnh_kernel* k, const std::vector<const cnh_tiled*>& arrays,
                      const std::vector<int>& leaf_array, const cnh_tiled* cur, const cnh_tiled* dst,
                      const std::vector<unsigned char>& scal, hipStream_t st, bool* handled,
                      RedReq* red) {
    *handled = false;
    const GroupProgram& p = k->prog;
    if (g_stencil_mode != 2)
        return 0;
    {
        std::lock_guard<std::mutex> lock(k->mu);
        if (!k->shape_known || k->shape_cfg[0] != g_direct_cfg.tx || k->shape_cfg[1] != g_direct_cfg.ry ||
            k->shape_cfg[2] != g_direct_cfg.rz) {
            std::string why;
            k->shape_rc = direct_shape(p, g_direct_cfg, k->shape, why);
            k->shape_cfg[0] = g_direct_cfg.tx;
            k->shape_cfg[1] = g_direct_cfg.ry;
            k->shape_cfg[2] = g_direct_cfg.rz;
            k->shape_known = true;
        }
    }
    if (k->shape_rc != 0)
        return 0;
    const DirectShape& sh = k->shape;
    if (!cur || arrays.empty() || cur->tile < 2 || (cur->tile % 2) != 0)
        return 0;
    // Which operand array is the assigned one (read through the window), which are the others:
    // the generated code numbers the others by name, the launch must hand it the same arrays.
    int self = -1;
    const cnh_tiled* others[kDirectMaxOther] = {nullptr, nullptr, nullptr, nullptr};
    if (leaf_array.size() != sh.other.size())
        return 0;
    for (size_t l = 0; l < sh.other.size(); ++l) {
        const int ai = leaf_array[l];
        if (ai < 0 || ai >= (int)arrays.size())
            return 0;
        if (sh.other[l] < 0) {
            if (self >= 0 && self != ai)
                return 0;
            self = ai;
        } else {
            const cnh_tiled*& slot = others[sh.other[l]];
            if (slot != nullptr && slot != arrays[(size_t)ai])
                return 0;
            slot = arrays[(size_t)ai];
        }
    }
    if (self < 0)
        return 0;
    const std::vector<const cnh_tiled*> own(1, arrays[(size_t)self]);
    if (sh.masked) {
        // The window array is not the assigned one: the launch reads that array's tiles and
        // writes the target's assigned elements in place. Both must be cut alike.
        const cnh_tiled* w = own[0];
        if (cur == nullptr || dst->tiles[0] != cur->tiles[0] || w->ndims != dst->ndims ||
            w->tile != dst->tile)
            return 0;
        for (int d = 0; d < w->ndims; ++d)
            if (w->shape[d] != dst->shape[d] || w->grid[d] != dst->grid[d] || w->offset[d] != 0 ||
                dst->offset[d] != 0 || w->pitch[d] != dst->pitch[d])
                return 0;
        return launch_direct(k, sh, own, others, (int)sh.other_names.size(), w, dst, scal, st, handled,
                             nullptr);   // the target's old values are not read: nothing to reduce here
    }
    return launch_direct(k, sh, own, others, (int)sh.other_names.size(), cur, dst, scal, st, handled, red);
}

int launch_direct(cnh_kernel* k, const DirectShape& sh, const std::vector<const cnh_tiled*>& arrays,
                  const cnh_tiled* const* others, int n_other, const cnh_tiled* cur,
                  const cnh_tiled* dst, const std::vector<unsigned char>& scal, hipStream_t st,
                  bool* handled, RedReq* red) {
    const GroupProgram& p = k->prog;
    const int nd = p.ndims, pad = CNH_MAX_ND - nd;
    int64_t ntiles = 1, vol = 1, volume = 1;
    for (int d = 0; d < nd; ++d) {
        if (cur->offset[d] != 0 || dst->offset[d] != 0 || arrays[0]->offset[d] != 0 ||
            arrays[0]->shape[d] != cur->shape[d])
            return 0;
        ntiles *= cur->grid[d];
        vol *= std::min(cur->tile, cur->shape[d]);
        volume *= cur->shape[d];
    }
    if (arrays[0]->tile != cur->tile || arrays[0]->tiles[0] != cur->tiles[0] || vol >= (1ll << 31))
        return 0;
    // In place: a sweep would read values it has already written, unless it assigns a lattice that
    // none of its shifted reads can meet (the colours of a red-black sweep).
    bool inplace = false;
    for (int64_t t = 0; t < ntiles; ++t)
        inplace = inplace || cur->tiles[t] == dst->tiles[t];
    if (inplace && !(sh.lattice && sh.inplace_safe))
        return 0;
    if (inplace && red != nullptr && red->mode != 0)
        return 0;                         // the old values do not survive: nothing to compare with
    // Pitched tiles (views into one row-major block): every array of the launch has to use the
    // same pitches, with a pitch of 1 along the rows.
    int64_t pitch[3] = {0, 0, 0};
    bool pitched = false;
    for (int d = 0; d < nd; ++d)
        if (cur->pitch[d] != 0)
            pitched = true;
    if (pitched) {
        for (int d = 0; d < nd; ++d) {
            if (cur->pitch[d] <= 0 || cur->pitch[d] >= (1ll << 31))
                return 0;
            pitch[pad + d] = cur->pitch[d];
        }
        if (pitch[2] != 1)
            return 0;
    }
    auto same_pitch = [&](const cnh_tiled* t) {
        for (int d = 0; d < nd; ++d)
            if (t->pitch[d] != cur->pitch[d])
                return false;
        return true;
    };
    if (!same_pitch(dst) || !same_pitch(arrays[0]))
        return 0;
    // the other arrays are read at the element's own position: same decomposition, other memory
    for (int j = 0; j < n_other; ++j) {
        const cnh_tiled* o = others[j];
        if (o == nullptr || o->ndims != cur->ndims || o->tile != cur->tile || !same_pitch(o))
            return 0;
        for (int d = 0; d < nd; ++d)
            if (o->offset[d] != 0 || o->shape[d] != cur->shape[d] || o->grid[d] != cur->grid[d] ||
                o->grid_lo[d] != cur->grid_lo[d])
                return 0;
        // (an operand at the element's own position may be the target itself when the window
        // array is another one: a lane then reads the very elements it writes)
        for (int64_t t = 0; t < ntiles; ++t)
            if (!sh.masked && o->tiles[t] == dst->tiles[t])
                return 0;
    }
    // Pairs of elements move as 128-bit accesses where every pair is 16-byte aligned: even rows
    // and pitches, aligned tile starts. The whole-array kernel below also has a form for the rest
    // (rows of odd length, the 2^k + 1 grids of multigrid); the per-tile kernels need the alignment.
    bool aligned = cur->shape[nd - 1] % 2 == 0 && pitch[1] % 2 == 0 && pitch[0] % 2 == 0;
    for (int64_t t = 0; t < ntiles && aligned; ++t) {
        aligned = !(((uintptr_t)cur->tiles[t] | (uintptr_t)dst->tiles[t]) & 15);
        for (int j = 0; j < n_other && aligned; ++j)
            aligned = !((uintptr_t)others[j]->tiles[t] & 15);
    }
    // Every array of the launch one row-major block behind its tile views: no tile logic at all.
    if (pitched && g_direct_flat) {
        const int esz = dtype_size(p.dtype);
        int64_t unused_pitch[3];
        auto one_block = [&](const cnh_tiled* t) { return one_block_of(t, esz, unused_pitch); };
        bool flat = one_block(cur) && one_block(dst) && pitch[1] >= cur->shape[nd - 1] && cur->shape[nd - 1] >= 2 &&
                    (nd < 3 || pitch[0] >= pitch[1] * cur->shape[1]) &&
                    pitch[0] * (nd == 3 ? cur->shape[0] : 1) + pitch[1] * cur->shape[nd - 2] < (1ll << 31);
        for (int j = 0; j < n_other && flat; ++j)
            flat = one_block(others[j]);
        if (flat) {
            FlatArgsDev f;
            std::memset(&f, 0, sizeof f);
            f.cur = cur->tiles[0];
            f.dst = dst->tiles[0];
            for (int j = 0; j < n_other; ++j)
                f.oth[j] = others[j]->tiles[0];
            for (int d = 0; d < 3; ++d) {
                f.shape[d] = 1;
                f.rs[d] = 0;
                f.re[d] = 1;
            }
            for (int d = 0; d < nd; ++d) {
                f.shape[pad + d] = cur->shape[d];
                f.rs[pad + d] = p.out_region[0].start[d];
                f.re[pad + d] = p.out_region[0].stop[d];
            }
            f.py = (int32_t)pitch[1];
            f.pz = (int32_t)pitch[0];
            f.nroots = sh.nroots;
            for (int d = 0; d < 3; ++d) {
                f.lat[d] = sh.lat[d];
                f.rs2[d] = 0;
                f.re2[d] = 0;
            }
            if (sh.nroots > 1)
                for (int d = 0; d < nd; ++d) {
                    f.rs2[pad + d] = p.out_region[1].start[d];
                    f.re2[pad + d] = p.out_region[1].stop[d];
                }
            if (sh.nroots > 1)
                for (int d = 0; d < pad; ++d)
                    f.re2[d] = 1;
            // a workgroup: 4 wavefronts stacked along y, each 128 columns x ry rows x rz planes
            const int foot[3] = {sh.rz, 4 * sh.ry, 128};
            // ordering block: 256^3 elements for rank 3 (measured on MI355X, 512^3: 382 us per
            // sweep against 390 with 128^3 and 449 with whole planes); rank 2: bands of whole rows
            const int dflt[3] = {256, nd == 3 ? 256 : 1 << 30, nd == 3 ? 256 : 1 << 30};
            int64_t launched = 1, gb[3];
            for (int d = 0; d < 3; ++d)
                f.nb[d] = (f.shape[d] + foot[d] - 1) / foot[d];
            // One or two unassigned columns beyond a multiple of 128 (the right-hand boundary of a
            // 2^k + 1 grid) get no workgroups of their own: the last lane of the row's last
            // wavefront copies them. Only into a second buffer; a sweep in place leaves them alone.
            // A launch that stores assigned elements only (a sweep from another array, a sweep in
            // place) needs no workgroups at all for columns beyond the assigned region.
            if (g_flat_tail && f.nb[2] >= 2 && f.re[2] <= 128 * (f.nb[2] - 1)) {
                const int beyond = f.shape[2] - 128 * (f.nb[2] - 1);
                const bool writes_everything = f.cur != f.dst && !sh.masked;
                if (!writes_everything) {
                    while (f.nb[2] >= 2 && f.re[2] <= 128 * (f.nb[2] - 1))
                        f.nb[2] -= 1;
                } else if (sh.tail_ok && beyond <= 2) {
                    f.tail = beyond;
                    f.nb[2] -= 1;
                }
            }
            for (int d = 0; d < 3; ++d) {
                const int want = g_flat_ob[d] > 0 ? g_flat_ob[d] : dflt[d];
                f.ob[d] = std::max(1, std::min(f.nb[d], want / foot[d]));
                gb[d] = (f.nb[d] + f.ob[d] - 1) / f.ob[d];
                // as many blocks as that, of equal size: a 257-wide array gets blocks of 129 + 128
                // columns' worth of workgroups instead of 256 + 1
                f.ob[d] = (int32_t)((f.nb[d] + gb[d] - 1) / gb[d]);
                launched *= gb[d] * f.ob[d];
            }
            CNH_CHECK(launched > 0 && launched < (1ll << 31), -3, "stencil launch of %lld workgroups",
                      (long long)launched);
            // Consecutive workgroup ids go to consecutive XCDs: every XCD takes one contiguous
            // eighth of the order. A count that is no multiple of 8 is padded with workgroups whose
            // place in the order lies beyond the last block (they leave at once); without that,
            // neighbours in the order would sit behind different L2s and each would fetch the rows
            // and the ends of cache lines they share (measured on a 4097^2 sweep: 25 % more fetched).
            launched = (launched + 7) / 8 * 8;
            f.nblocks8 = (int32_t)(launched / 8);
            f.per_block = fdiv_make((uint32_t)(f.ob[0] * f.ob[1] * f.ob[2]));
            {
                // a grid that does not fill its ordering blocks: spread every block over the XCDs
                bool ragged = false;
                for (int d = 0; d < 3; ++d)
                    ragged = ragged || f.nb[d] % f.ob[d] != 0;
                const int64_t per = (int64_t)f.ob[0] * f.ob[1] * f.ob[2];
                f.sub8 = ragged && per % 8 == 0 && launched > per ? (int32_t)(per / 8) : 0;
                f.fsub = fdiv_make((uint32_t)std::max(1, f.sub8));
            }
            f.gb1 = fdiv_make((uint32_t)gb[1]);
            f.gb2 = fdiv_make((uint32_t)gb[2]);
            f.obx = fdiv_make((uint32_t)f.ob[2]);
            f.oby = fdiv_make((uint32_t)f.ob[1]);
            const bool nts = volume * (2 + n_other) * esz >= ((int64_t)g_stencil_nt_mib << 20);
            hipFunction_t fn;
            const bool reducing = red != nullptr && red->mode != 0 && p.dtype == CNH_F64 && !sh.lattice;
            if (reducing) {
                // one partial per launched wavefront, folded in index order by a second launch
                void* slots = nullptr;
                if (int rc = reduce_workspace(st, (size_t)(launched * 4 + kFoldRuns) * sizeof(double), &slots))
                    return rc;
                f.slots = slots;
                DirectConfig rcfg = g_direct_cfg;
                rcfg.reduce = true;
                const std::string name = std::string(aligned ? "grp_direct_flat_red" : "grp_direct_flatu_red") +
                                         (red->mode == 1 ? "1" : "2") + (nts ? "_nts" : "");
                if (int rc = get_function(k, rcfg.variant(), name.c_str(), &fn))
                    return rc;
            } else {
                const std::string name = std::string(aligned ? "grp_direct_flat" : "grp_direct_flatu") + (nts ? "_nts" : "");
                if (int rc = get_function(k, g_direct_cfg.variant(), name.c_str(), &fn))
                    return rc;
            }
            void* params[] = {&f, const_cast<unsigned char*>(scal.data())};
            if (int rc = launch(fn, launched, params, st))
                return rc;
            if (reducing) {
                if (int rc = reduce_slots_f64(red->mode == 2, static_cast<double*>(f.slots),
                                              launched * 4, static_cast<double*>(red->out), st))
                    return rc;
                red->done = true;
            }
            *handled = true;
            return 0;
        }
    }
    if (!aligned || sh.lattice || sh.other_shifted)
        return 0;                         // the per-tile kernels take aligned unit-step sweeps of one window only
    // a lane's own rows and planes must not straddle tiles: the tile edge (a power of two) has
    // to be a multiple of what one lane owns
    if (cur->tile % sh.ry != 0 || cur->tile % sh.rz != 0)
        return 0;
    DirectArgsDev a;
    std::memset(&a, 0, sizeof a);
    a.tile = cur->tile;
    for (int d = 0; d < 3; ++d) {
        a.shape[d] = 1;
        a.grid[d] = 1;
        a.rs[d] = 0;
        a.re[d] = 1;
    }
    for (int d = 0; d < nd; ++d) {
        a.shape[pad + d] = cur->shape[d];
        a.grid[pad + d] = cur->grid[d];
        a.rs[pad + d] = p.out_region[0].start[d];
        a.re[pad + d] = p.out_region[0].stop[d];
    }
    const int ext[3] = {sh.rz, sh.ty * sh.ry, sh.tx * 2};
    int64_t per_tile = 1;
    for (int d = 0; d < 3; ++d) {
        const int edge = std::min(a.tile, a.shape[d]);
        a.tb[d] = (edge + ext[d] - 1) / ext[d];
        per_tile *= a.tb[d];
    }
    const int64_t blocks = per_tile * ntiles;
    CNH_CHECK(blocks > 0 && blocks < (1ll << 31), -3, "stencil launch of %lld workgroups",
              (long long)blocks);
    a.nblocks = (int)blocks;
    a.nblocks8 = blocks % 8 == 0 ? (int)(blocks / 8) : 0;
    // Ordering groups: G^3 neighbouring full tiles whose joint z-slab still fits an L2 (edge of a
    // group at most 256 elements), G as large as the grid allows. Rank 3 only.
    int G = 1, Gx = 1;
    if (nd == 3 && g_direct_group == 1) {
        for (int cand = 2; cand <= 4; cand *= 2) {
            bool ok = (int64_t)cand * a.tile <= 256;
            for (int d = 0; d < 3 && ok; ++d)
                ok = a.grid[d] % cand == 0 && a.shape[d] == a.grid[d] * a.tile;
            if (ok)
                G = cand;
        }
    }
    // Mode 2: the tiles of one row of the tile grid along x form a group, so that the column
    // pairs a workgroup reads from its x neighbours are lines those neighbours load just then.
    if (nd == 3 && g_direct_group == 2 && a.grid[2] > 1 && a.grid[2] <= 8 &&
        a.shape[2] == a.grid[2] * a.tile)
        Gx = a.grid[2];
    for (int d = 0; d < 3; ++d)
        a.sg[d] = (d >= pad) ? G : 1;
    if (Gx > 1)
        a.sg[2] = Gx;
    a.per_group = fdiv_make((uint32_t)(per_tile * a.sg[0] * a.sg[1] * a.sg[2]));
    a.ggrid1 = fdiv_make((uint32_t)(a.grid[1] / a.sg[1]));
    a.ggrid2 = fdiv_make((uint32_t)(a.grid[2] / a.sg[2]));
    a.grow = fdiv_make((uint32_t)(a.tb[2] * a.sg[2]));
    a.gcol = fdiv_make((uint32_t)(a.tb[1] * a.sg[1]));
    a.tbz = fdiv_make((uint32_t)a.tb[0]);
    a.tby = fdiv_make((uint32_t)a.tb[1]);
    a.tbx = fdiv_make((uint32_t)a.tb[2]);
    a.stagger = g_direct_stagger ? (int)(a.per_group.d / 8) : 0;
    const void* dcur = nullptr;
    const void* ddst = nullptr;
    if (int rc = desc_upload(cur->tiles, (size_t)ntiles * sizeof(void*), st, &dcur))
        return rc;
    if (int rc = desc_upload(dst->tiles, (size_t)ntiles * sizeof(void*), st, &ddst))
        return rc;
    a.cur = dcur;
    a.dst = const_cast<void*>(ddst);
    for (int j = 0; j < n_other; ++j)
        if (int rc = desc_upload(others[j]->tiles, (size_t)ntiles * sizeof(void*), st, &a.oth[j]))
            return rc;
    a.py = (int32_t)pitch[1];
    a.pz = (int32_t)pitch[0];
    const bool nt_stores = volume * (2 + n_other) * dtype_size(p.dtype) >= ((int64_t)g_stencil_nt_mib << 20); // the written stream is not read back soon
    // Two launches over the same grid: wavefronts that lie inside their tile in y and z take the
    // lean kernel, the other kernel does what is left (all of it when the lean one does not apply).
    // measured on MI355X: the lean kernel pays off for rank 2 (tiles much wider than a wavefront
    // run: 8192^2 183 against 200 us); with the 128-wide tiles of rank 3 every wavefront reads both
    // x neighbours, and it pays a little once those reads are one gathered load per wavefront
    // (512^3: 424.0 against 430.7 us, six alternating runs)
    const bool want_lean = g_direct_lean < 0 ? true : g_direct_lean != 0;
    const bool lean = want_lean && sh.tx % 64 == 0 && sh.halo[2] >= 1;
    int skip_fast = lean ? 1 : 0;
    hipFunction_t fn;
    // When every workgroup away from the y and z faces of its tile consists of wavefronts the
    // lean kernel takes, the second launch covers the face workgroups only.
    const void* dlist = nullptr;
    int64_t rest_blocks = blocks;
    bool faces_only = lean && a.shape[2] % 128 == 0;
    for (int d = 0; d < 2 && faces_only; ++d) {
        // a partial last tile ends before its last workgroup row: its end is not on the list
        if (a.grid[d] > 1 && a.shape[d] != a.grid[d] * a.tile)
            faces_only = false;
        else if (sh.halo[d] > 0)
            faces_only = a.rs[d] <= ext[d] && a.re[d] >= a.shape[d] - ext[d];
        else
            faces_only = a.rs[d] == 0 && a.re[d] == a.shape[d];
    }
    std::vector<int32_t> list;
    if (faces_only) {
        // positions in the order locate() decodes: group by group, x fastest inside a group
        const int gx = a.tb[2] * a.sg[2], gy = a.tb[1] * a.sg[1], gz = a.tb[0] * a.sg[0];
        const int64_t per_group = (int64_t)gx * gy * gz;
        const int64_t ngroups = blocks / per_group;
        for (int64_t g = 0; g < ngroups; ++g)
            for (int z = 0; z < gz; ++z) {
                const int bz = z % a.tb[0];
                const bool zf = sh.halo[0] > 0 && (bz == 0 || bz == a.tb[0] - 1);
                for (int y = 0; y < gy; ++y) {
                    const int by = y % a.tb[1];
                    const bool yf = sh.halo[1] > 0 && (by == 0 || by == a.tb[1] - 1);
                    if (!zf && !yf)
                        continue;
                    for (int x = 0; x < gx; ++x) {
                        // undo the stagger: position w' = w + (g & 7) * stagger (mod per_group)
                        int64_t w = ((int64_t)z * gy + y) * gx + x;
                        int64_t pos = w - (int64_t)(g & 7) * a.stagger;
                        if (pos < 0)
                            pos += per_group;
                        list.push_back((int32_t)(g * per_group + pos));
                    }
                }
            }
        if (list.empty())
            rest_blocks = 0;
        else {
            if (int rc = desc_upload(list.data(), list.size() * sizeof(int32_t), st, &dlist))
                return rc;
            rest_blocks = (int64_t)list.size();
        }
    }
    if (lean && g_direct_merge) {
        // lean part and the rest in one launch
        const bool reducing = red != nullptr && red->mode != 0 && p.dtype == CNH_F64 && !sh.masked;
        const int64_t launched = blocks + rest_blocks;
        if (reducing) {
            // one partial per launched wavefront, folded in index order by a second launch
            void* slots = nullptr;
            if (int rc = reduce_workspace(st, (size_t)(launched * 4 + kFoldRuns) * sizeof(double), &slots))
                return rc;
            a.slots = slots;
            DirectConfig rcfg = g_direct_cfg;
            rcfg.reduce = true;
            const char* name = red->mode == 1 ? (nt_stores ? "grp_direct_both_red1_nts" : "grp_direct_both_red1")
                                              : (nt_stores ? "grp_direct_both_red2_nts" : "grp_direct_both_red2");
            if (int rc = get_function(k, rcfg.variant(), name, &fn))
                return rc;
        } else if (int rc = get_function(k, g_direct_cfg.variant(),
                                         nt_stores ? "grp_direct_both_nts" : "grp_direct_both", &fn))
            return rc;
        void* params[] = {&a, const_cast<unsigned char*>(scal.data()), &dlist};
        if (int rc = launch(fn, launched, params, st))
            return rc;
        if (reducing) {
            if (int rc = reduce_slots_f64(red->mode == 2, static_cast<double*>(a.slots), launched * 4,
                                          static_cast<double*>(red->out), st))
                return rc;
            red->done = true;
        }
        *handled = true;
        return 0;
    }
    if (lean) {
        if (int rc = get_function(k, g_direct_cfg.variant(),
                                  nt_stores ? "grp_direct_fast_nts" : "grp_direct_fast", &fn))
            return rc;
        void* params[] = {&a, const_cast<unsigned char*>(scal.data())};
        if (int rc = launch(fn, blocks, params, st))
            return rc;
    }
    if (rest_blocks > 0) {
        if (int rc = get_function(k, g_direct_cfg.variant(),
                                  nt_stores ? "grp_direct_rest_nts" : "grp_direct_rest", &fn))
            return rc;
        void* params[] = {&a, const_cast<unsigned char*>(scal.data()), &skip_fast, &dlist};
        if (int rc = launch(fn, rest_blocks, params, st))
            return rc;
    }
    *handled = true;
    return 0;
}

} // namespace

extern "C" int64_t cnh_code_objects_from_disk(void) {
    std::lock_guard<std::mutex> lk(g_cmu);
    return g_disk_hits;
}

extern "C" int64_t cnh_code_objects(void) {
    std::lock_guard<std::mutex> lk(g_cmu);
    return (int64_t)g_code.size();
}

extern "C" int cnh_set_option(const char* name, int value) {
    CNH_CHECK(name != nullptr, -2, "null option name");
    if (std::strcmp(name, "tiles_block") == 0) {
        g_tiles_block = value != 0;
        return 0;
    }
    if (std::strcmp(name, "stencil_mode") == 0) {
        CNH_CHECK(value >= 0 && value <= 2, -2, "stencil_mode must be 0, 1 or 2");
        g_stencil_mode = value;
        g_slide_enabled = value == 1;
        return 0;
    }
    if (std::strcmp(name, "gemv_xlds") == 0) {
        CNH_CHECK(value == 0 || value == 1, -2, "gemv_xlds: 0 or 1");
        gemv_set_xlds(value);
        return 0;
    }
    if (std::strcmp(name, "gemm_buffer_loads") == 0) {
        CNH_CHECK(value == 0 || value == 1, -2, "gemm_buffer_loads: 0 or 1");
        gemm_set_buffer_loads(value);
        return 0;
    }
    if (std::strcmp(name, "product_statements") == 0) {
        CNH_CHECK(value == 0 || value == 1, -2, "product_statements: 0 or 1");
        g_product_statements = value;
        return 0;
    }
    if (std::strcmp(name, "gemm_ksplit") == 0) {
        CNH_CHECK(value == 0 || value == 1, -2, "gemm_ksplit: 0 or 1");
        gemm_set_ksplit(value);
        return 0;
    }
    if (std::strcmp(name, "direct_lean") == 0) {
        g_direct_lean = value;
        return 0;
    }
    if (std::strcmp(name, "tiles_rows") == 0) {
        g_tiles_rows = value != 0;
        return 0;
    }
    if (std::strcmp(name, "direct_merge") == 0) {
        g_direct_merge = value != 0;
        return 0;
    }
    if (std::strcmp(name, "direct_stagger") == 0) {
        g_direct_stagger = value != 0;
        return 0;
    }
    if (std::strcmp(name, "direct_group") == 0) {
        g_direct_group = value;
        return 0;
    }
    if (std::strcmp(name, "direct_tx") == 0) {
        g_direct_cfg.tx = value;
        return 0;
    }
    if (std::strcmp(name, "direct_ry") == 0) {
        g_direct_cfg.ry = value;
        return 0;
    }
    if (std::strcmp(name, "direct_rz") == 0) {
        g_direct_cfg.rz = value;
        return 0;
    }
    if (std::strcmp(name, "slide2d_march") == 0) {
        g_slide_cfg.march2d = value != 0;
        return 0;
    }
    if (std::strcmp(name, "direct_flat") == 0) {
        g_direct_flat = value != 0;
        return 0;
    }
    if (std::strcmp(name, "block_pairs") == 0) {
        g_block_pairs = value != 0;
        return 0;
    }
    if (std::strcmp(name, "flat_nt_mib") == 0) {
        CNH_CHECK(value >= 0, -2, "threshold must not be negative");
        g_flat_nt_mib = value;
        return 0;
    }
    if (std::strcmp(name, "stencil_nt_mib") == 0) {
        CNH_CHECK(value >= 0, -2, "threshold must not be negative");
        g_stencil_nt_mib = value;
        return 0;
    }
    if (std::strcmp(name, "flat_tail") == 0) {
        g_flat_tail = value != 0;
        return 0;
    }
    if (std::strcmp(name, "flat_obz") == 0 || std::strcmp(name, "flat_oby") == 0 ||
        std::strcmp(name, "flat_obx") == 0) {
        CNH_CHECK(value >= 0, -2, "ordering block extent must not be negative");
        g_flat_ob[name[7] == 'z' ? 0 : (name[7] == 'y' ? 1 : 2)] = value;
        return 0;
    }
    if (std::strcmp(name, "slide_bx") == 0) {
        g_slide_cfg.bx = value;
        return 0;
    }
    if (std::strcmp(name, "slide_ry") == 0) {
        g_slide_cfg.ry = value;
        return 0;
    }
    if (std::strcmp(name, "slide_zc") == 0) {
        g_slide_cfg.zc = value;
        return 0;
    }
    if (std::strcmp(name, "slide_pd") == 0) {
        g_slide_cfg.pd = value;
        return 0;
    }
    return set_error(-2, "unknown option '%s'", name);
}

namespace {
int launch_group_tiles_impl(cnh_kernel* k, int n_in, const cnh_tiled* in, int n_scalar,
                            const void* const* scalars, int scalars_on_device, const cnh_tiled* cur,
                            const cnh_tiled* dst, cnh_stream s, RedReq* red);
}

extern "C" int cnh_launch_group_tiles(cnh_kernel* k, int n_in, const cnh_tiled* in, int n_scalar,
                                      const void* const* scalars, int scalars_on_device,
                                      const cnh_tiled* cur, const cnh_tiled* dst, cnh_stream s) {
    return launch_group_tiles_impl(k, n_in, in, n_scalar, scalars, scalars_on_device, cur, dst, s, nullptr);
}

extern "C" int cnh_launch_group_tiles_residual(cnh_kernel* k, int n_in, const cnh_tiled* in, int n_scalar,
                                               const void* const* scalars, int scalars_on_device,
                                               const cnh_tiled* cur, const cnh_tiled* dst, int mode,
                                               void* out, cnh_stream s) {
    CNH_CHECK(mode == 0 || mode == 1, -2, "residual mode %d is neither 0 (sum of squares) nor 1 (maximum)",
              mode);
    CNH_CHECK(out != nullptr && cur != nullptr && dst != nullptr, -2, "null argument");
    CNH_CHECK(k != nullptr && k->prog.dtype == CNH_F64, -2, "the residual forms need an fp64 group");
    CNH_CHECK(cur->tiles != nullptr && dst->tiles != nullptr && cur->tiles[0] != dst->tiles[0], -4,
              "a residual needs the old contents: cur and dst must be different buffers");
    RedReq red;
    red.mode = mode + 1;
    red.out = out;
    if (int rc = launch_group_tiles_impl(k, n_in, in, n_scalar, scalars, scalars_on_device, cur, dst, s, &red))
        return rc;
    if (red.done)
        return 0;
    // Not taken by a kernel that reduces on the way: a second pass over both buffers. Contiguous
    // tiles are one chunk each; views into one block without gaps are one chunk together.
    const int nd = dst->ndims;
    int64_t ntiles = 1, total = 1;
    for (int d = 0; d < nd; ++d) {
        ntiles *= dst->grid[d];
        total *= dst->shape[d];
    }
    std::vector<const void*> pa, pb;
    std::vector<int64_t> cnt;
    if (is_pitched(dst)) {
        bool gapless = dst->pitch[nd - 1] == 1;
        for (int d = nd - 2; d >= 0 && gapless; --d)
            gapless = dst->pitch[d] == dst->pitch[d + 1] * dst->shape[d + 1];
        for (int d = 0; d < nd && gapless; ++d)
            gapless = dst->offset[d] == 0;
        CNH_CHECK(gapless, -4, "residual over pitched views with gaps between rows or planes");
        pa.push_back(dst->tiles[0]);
        pb.push_back(cur->tiles[0]);
        cnt.push_back(total);
    } else {
        for (int64_t t = 0; t < ntiles; ++t) {
            int64_t rem = t, n = 1;
            for (int d = nd - 1; d >= 0; --d) {
                const int g = dst->grid_lo[d] + (int)(rem % dst->grid[d]);
                rem /= dst->grid[d];
                const int lo = std::max(g * dst->tile, dst->offset[d]);
                const int hi = std::min((g + 1) * dst->tile, dst->offset[d] + dst->shape[d]);
                n *= std::max(0, hi - lo);
            }
            pa.push_back(dst->tiles[t]);
            pb.push_back(cur->tiles[t]);
            cnt.push_back(n);
        }
    }
    if (mode == 0)
        return cnh_sumsq_diff_tiles((int)pa.size(), pa.data(), pb.data(), cnt.data(), out, s);
    return cnh_maxabs_diff_tiles((int)pa.size(), pa.data(), pb.data(), cnt.data(), out, s);
}

namespace {
int launch_group_tiles_impl(cnh_kernel* k, int n_in, const cnh_tiled* in, int n_scalar,
                            const void* const* scalars, int scalars_on_device, const cnh_tiled* cur,
                            const cnh_tiled* dst, cnh_stream s, RedReq* red) {
    if (int rc = ensure_init())
        return rc;
    CNH_CHECK(k != nullptr, -2, "null kernel");
    const GroupProgram& p = k->prog;
    const int nd = p.ndims;
    // Several roots: two to four SET_REGION roots that assign lattices of one array with the same
    // steps. Two of them may be the lattices of one colour of a red-black sweep (the lattice sweep
    // of the register-window kernel); otherwise they run as one scatter over arrays stored as one
    // block each, in place.
    const int nroots = (int)p.out_roots.size();
    bool multi = nroots >= 2 && nroots <= 4;
    for (int r = 0; r < nroots && multi; ++r) {
        multi = p.out_is_set_region[r] && p.out_target[r] == p.out_target[0] && !p.out_region[r].is_global;
        for (int d = 0; d < nd && multi; ++d)
            multi = p.out_region[r].step[d] == p.out_region[0].step[d];
    }
    CNH_CHECK(nroots == 1 || multi, -17,
              "the tiled launch needs one output root (or two to four SET_REGION roots on one array with the same steps)");
    CNH_CHECK(n_in == (int)p.leaves.size(), -4, "group expects %d tiled inputs, got %d",
              (int)p.leaves.size(), n_in);
    if (int rc = check_tiled(dst, nd, "dst"))
        return rc;
    if (cur) {
        if (int rc = check_tiled(cur, nd, "cur"))
            return rc;
        CNH_CHECK(cur->tile == dst->tile, -4, "cur and dst differ in tile edge");
        for (int d = 0; d < nd; ++d)
            CNH_CHECK(cur->offset[d] == dst->offset[d] && cur->shape[d] == dst->shape[d] &&
                          cur->pitch[d] == dst->pitch[d], -4, "cur and dst differ in decomposition");
    }
    for (int i = 0; i < n_in; ++i)
        if (int rc = check_tiled(&in[i], nd, "input"))
            return rc;
    std::vector<unsigned char> scal;
    if (int rc = pack_scalars(p, n_scalar, scalars, scalars_on_device, scal))
        return rc;
    hipStream_t st = as_stream(s);
    const int pad = CNH_MAX_ND - nd;

    // Assigned region (target coordinates) and the input region of every distinct load.
    int rs[3] = {0, 0, 0}, re[3] = {1, 1, 1}, rst[3] = {1, 1, 1};
    const bool set_region = p.out_is_set_region[0] && !p.out_region[0].is_global;
    for (int d = 0; d < nd; ++d) {
        if (set_region) {
            rs[pad + d] = p.out_region[0].start[d];
            re[pad + d] = p.out_region[0].stop[d];
            rst[pad + d] = p.out_region[0].step[d];
        } else {
            rs[pad + d] = 0;
            re[pad + d] = dst->shape[d];
            rst[pad + d] = 1;
        }
        CNH_CHECK(rst[pad + d] >= 1 && rs[pad + d] >= 0 && re[pad + d] <= dst->shape[d], -4,
                  "assigned region [%d:%d:%d] does not fit the target extent %d in dim %d",
                  rs[pad + d], re[pad + d], rst[pad + d], dst->shape[d], d);
    }
    const int NL = (int)p.load_leaf.size();
    const int NLA = NL > 0 ? NL : 1;
    std::vector<const cnh_tiled*> arrays;
    std::vector<int> leaf_array;   // per distinct load: index into `arrays`
    std::vector<int32_t> targs(13 + 7 * NLA, 0);   // TilesArgs of the generated kernel
    std::vector<std::array<int32_t, 3>> leaf_lim((size_t)NLA, std::array<int32_t, 3>{0, 0, 0});
    for (int d = 0; d < 3; ++d) {
        targs[d] = d >= pad ? dst->offset[d - pad] : 0;
        targs[3 + d] = rs[d];
        targs[6 + d] = re[d];
        targs[9 + d] = rst[d];
    }
    for (int l = 0; l < NL; ++l) {
        const LeafUse& u = p.leaves[p.load_leaf[l]];
        const cnh_tiled* arr = &in[p.load_leaf[l]];
        int ai = -1;
        for (size_t a = 0; a < arrays.size(); ++a)
            if (arrays[a]->tiles[0] == arr->tiles[0] && arrays[a]->tile == arr->tile &&
                std::memcmp(arrays[a]->offset, arr->offset, sizeof arr->offset) == 0 &&
                std::memcmp(arrays[a]->shape, arr->shape, sizeof arr->shape) == 0)
                ai = (int)a;
        if (ai < 0) {
            ai = (int)arrays.size();
            arrays.push_back(arr);
        }
        int32_t* lr = &targs[13 + 7 * l];
        lr[0] = ai;
        leaf_array.push_back(ai);
        for (int d = 0; d < 3; ++d) {
            lr[1 + d] = 0;
            lr[4 + d] = 1;
        }
        for (int d = 0; d < nd; ++d) {
            int start = u.has_region ? u.region.start[d] : 0;
            int stop = u.has_region ? u.region.stop[d] : arr->shape[d];
            int step = u.has_region ? u.region.step[d] : 1;
            CNH_CHECK(step >= 1, -4, "input %d: step %d in dim %d", l, step, d);
            int count = (stop - start + step - 1) / step;
            int ocount = (re[pad + d] - rs[pad + d] + rst[pad + d] - 1) / rst[pad + d];
            int owner = 0;                                // the root whose statement reads this leaf
            while (multi && owner + 1 < nroots && p.out_roots[owner] < u.root)
                owner++;
            if (owner > 0) {
                const cnh_region& r2 = p.out_region[owner];
                CNH_CHECK(r2.step[d] >= 1 && r2.start[d] >= 0 && r2.stop[d] <= dst->shape[d] && r2.stop[d] > r2.start[d], -4,
                          "assigned region %d [%d:%d:%d] does not fit the target extent %d in dim %d", owner,
                          r2.start[d], r2.stop[d], r2.step[d], dst->shape[d], d);
                ocount = (r2.stop[d] - r2.start[d] + r2.step[d] - 1) / r2.step[d];
            }
            leaf_lim[(size_t)l][pad + d] = count - 1;
            CNH_CHECK(count == ocount, -4,
                      "input %d has %d elements in dim %d, the assigned region has %d", l, count, d,
                      ocount);
            CNH_CHECK(start >= 0 && start + (count - 1) * step < arr->shape[d], -4,
                      "input %d: region [%d:%d:%d] leaves the array extent %d in dim %d", l, start,
                      stop, step, arr->shape[d], d);
            lr[1 + pad + d] = start;
            lr[4 + pad + d] = step;
        }
    }

    // Same-array unit-step stencil with ping-pong buffers: register-window or LDS sliding window.
    {
        bool handled = false;
        if (int rc = try_launch_direct(k, arrays, leaf_array, cur, dst, scal, st, &handled, red))
            return rc;
        if (handled)
            return 0;
        // the sliding-window kernel addresses a tile through its own extents; the general gather
        // below takes pitched views too
        bool pitched = is_pitched(dst) || (cur && is_pitched(cur));
        for (const cnh_tiled* a : arrays)
            pitched = pitched || is_pitched(a);
        if (!pitched && !multi)
            if (int rc = try_launch_slide(k, arrays, cur, dst, scal, st, &handled))
                return rc;
        if (handled)
            return 0;
    }

    // Every array of the launch one row-major block (or a single tile): the gather without tiles.
    if (g_tiles_block) {
        const int esz = dtype_size(p.dtype);
        int64_t dpitch[3] = {0, 0, 1}, cpitch[3] = {0, 0, 1};
        bool block = one_block_of(dst, esz, dpitch) &&
                     (cur == nullptr || (one_block_of(cur, esz, cpitch) && cpitch[0] == dpitch[0] && cpitch[1] == dpitch[1]));
        std::vector<std::array<int64_t, 3>> apitch(arrays.size(), std::array<int64_t, 3>{0, 0, 1});
        for (size_t a = 0; a < arrays.size() && block; ++a)
            block = one_block_of(arrays[a], esz, apitch[a].data()) && apitch[a][0] < (1ll << 31) && apitch[a][1] < (1ll << 31);
        block = block && dpitch[0] < (1ll << 31) && dpitch[1] < (1ll << 31);
        if (multi)
            // no root may read the assigned array: every lane stores to several lattices, and
            // nothing orders those stores against another lane's loads
            for (size_t a = 0; a < arrays.size() && block; ++a)
                block = arrays[a]->tiles[0] != dst->tiles[0];
        block = block && (!multi || cur == nullptr || cur->tiles[0] == dst->tiles[0]);
        // and the lattices must not share a point (the order of two stores to it would be open)
        for (int a = 0; a < nroots && multi && block; ++a)
            for (int b = a + 1; b < nroots && block; ++b) {
                bool apart = false;
                for (int d = 0; d < nd; ++d) {
                    const cnh_region &ra = p.out_region[a], &rb = p.out_region[b];
                    apart = apart || (ra.start[d] - rb.start[d]) % ra.step[d] != 0 ||
                            ra.stop[d] <= rb.start[d] || rb.stop[d] <= ra.start[d];
                }
                block = apart;
            }
        if (block) {
            BlockHeadDev h;
            std::memset(&h, 0, sizeof h);
            h.dst = dst->tiles[0];
            h.cur = cur ? cur->tiles[0] : nullptr;
            const bool in_place = h.cur == nullptr || h.cur == h.dst;
            for (int d = 0; d < 3; ++d) {
                h.shape[d] = d >= pad ? dst->shape[d - pad] : 1;
                h.rs[d] = rs[d];
                h.re[d] = re[d];
                h.rst[d] = rst[d];
                h.cnt[d] = std::max(0, (re[d] - rs[d] + rst[d] - 1) / rst[d]);
            }
            h.dpy = (int32_t)dpitch[1];
            h.dpz = (int32_t)dpitch[0];
            h.lattice = in_place ? 1 : 0;
            if (multi) {
                h.nroots = nroots;
                for (int r = 0; r < nroots; ++r)
                    for (int d = 0; d < 3; ++d) {
                        const cnh_region& rr = p.out_region[r];
                        h.rrs[r][d] = d >= pad ? rr.start[d - pad] : 0;
                        h.rcnt[r][d] = d >= pad ? std::max(0, (rr.stop[d - pad] - rr.start[d - pad] + rr.step[d - pad] - 1) / rr.step[d - pad]) : 1;
                        CNH_CHECK(d < pad || (rr.start[d - pad] >= 0 && rr.stop[d - pad] <= dst->shape[d - pad]), -4,
                                  "assigned region %d leaves the target in dim %d", r, d - pad);
                        h.cnt[d] = r == 0 ? h.rcnt[r][d] : std::max(h.cnt[d], h.rcnt[r][d]);
                    }
                // lattices side by side along the rows (step 2, the same rows, first columns one
                // apart) are stored as pairs of elements
                for (int r = 0; r < 4; ++r)
                    h.rmate[r] = -1;
                for (int r = 0; r < nroots && g_block_pairs && h.rst[2] == 2; ++r)
                    for (int m = 0; m < nroots && h.rmate[r] == -1; ++m)
                        if (m != r && h.rmate[m] == -1 && h.rrs[m][2] == h.rrs[r][2] + 1 &&
                            h.rrs[m][0] == h.rrs[r][0] && h.rrs[m][1] == h.rrs[r][1] &&
                            h.rcnt[m][0] == h.rcnt[r][0] && h.rcnt[m][1] == h.rcnt[r][1]) {
                            h.rmate[r] = m;
                            h.rmate[m] = -2;
                        }
            }
            // unit steps along the rows everywhere, in place, one root: pairs of elements per access
            bool pairs = in_place && !multi && g_block_pairs && rst[2] == 1 && NL > 0;
            for (int l = 0; l < NL && pairs; ++l)
                pairs = targs[13 + 7 * l + 4 + 2] == 1;
            int64_t W2 = in_place ? h.cnt[2] : h.shape[2];
            const int64_t rows = in_place ? (int64_t)h.cnt[0] * h.cnt[1] : (int64_t)h.shape[0] * h.shape[1];
            if (rows <= 0 || W2 <= 0)
                return 0;
            if (pairs)
                W2 = (W2 + 1) / 2;              // geometry in pairs: a lane takes two of them
            const int per_lane = pairs ? 2 : 4;
            int lanes = 16;
            while (lanes < 256 && lanes * per_lane < W2)
                lanes *= 2;
            int rsh = 0;
            while (g_tiles_rows && (256 >> rsh) > lanes && (1 << rsh) < rows)
                rsh++;
            lanes = 256 >> rsh;
            const int64_t nchunks = (W2 + lanes * per_lane - 1) / (lanes * per_lane);
            // padded to a multiple of 8: every XCD takes a contiguous eighth of the workgroups
            const int64_t nblocks = (((rows + (1 << rsh) - 1) >> rsh) * nchunks + 7) / 8 * 8;
            if (nblocks < (1ll << 31) && rows < (1ll << 31)) {
                h.nchunks = (int32_t)nchunks;
                h.rsh = rsh;
                h.nblk8 = (int32_t)(nblocks / 8);
                std::vector<unsigned char> args(sizeof h + (size_t)NLA * sizeof(BlockLeafDev), 0);
                std::memcpy(args.data(), &h, sizeof h);
                for (int l = 0; l < NL; ++l) {
                    const int32_t* lr = &targs[13 + 7 * l];
                    BlockLeafDev lf;
                    lf.base = arrays[(size_t)lr[0]]->tiles[0];
                    lf.py = (int32_t)apitch[(size_t)lr[0]][1];
                    lf.pz = (int32_t)apitch[(size_t)lr[0]][0];
                    for (int d = 0; d < 3; ++d) {
                        lf.start[d] = lr[1 + d];
                        lf.step[d] = lr[4 + d];
                        lf.lim[d] = leaf_lim[(size_t)l][d];
                    }
                    lf.unused = 0;
                    std::memcpy(args.data() + sizeof h + (size_t)l * sizeof lf, &lf, sizeof lf);
                }
                hipFunction_t fn;
                const char* name = multi   ? (rsh > 0 ? "grp_scatter_rows" : "grp_scatter")
                                   : pairs ? (rsh > 0 ? "grp_block_pairs_rows" : "grp_block_pairs")
                                           : (rsh > 0 ? "grp_block_rows" : "grp_block");
                if (int rc = get_function(k, "tiles", name, &fn))
                    return rc;
                void* params[] = {args.data(), scal.data()};
                return launch(fn, nblocks, params, st);
            }
        }
    }

    CNH_CHECK(!multi, -17, "a group with several SET_REGION roots runs in place over arrays stored as one block "
              "each, as a lattice sweep (two roots that read the array between their points) or as a scatter "
              "(roots that do not read it), and this one fits neither");
    // Destination tiles.
    int64_t ntiles = 1;
    for (int d = 0; d < nd; ++d)
        ntiles *= dst->grid[d];
    std::vector<DTileDev> dts;
    int64_t blocks = 0;
    bool lattice = false, any_rows = false;
    for (int64_t t = 0; t < ntiles; ++t) {
        int ti[3] = {0, 0, 0};
        int64_t rem = t;
        for (int d = nd - 1; d >= 0; --d) {
            ti[d] = (int)(rem % dst->grid[d]);
            rem /= dst->grid[d];
        }
        DTileDev dt;
        std::memset(&dt, 0, sizeof dt);
        for (int d = 0; d < 3; ++d) {
            dt.cs[d] = 0;
            dt.w[d] = 1;
        }
        bool empty = false;
        for (int d = 0; d < nd; ++d) {
            int g = dst->grid_lo[d] + ti[d];
            int lo = std::max(g * dst->tile, dst->offset[d]);
            int hi = std::min((g + 1) * dst->tile, dst->offset[d] + dst->shape[d]);
            if (hi <= lo)
                empty = true;
            dt.cs[pad + d] = lo;
            dt.w[pad + d] = hi - lo;
        }
        if (empty)
            continue;
        dt.dst = dst->tiles[t];
        dt.cur = cur ? cur->tiles[t] : nullptr;
        dt.py = nd >= 2 ? (int32_t)dst->pitch[nd - 2] : 0;
        dt.pz = nd >= 3 ? (int32_t)dst->pitch[0] : 0;
        // In place (or with nothing to copy from), elements outside the assigned region keep
        // their values without being touched: the launch walks the points of the region's index
        // lattice that fall into the tile (bs = index of the first one along each dimension,
        // bw = how many), and skips tiles the region misses. A ping-pong launch writes every
        // element of the new buffer and walks the whole tile.
        const bool in_place = dt.cur == nullptr || dt.cur == dt.dst;
        lattice = in_place;
        for (int d = 0; d < 3; ++d) {
            dt.bs[d] = 0;
            dt.bw[d] = dt.w[d];
            if (in_place && d >= pad) {
                const int off = dst->offset[d - pad];
                const int lo = std::max(dt.cs[d], rs[d] + off) - off;           // array coordinates
                const int hi = std::min(dt.cs[d] + dt.w[d], re[d] + off) - off;
                if (hi <= lo) {
                    empty = true;
                    continue;
                }
                const int kfirst = (lo - rs[d] + rst[d] - 1) / rst[d];          // first index with point >= lo
                const int klast = (hi - 1 - rs[d]) / rst[d];                    // last index with point < hi
                if (klast < kfirst)
                    empty = true;
                dt.bs[d] = kfirst;
                dt.bw[d] = klast - kfirst + 1;
            }
        }
        if (empty)
            continue;
        // Four elements per lane along the last dimension. A row shorter than 1024 elements
        // shares its workgroup with the rows after it: 2^rsh rows of 256 >> rsh lanes each.
        const int64_t rows = (int64_t)dt.bw[0] * dt.bw[1];
        int lanes = 16;
        while (lanes < 256 && lanes * 4 < dt.bw[2])
            lanes *= 2;
        dt.rsh = 0;
        while (g_tiles_rows && (256 >> dt.rsh) > lanes && (1 << dt.rsh) < rows)
            dt.rsh++;
        lanes = 256 >> dt.rsh;
        dt.nchunks = (dt.bw[2] + lanes * 4 - 1) / (lanes * 4);
        dt.blk0 = blocks;
        blocks += ((rows + (1 << dt.rsh) - 1) >> dt.rsh) * dt.nchunks;
        any_rows = any_rows || dt.rsh > 0;
        dts.push_back(dt);
    }
    if (dts.empty())
        return 0;
    targs[12] = lattice ? 1 : 0;

    std::vector<TiledDev> adev(arrays.size() ? arrays.size() : 1);
    for (size_t a = 0; a < arrays.size(); ++a)
        if (int rc = make_tiled_dev(arrays[a], st, adev[a]))
            return rc;
    const void* d_arrs = nullptr;
    const void* d_dts = nullptr;
    if (int rc = desc_upload(adev.data(), adev.size() * sizeof(TiledDev), st, &d_arrs))
        return rc;
    if (int rc = desc_upload(dts.data(), dts.size() * sizeof(DTileDev), st, &d_dts))
        return rc;
    hipFunction_t fn;
    if (int rc = get_function(k, "tiles", any_rows ? "grp_tiles_rows" : "grp_tiles", &fn))
        return rc;
    int ndt = (int)dts.size();
    void* params[] = {&d_arrs, &d_dts, &ndt, targs.data(), scal.data()};
    return launch(fn, blocks, params, st);
}
} // namespace
