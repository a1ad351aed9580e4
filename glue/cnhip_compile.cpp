// ArrayDAGGroup::compile_node on libcnhip: the AST of a fusible DAG node is flattened into the
// node array of include/cnhip.h and handed to cnh_compile_group, which generates and caches HIP
// source for the group (hipRTC builds a variant on its first launch).
// Replaces src/dag_group_compile.cpp:6-41 upstream; ArrayDAGGroup::compile (:43-56) stays as it
// is: it stores the returned pointer in compile_cache[node->identifier] and a null pointer still
// means "interpreter fallback" (src/execute_node.cpp:102-112).
// Not compiled in this repository (needs charm++.h and charmtyles).
#include "backend.hpp"

#include <unordered_map>
#include <vector>

#include "cnhip.h"

namespace {

// Region* of charmtyles -> cnh_region. A null or global region means "the whole array".
cnh_region to_cnh_region(const Region* r, int ndims) {
    cnh_region out = {};
    if (r == nullptr || r->is_global) {
        out.is_global = 1;
        return out;
    }
    out.ndims = ndims;
    // ArrayRegion<N> keeps start/stop/step as std::array<int, N> (src/array_region.hpp:21-33)
    auto fill = [&](const auto* ar) {
        for (int d = 0; d < ndims; ++d) {
            out.start[d] = ar->start[d];
            out.stop[d] = ar->stop[d];
            out.step[d] = ar->step[d];
        }
    };
    switch (ndims) {
    case 1: fill(static_cast<const ArrayRegion<1>*>(r)); break;
    case 2: fill(static_cast<const ArrayRegion<2>*>(r)); break;
    case 3: fill(static_cast<const ArrayRegion<3>*>(r)); break;
    default: out.is_global = 1; out.ndims = 0; break;
    }
    return out;
}

// Copies `n` and, first, everything below it into `flat`; returns the index of `n`'s copy.
// Leaves (NOOP / CREATE nodes, scalars, broadcast arrays) are copied once per pointer, so a leaf
// used by several roots is one entry; the kernel's argument list is still one memref per leaf USE,
// which cnh_compile_group derives from the operand slots (src/jit.cpp:223-263 upstream).
int flatten(const ASTNode* n, std::vector<cnh_ast_node>& flat,
            std::unordered_map<const ASTNode*, int>& seen) {
    auto hit = seen.find(n);
    if (hit != seen.end())
        return hit->second;
    int operand_index[2] = {-1, -1};
    const int n_operands = (int)n->operands.size();
    for (int i = 0; i < n_operands && i < 2; ++i)
        operand_index[i] = flatten(n->operands[i], flat, seen);

    cnh_ast_node c = {};
    c.result_name = n->result_name;
    c.opcode = n->opcode;
    c.is_temp = n->is_temp ? 1 : 0;
    c.is_scalar = n->is_scalar ? 1 : 0;
    c.is_broadcast = n->is_broadcast ? 1 : 0;
    c.ndims = n->ndims;
    c.dtype = static_cast<int>(n->dtype);          // wire values 0..3, charmnumeric.py:34-40
    c.scalar = n->scalar;                          // always read as double, src/jit.cpp:111-113
    c.n_operands = n_operands < 2 ? n_operands : 2;
    for (int i = 0; i < 2; ++i) {
        c.operands[i] = operand_index[i];
        c.operand_regions[i].is_global = 1;
    }
    for (int i = 0; i < c.n_operands; ++i) {
        const Region* r = n->get_operand_region(i);
        if (r != nullptr && !r->is_global) {
            c.has_operand_region[i] = 1;
            c.operand_regions[i] = to_cnh_region(r, n->operands[i]->ndims);
        }
    }
    c.region = to_cnh_region(n->region, n->ndims);
    flat.push_back(c);
    const int at = (int)flat.size() - 1;
    seen.emplace(n, at);
    return at;
}

// Element type of the group: the first root that is not FLOAT32 decides (src/jit.cpp:50-69).
int group_dtype(const AST* ast) {
    for (const ASTNode* root : ast->roots)
        if (root->dtype != DType::FLOAT32)
            return static_cast<int>(root->dtype);
    return CNH_F32;
}

} // namespace

void* ArrayDAGGroup::compile_node(DAGNode* node) {
    std::vector<cnh_ast_node> flat;
    std::vector<int32_t> roots;
    std::unordered_map<const ASTNode*, int> seen;
    for (const ASTNode* root : node->ast->roots)       // temporaries first, as the AST lists them
        roots.push_back(flatten(root, flat, seen));
    if (roots.empty())
        return nullptr;

    cnh_ast ast;
    ast.n_nodes = (int32_t)flat.size();
    ast.n_roots = (int32_t)roots.size();
    ast.nodes = flat.data();
    ast.roots = roots.data();

    int rank = 1;
    for (int r : roots)
        rank = flat[r].ndims > rank ? flat[r].ndims : rank;

    cnh_kernel* kernel = nullptr;
    if (cnh_compile_group(&ast, group_dtype(node->ast), rank, (uint64_t)node->identifier, &kernel) != 0) {
        DBG_PRINT("[PE %d] compile_node %ld: %s -> interpreter\n", CkMyPe(), (long)node->identifier,
                  cnh_last_error());
        return nullptr;                                 // same contract as a failed JIT build
    }
    module_cache[node->identifier] = kernel;            // released with cnh_kernel_release on teardown
    return kernel;
}
