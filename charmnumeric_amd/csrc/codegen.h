// AST -> HIP source for one fused group. Host-only (no device code here).
// The numerical definition of a group follows the upstream JIT (src/jit.cpp:28-150,223-459):
// roots are evaluated in list order, every op is one IEEE operation in the group's element type,
// scalar leaves are constants cast to that type, size-1 arrays are run-time scalars.
#pragma once

#include <string>
#include <vector>

#include "common.h"

namespace cnh {

struct LeafUse {
    int node;        // index into the AST node array
    int root;        // position in the root list
    int operand;     // operand slot of that root
    int load;        // index of the distinct load this use maps to
    int name;        // array name (result_name of the leaf)
    bool has_region; // an explicit, non-global region is attached
    cnh_region region;
};

struct GroupProgram {
    int dtype = CNH_F32;
    int ndims = 1;
    std::vector<LeafUse> leaves;  // argument order: one memref per leaf use
    std::vector<int> load_leaf;   // distinct load -> the leaf use that supplies its memref
    std::vector<int> bcast_nodes; // one run-time scalar per unique broadcast leaf
    std::vector<int> bcast_names; // array name of each broadcast leaf
    std::vector<int> out_names;   // result name of each output root
    std::vector<int> out_roots;   // root positions of the non-temp roots
    std::vector<int> out_is_set_region;
    std::vector<int> out_target;  // SET_REGION target array name (or result name)
    std::vector<cnh_region> out_region; // SET_REGION region (is_global when absent)
    std::vector<std::string> out_expr;  // value expression of each output
    std::string body;             // statements computing t<k> from l<load>, s<bcast>
    bool uses_transcendental = false;
};

// Returns 0 or a negative code with the reason in `err` for an AST the upstream JIT could not
// compile either (tanh/exp on integers, a unary op on a scalar, unknown opcodes).
int build_group_program(const cnh_ast* ast, int dtype, int ndims, GroupProgram& out,
                        std::string& err);

// Source text of a kernel variant. `variant` is one of "flat", "nd", "tiles", "slide".
int emit_variant_source(const GroupProgram& p, const std::string& variant, std::string& src,
                        std::string& err);

const char* dtype_ctype(int dtype);

} // namespace cnh
