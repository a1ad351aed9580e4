// AST -> HIP source for one fused group. Host-only (no device code here).
// The numerical definition of a group follows the upstream JIT (src/jit.cpp:28-150,223-459):
// roots are evaluated in list order, every op is one IEEE operation in the group's element type,
// scalar leaves are constants cast to that type, size-1 arrays are run-time scalars.
#pragma once

#include <array>
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
    // Literal scalars that are passed with the launch instead of being written into the source
    // (s[NS + i] in the body): the text, and with it the code object, does not depend on them.
    std::vector<double> lit_values;
    std::vector<int> out_names;   // result name of each output root
    std::vector<int> out_roots;   // root positions of the non-temp roots
    std::vector<int> out_is_set_region;
    std::vector<int> out_reduce;  // 0: stored element by element; 1: summed, 2: largest |value|,
                                  // 3: a value without an index, stored once (CNH_OP_SCALAR_OF)
    std::vector<int> out_target;  // SET_REGION target array name (or result name)
    std::vector<cnh_region> out_region; // SET_REGION region (is_global when absent)
    std::vector<std::string> out_expr;  // value expression of each output
    std::string body;             // statements computing t<k> from l<load>, s<bcast>
    bool uses_transcendental = false;
    // outputs that are not stored element by element (dense launches only)
    int reductions() const {
        int n = 0;
        for (int r : out_reduce)
            n += r != 0;
        return n;
    }
    // those of them that are reduced over the launch and leave partial results
    int folds() const {
        int n = 0;
        for (int r : out_reduce)
            n += r == 1 || r == 2;
        return n;
    }
};

// Returns 0 or a negative code with the reason in `err` for an AST the upstream JIT could not
// compile either (tanh/exp on integers, a unary op on a scalar, unknown opcodes).
int build_group_program(const cnh_ast* ast, int dtype, int ndims, GroupProgram& out,
                        std::string& err);
// The value of literal scalar `c` in element type `dtype`, as the generated source would spell it
// (integers cast through int64, floats through double; src/jit.cpp:108-116 upstream), written to
// out (4 or 8 bytes).
void literal_value(int dtype, double c, void* out);

// Launch geometry of the sliding-window variant. Kernel dimensions are (march, row, column).
// A rank-3 array maps to them one to one. A rank-2 array maps to (-, dim0, dim1) — one patch per
// workgroup, nothing to march — or, with march2d, to (dim0, -, dim1): a row strip marched down.
// Overrides of the built-in geometry (0 = keep the default); the variant name carries them.
struct SlideConfig {
    int march2d = 1, bx = 0, ry = 0, zc = 0, pd = 0;
    std::string variant() const;                      // "slide" or "slide@m,bx,ry,zc,pd"
    static bool parse(const std::string& variant, SlideConfig& out);
};
struct SlideShape {
    bool march2d = false;
    int halo[3] = {0, 0, 0};
    int bx = 0, ty = 0, ry = 0, zc = 0, pd = 1;       // patch width, lane rows, rows per lane,
                                                       // march chunk, planes in flight
    std::vector<std::array<int, 3>> shifts; // per distinct load, in kernel dimensions
    int kdim(int ndims, int d) const {
        if (ndims == 3)
            return d;
        return march2d ? (d == 0 ? 0 : 2) : d + 1;
    }
};
// 0 when the group is a same-array unit-step stencil the sliding-window variant can run.
int slide_shape(const GroupProgram& p, const SlideConfig& cfg, SlideShape& sh, std::string& err);

// Register-window stencil variant (no LDS): lane grid tx x (256/tx), ry rows and rz planes per lane.
struct DirectConfig {
    int tx = 0, ry = 0, rz = 0;                       // 0 = built-in default
    bool reduce = false;                              // the forms that also reduce what they change
    std::string variant() const;                      // "direct@tx,ry,rz" or "directr@tx,ry,rz"
    static bool parse(const std::string& variant, DirectConfig& out);
};
struct DirectShape {
    int halo[3] = {0, 0, 0};
    int tx = 0, ty = 0, ry = 0, rz = 0;
    std::vector<std::array<int, 3>> shifts; // per distinct load, dims padded to (z, y, x)
    std::vector<std::array<int, 3>> shifts2; // the same for the second root of a lattice pair (a load
                                             // both roots use may sit at another offset from each lattice)
    // per distinct load: -1 = the assigned array itself (read through the window), else which of
    // the other arrays it reads at the element's own position (source terms, weights)
    std::vector<int> other;
    std::vector<int> other_names; // array names in the order the indices above number them
    // The array read through the window. Usually the assigned one (a sweep in place); when only
    // another array is read at shifted positions (unew[interior] = f(u shifted)), that one: the
    // launch then reads its tiles and writes the assigned elements of the target, nothing else.
    int window_name = 0;
    bool masked = false;
    // Lattices: every region of the group has the same step (1 or 2) per dimension, lat[d] = step - 1
    // in kernel dimensions (z, y, x). One or two SET_REGION roots on the same array whose lattices
    // share no point (the two halves of one colour of a red-black sweep). inplace_safe: no shifted
    // read of the assigned array can meet an assigned point, so the sweep may run in place.
    int lat[3] = {0, 0, 0};
    int nroots = 1;
    bool lattice = false, inplace_safe = false;
    // Every output row of a lane holds the pair to the right of the wavefront's 128 columns (some
    // load reads the window array at (0, 0, +1) or (0, 0, +2)): the last lane of a row's last
    // wavefront can then copy one or two columns beyond it that no statement assigns, which saves
    // the workgroups a 128 k + 1 (or + 2) wide array would otherwise launch for them.
    bool tail_ok = false;
    // Some array other than the window array is read at shifted positions too (two arrays of a
    // staggered or variable-coefficient stencil): the whole-array kernel then keeps a window per
    // array; the per-tile kernels do not take such groups.
    bool other_shifted = false;
};
constexpr int kDirectMaxOther = 4;
int direct_shape(const GroupProgram& p, const DirectConfig& cfg, DirectShape& sh, std::string& err);

// Source text of a kernel variant. `variant` is one of "flat", "nd", "tiles", "slide".
int emit_variant_source(const GroupProgram& p, const std::string& variant, std::string& src,
                        std::string& err);

const char* dtype_ctype(int dtype);

// Text of the fp64 matrix-core product kernel (gemm_kernel.inc), for the variant that appends a
// group's statements to it (codegen_product.cpp).
std::string gemm_kernel_text();

// fp64 exp/tanh restated to agree bit for bit with the host C library (codegen_libm.cpp).
std::string libm_f64_text();
std::string libm_f32_text();

} // namespace cnh
