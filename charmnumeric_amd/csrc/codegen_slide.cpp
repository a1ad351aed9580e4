// Sliding-window (LDS ring) source for same-array unit-step stencils.
#include "codegen.h"

namespace cnh {

std::string slide_source(const GroupProgram&, std::string& err) {
    err = "sliding-window variant not available for this group";
    return std::string();
}

} // namespace cnh
