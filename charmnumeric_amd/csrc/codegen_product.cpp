// Text of the matrix-core product kernel for run-time compilation with a group's statements.
#include "codegen.h"

namespace cnh {

namespace {
const char* kGemmKernel =
#include "build/gemm_kernel_text.inc"
    ;
} // namespace

std::string gemm_kernel_text() { return kGemmKernel; }

} // namespace cnh
