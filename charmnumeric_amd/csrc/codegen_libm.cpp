// Device text of the fp64 exp/tanh that match the host C library bit for bit.
#include "codegen.h"

#include <cstdio>

namespace cnh {

namespace {
const unsigned long long kExpTab[256] = {
#include "exp_table.inc"
};
const char* kLibmBody =
#include "libm_f64.inc"
    ;
const unsigned long long kExp2fTab[32] = {
#include "exp2f_table.inc"
};
const char* kLibmBodyF32 =
#include "libm_f32.inc"
    ;
} // namespace

std::string libm_f64_text() {
    std::string s = "#define CN_DEV __device__ __forceinline__\n"
                    "__device__ const unsigned long long CN_EXP_TAB[256] = {\n";
    char buf[32];
    for (int i = 0; i < 256; ++i) {
        std::snprintf(buf, sizeof buf, "0x%016llxull,%s", kExpTab[i], (i % 4 == 3) ? "\n" : " ");
        s += buf;
    }
    s += "};\n";
    s += kLibmBody;
    return s;
}

std::string libm_f32_text() {
    std::string s = "#define CN_DEV __device__ __forceinline__\n"
                    "__device__ const unsigned long long CN_EXP2F_TAB[32] = {\n";
    char buf[32];
    for (int i = 0; i < 32; ++i) {
        std::snprintf(buf, sizeof buf, "0x%016llxull,%s", kExp2fTab[i], (i % 4 == 3) ? "\n" : " ");
        s += buf;
    }
    s += "};\n";
    s += kLibmBodyF32;
    return s;
}

} // namespace cnh
