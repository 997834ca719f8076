#include "common.h"
extern "C" int spy_gemm_skinny() { return spy_fail("spy_gemm_skinny: not built yet"); }
