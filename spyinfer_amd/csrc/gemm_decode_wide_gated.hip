// The gated decode product (gate/up with the SwiGLU in the epilogue) whose blocks walk runs of column tiles; see
// gemm_decode_wide.h.
#include "gemm_decode_wide.h"

bool gd_wide_gated(const GdArgs& a, bool f32_out) {
    if (f32_out) return wide_rows<EPI_GATED, float, false>(a);
    return a.ot ? wide_rows<EPI_GATED, bf16_t, true>(a) : wide_rows<EPI_GATED, bf16_t, false>(a);
}
