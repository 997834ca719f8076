// Decode products for matrices of many columns (the output head, other stored products): blocks that walk runs of column
// tiles.  Part of the decode products of gemm_decode.hip; the gated product is built in gemm_decode_wide_gated.hip.
#include "gemm_decode_wide.h"

bool gd_wide_gated(const GdArgs& a, bool f32_out);

bool gd_wide_try(const GdArgs& a, int epi, bool scaled, bool f32_out) {
    if (!scaled || !a.xt || a.M > 128 || a.N % 16 != 0 || a.K % GD_CHUNK != 0) return false;
    if (epi == EPI_STORE) return f32_out ? wide_rows<EPI_STORE, float, false>(a) : wide_rows<EPI_STORE, bf16_t, false>(a);
    if (epi == EPI_GATED) return gd_wide_gated(a, f32_out);
    return false;
}
