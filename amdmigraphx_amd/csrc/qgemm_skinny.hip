// quant_dot for few rows (M <= 128 against a large [K, N] weight): these shapes
// move far more weight bytes than they do arithmetic, so they are bound by HBM
// and want the whole chip streaming B, which a 256 x 256 output tiling cannot
// provide (N / 256 workgroups).  Not specialised yet: every shape is served by
// the tiled MFMA kernel or the any-stride kernel.
#include "common.h"

bool mi355_skinny_gemm_supported(const mi355_quant_dot_desc*, const void*, const void*, const void*)
{
    return false;
}

int mi355_skinny_gemm_launch(const mi355_quant_dot_desc*,
                             const void*,
                             const void*,
                             void*,
                             const float*,
                             const float*,
                             const int32_t*,
                             const int32_t*,
                             hipStream_t)
{
    return MI355_ERR_UNSUPPORTED;
}
