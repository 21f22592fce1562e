// Launcher of the large-tile implicit GEMM (big_gemm_kernel.h).  It lives in a translation unit of its own because that
// kernel keeps its accumulators in AGPRs, while the rest of the library is compiled with MFMA results in VGPRs.
#pragma once

#include "conv_kernels.h"

namespace mi355x
{

// Block tile bm x bn must be one of 256x256, 256x128, 128x256; needs a.Ci % 128 == 0, a.K_pad % 128 == 0 and a weight
// matrix of at least ceil(Co / bn) * bn rows.  Fills a.tiles_m / a.tiles_n itself.
int LaunchBigGemm(IgemmArgs a, int bm, int bn, hipStream_t stream);

// One-time set-up of the kernels' dynamic LDS limits (called at plan creation, outside any graph capture).
int PrepareBigGemm();

} // namespace mi355x
