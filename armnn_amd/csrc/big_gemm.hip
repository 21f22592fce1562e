// Large-tile implicit GEMM: kernel instantiations and launcher (see big_gemm.h for why this is a separate file).
#include "big_gemm.h"

#include <algorithm>
#include <cmath>

#include "big_gemm_kernel.h"

namespace mi355x
{
namespace
{

template <int BM, int BN, int ST, bool U8, bool AW>
int SetLimit()
{
    MI355X_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&BigGemmKernel<BM, BN, ST, U8, AW, true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   BigGemmSmemBytes<BM, BN, ST>()));
    MI355X_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&BigGemmKernel<BM, BN, ST, U8, AW, false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   BigGemmSmemBytes<BM, BN, ST>()));
    return 0;
}

template <int BM, int BN, int ST>
int SetLimits()
{
    if (int rc = SetLimit<BM, BN, ST, false, false>()) return rc;
    if (int rc = SetLimit<BM, BN, ST, true, false>()) return rc;
    if (int rc = SetLimit<BM, BN, ST, false, true>()) return rc;
    return SetLimit<BM, BN, ST, true, true>();
}

template <int BM, int BN, int ST, bool U8, bool AW>
int Launch(IgemmArgs a, hipStream_t stream)
{
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.Co + BN - 1) / BN;
    const int nblocks = a.tiles_m * a.tiles_n;
    // tile rows an XCD walks together: its run of tiles is about as tall as it is wide, in elements
    const double per_xcd = std::max(1.0, nblocks / 8.0);
    int xcd_rows = static_cast<int>(std::lround(std::sqrt(per_xcd * BN / BM)));
    xcd_rows = std::max(1, std::min(xcd_rows, a.tiles_m));
    const int grid = (nblocks + 7) / 8 * 8;
    constexpr int smem = BigGemmSmemBytes<BM, BN, ST>();
    NoteKernel("BigGemmKernel<%d, %d, %d, %s, %s, %s>", BM, BN, ST, BoolName(U8), BoolName(AW), BoolName(a.unit != 0));
    if (a.unit) hipLaunchKernelGGL((BigGemmKernel<BM, BN, ST, U8, AW, true>), dim3(grid), dim3(256), smem, stream, a, xcd_rows);
    else hipLaunchKernelGGL((BigGemmKernel<BM, BN, ST, U8, AW, false>), dim3(grid), dim3(256), smem, stream, a, xcd_rows);
    MI355X_HIP(hipGetLastError());
    return 0;
}

template <int BM, int BN, int ST>
int LaunchFlags(const IgemmArgs& a, hipStream_t stream)
{
    const bool u8 = a.xor_mask != 0, aw = a.zw_neg != 0;
    if (aw) return u8 ? Launch<BM, BN, ST, true, true>(a, stream) : Launch<BM, BN, ST, false, true>(a, stream);
    return u8 ? Launch<BM, BN, ST, true, false>(a, stream) : Launch<BM, BN, ST, false, false>(a, stream);
}

} // namespace

int PrepareBigGemm()
{
    static const int rc = [] {
        if (int r = SetLimits<256, 256, 2>()) return r;
        if (int r = SetLimits<256, 128, 3>()) return r;
        return SetLimits<128, 256, 3>();
    }();
    return rc;
}

int LaunchBigGemm(IgemmArgs a, int bm, int bn, hipStream_t stream)
{
    if ((a.Ci % 128) != 0 || (a.K_pad % 128) != 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "large-tile GEMM needs channels %% 128 == 0");
    if (!a.unit && a.Kh * a.Kw > 32) return SetError(MI355X_ERR_UNSUPPORTED, "large-tile GEMM: filters of more than 32 taps are not supported");
    if (a.M <= 0) return 0;
    if (int rc = PrepareBigGemm()) return rc;
    if (bm == 256 && bn == 256) return LaunchFlags<256, 256, 2>(a, stream);
    if (bm == 256 && bn == 128) return LaunchFlags<256, 128, 3>(a, stream);
    if (bm == 128 && bn == 256) return LaunchFlags<128, 256, 3>(a, stream);
    return SetError(MI355X_ERR_INVALID_ARGUMENT, "no large-tile GEMM of %d x %d", bm, bn);
}

} // namespace mi355x
