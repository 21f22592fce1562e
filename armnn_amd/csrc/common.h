// Internal helpers shared by the device library's translation units (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "armnn_mi355x.h"

namespace mi355x
{

// thread-local message behind mi355x_last_error()
char* ErrorBuffer();
int SetError(int code, const char* fmt, ...);

// Records the name of the kernel the calling thread is about to launch, as a profiler would list it (without the
// namespace and the argument list); mi355x_last_kernel() returns it.  Measurement support: lets a benchmark label its
// per-layer timings with kernel symbols.
void NoteKernel(const char* fmt, ...);
inline const char* BoolName(bool b) { return b ? "true" : "false"; }

inline int HipFail(hipError_t e, const char* what)
{
    return SetError(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

#define MI355X_HIP(expr)                                             \
    do {                                                             \
        hipError_t e_ = (expr);                                      \
        if (e_ != hipSuccess) return ::mi355x::HipFail(e_, #expr);   \
    } while (0)

inline hipStream_t ToHip(mi355x_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool IsActivationDtype(int32_t d) { return d == MI355X_QASYMM_S8 || d == MI355X_QASYMM_U8; }

// armnn::Quantize (src/armnn/TypesUtils.cpp:29-45) on the host, used to turn activation bounds into codes
int32_t QuantizeHost(float value, float scale, int32_t offset, int32_t dtype);

// Integer clamp equivalent to an Activation layer that follows a layer with the same output quantization:
// q2 = clamp(q1, Quantize(b), Quantize(a)) for BoundedReLu, clamp(q1, Quantize(0), type max) for ReLu.
void ActivationClamp(int32_t activation, float a, float b, const mi355x_quant& out, int32_t* lo, int32_t* hi);

// Parameters of the shared requantization epilogue
struct Requant
{
    float   out_scale;
    float   out_offset_f;   // float(offset)
    float   type_min_f;     // float(lowest) of the output type
    float   type_max_f;
    int32_t act_lo;         // fused activation clamp in the quantized domain (already within the type range)
    int32_t act_hi;
    int32_t out_is_u8;
    // fast path: multiply by fl(1/scale) instead of dividing; exact division is redone only for values that land
    // within kTieWindow of a rounding tie, so the result is bit-identical to the division everywhere
    float   inv_scale;
    float   act_lo_f, act_hi_f;
    int32_t fast_ok;
    // Convolution / FullyConnected epilogue: codes are produced as unsigned bytes with v_cvt_pk_u8_f32 (converts,
    // saturates to 0..255 and packs in one instruction).  Signed outputs are computed 128 higher (pk_bias is folded into
    // the per-channel constant fb on the host) and the finished dword is xor-ed with 0x80808080.
    int32_t  pk_bias;       // 128 for QAsymmS8 outputs, 0 for QAsymmU8
    uint32_t pk_xor;        // 0x80808080 or 0
    float    pk_lo_f, pk_hi_f;   // activation clamp in the biased domain
    int32_t  pk_full;       // the clamp is 0..255: the instruction's own saturation does it
};

Requant MakeRequant(const mi355x_quant& out, int32_t activation, float a, float b);

// process-wide options set through mi355x_set_option()
struct Options
{
    int exact_division_epilogue = 0;   // 1: every output takes the fp32 division (no reciprocal fast path)
    int igemm_tile = 0;                // 0: automatic; 64, 96 (128x64), 128, 256, 512 (256x256), or 2256 / 2128 / 1256 (large-tile kernel), 2064 / 4064 (64x64 with K split over 2 / 4 wave groups), or 3000 (resident-tile kernel): every MFMA plan created meanwhile uses that implicit-GEMM tile
    int igemm_lds = 2;                 // LDS stages of the direct-to-LDS implicit GEMM (2 or 3); 0: use the register-staged kernel
    int dw_rows = 0;                   // output rows per thread of the 3x3 depthwise kernel: 0 automatic, 1 or 2 forced
    int pw_slab = 0;                   // output channels per slab of the weight-stationary pointwise kernel: 0 automatic, 32 / 64 / 128 forced
    int dw_cb = 0;                     // channels per block of the 3x3 depthwise kernel: 0 automatic (128 where the count allows), 32 forced
    int dw_mfma = 1;                   // 3x3 depthwise: 1 on the matrix cores (tile chosen from the feature map), 0 on the VALU kernel, 7 / 8 / 14 / 16 that tile edge where the stride allows it
    int stem_dot4 = 0;                 // 1: small-Ci convolutions stay on the v_dot4 kernel (tests compare it with the MFMA one)
    int igemm_xcd_cols = 0;            // direct-to-LDS implicit GEMM: 0 split the XCDs over the output channels where the weights are heavy, 1 never, 2 wherever possible
    int dwpw_stream = 1;               // 0: fused depthwise + pointwise launches never take the persistent kernel for 32 / 64 / 128 channels between the layers
    int pwdw_auto = 1;                 // 1: mi355x_conv2d_fusion_pays may recommend a 1x1 convolution + the depthwise layer behind it (7 x 7 maps)
    int pwdw_mf = 0;                   // 32-pixel fragments per block of the whole-image kernels (1x1 convolution + depthwise / + pooling): 0 automatic, 2, 4 or 7 forced
    int pool_small = 1;                // 0: pooling over a whole image of at most 64 pixels runs on the LDS-staged kernel (tests compare the two)
    int pwpool_auto = 1;               // 1: mi355x_conv2d_pool_fusion_pays may recommend a 1x1 convolution + the global pooling behind it
    int dwpw_panel = 1;                // 0: fused depthwise + pointwise launches never take the one-block-per-tile-over-all-channels kernel
    int chain_stages = 2;              // LDS stages of the matrix-core tiles inside a layer chain (2, 3 or 4), read at mi355x_chain_create
    int chain_defer_signal = 0;        // 1: layer chains count a tile as finished behind the next tile's loads (no wait for its stores)
    int chain_panel = 0;               // 1: layer chains run 1x1 convolutions with 256 or 512 input channels and many rows as one work item per
                                       // 64 output rows, the activation panel resident in LDS (gemm_panel_task.h); slower than 64 x 64 tiles today
    int chain_blocks_per_cu = 0;       // persistent blocks per CU of a layer chain: 0 as many as fit, else at most this many
};
Options& GlobalOptions();

// Copies plan constants to the device and returns when they are there.  Uses a stream of the library's own, never the
// legacy default stream: that one may not be touched while any thread captures a graph.
int UploadNow(void* dst_dev, const void* src_host, size_t bytes);

} // namespace mi355x
