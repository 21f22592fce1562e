/*
 * CPU restatement of the Arm NN CpuRef quantized hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker for the HIP kernels: it restates, in plain C, what the reference's
 * CpuRef workloads compute for quantized Convolution2d / DepthwiseConvolution2d / FullyConnected
 * (and the few bandwidth-bound layers the two benchmark networks need).  Nothing in the shipped
 * product may call it; only tests, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function cites the reference file:line it follows (paths relative to the Arm NN 35.0.0 tree).
 * The arithmetic is float32 exactly as in the reference: operands are dequantized to float,
 * accumulated in a scalar float in the reference's loop order, and re-quantized with
 * round-half-away-from-zero.  Build WITHOUT -ffast-math and WITH -ffp-contract=off.
 *
 * Parity status of each function (what pins it) is listed in oracle/README.md.
 */
#ifndef CPUREF_ORACLE_H
#define CPUREF_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Data-type codes (same numbering as the device library's header). */
enum {
    ORC_QASYMM_S8 = 0,   /* armnn::DataType::QAsymmS8 */
    ORC_QASYMM_U8 = 1,   /* armnn::DataType::QAsymmU8 */
    ORC_QSYMM_S8  = 2,   /* armnn::DataType::QSymmS8  */
    ORC_SIGNED32  = 3,   /* armnn::DataType::Signed32 */
    ORC_FLOAT32   = 4    /* armnn::DataType::Float32  */
};

enum { ORC_ACT_NONE = 0, ORC_ACT_RELU = 1, ORC_ACT_BOUNDED_RELU = 2 };
enum { ORC_POOL_MAX = 0, ORC_POOL_AVERAGE = 1 };
enum { ORC_PAD_IGNORE_VALUE = 0, ORC_PAD_EXCLUDE = 1 };
enum { ORC_NHWC = 0, ORC_NCHW = 1 };

/* A tensor = data pointer + the subset of armnn::TensorInfo the hot path reads
 * (include/armnn/Tensor.hpp:152-274). quant_dim < 0 means "not set". */
typedef struct {
    void*        data;
    int32_t      dtype;
    uint32_t     ndim;
    uint32_t     shape[6];
    const float* scales;     /* n_scales entries; n_scales==1 => per-tensor */
    uint32_t     n_scales;
    int32_t      quant_dim;
    int32_t      offset;
} orc_tensor;

typedef struct {
    uint32_t pad_top, pad_left;             /* bottom/right are implicit in the output shape */
    uint32_t stride_x, stride_y;
    uint32_t dilation_x, dilation_y;
    int32_t  bias_enabled;
    int32_t  data_layout;                   /* ORC_NHWC / ORC_NCHW */
    int32_t  depthwise;                     /* 0: weights [O,Kh,Kw,I]; 1: weights [1,Kh,Kw,I*M] */
} orc_conv_params;

typedef struct {
    int32_t  pool_type, padding_method;
    uint32_t pad_left, pad_right, pad_top, pad_bottom;
    uint32_t pool_w, pool_h, stride_x, stride_y;
} orc_pool_params;

/* -- scalar arithmetic: src/armnn/TypesUtils.cpp:29-56 -- */
float   orc_dequantize_s8(int8_t v, float scale, int32_t offset);
float   orc_dequantize_u8(uint8_t v, float scale, int32_t offset);
float   orc_dequantize_s32(int32_t v, float scale, int32_t offset);
int8_t  orc_quantize_s8(float v, float scale, int32_t offset);
uint8_t orc_quantize_u8(float v, float scale, int32_t offset);

/* -- decoders / encoders: workloads/BaseIterator.hpp, Decoders.hpp:19-126, Encoders.hpp:19-91 -- */
/* Decode a whole tensor to float (Decoder<float>::DecodeTensor). `is_depthwise` is forwarded to the
 * per-axis int32 decoder exactly as Convolve forwards it to the FILTER decoder only. Returns 0 / -1. */
int orc_decode_tensor(const orc_tensor* t, int is_depthwise, float* out);
/* Encoder<float>::Set for `n` consecutive elements starting at index 0. */
int orc_encode_tensor(const float* values, size_t n, const orc_tensor* out);

/* -- float-domain kernels on already-decoded vectors -- */
/* workloads/ConvImpl.cpp:68-233, literal loop nest (batch,cOut,y,x,cIn,ky,kx). */
int orc_convolve_f32(const uint32_t in_shape[4], const float* in, const uint32_t out_shape[4], float* out,
                     const uint32_t filter_shape[4], const float* filter, const float* bias,
                     const orc_conv_params* p);
/* Same result bit for bit (per-output tap order kept), vectorised over output channels + OpenMP. NHWC only. */
int orc_convolve_f32_fast(const uint32_t in_shape[4], const float* in, const uint32_t out_shape[4], float* out,
                          const uint32_t filter_shape[4], const float* filter, const float* bias,
                          const orc_conv_params* p);
/* workloads/FullyConnected.cpp:13-65 */
int orc_fully_connected_f32(uint32_t batch, uint32_t K, uint32_t O, const float* in, const float* w,
                            const float* bias, int transpose_weights, float* out);
int orc_fully_connected_f32_fast(uint32_t batch, uint32_t K, uint32_t O, const float* in, const float* w,
                                 const float* bias, int transpose_weights, float* out);
/* workloads/Activation.cpp:13-42 (ReLu / BoundedReLu only) */
float orc_activation_f32(float in, int function, float a, float b);

/* -- whole workloads on quantized tensors (what RefXxxWorkload::Execute does) -- */
/* RefConvolution2dWorkload.cpp:38-58 / RefDepthwiseConvolution2dWorkload.cpp:38-62.
 * `fast` selects orc_convolve_f32_fast (NHWC only). bias may be NULL when !bias_enabled. */
int orc_conv2d(const orc_tensor* in, const orc_tensor* weights, const orc_tensor* bias,
               const orc_tensor* out, const orc_conv_params* p, int fast);
/* RefFullyConnectedWorkload.cpp:16-67 */
int orc_fully_connected(const orc_tensor* in, const orc_tensor* weights, const orc_tensor* bias,
                        const orc_tensor* out, int bias_enabled, int transpose_weights, int fast);
/* RefActivationWorkload.cpp:23-36 + Activation.cpp:99-117 */
int orc_activation(const orc_tensor* in, const orc_tensor* out, int function, float a, float b);
/* workloads/Pooling2d.cpp:142-303 (NHWC or NCHW) */
int orc_pooling2d(const orc_tensor* in, const orc_tensor* out, const orc_pool_params* p, int data_layout);
/* workloads/Softmax.cpp:16-69 */
int orc_softmax(const orc_tensor* in, const orc_tensor* out, float beta, int axis);
/* RefElementwiseBinaryWorkload.cpp:27-107 (BinaryOperation::Add, float path) with Broadcast.cpp:11-33 */
int orc_add(const orc_tensor* in0, const orc_tensor* in1, const orc_tensor* out);

/* workloads/Pad.cpp:39-236 (constant padding, any rank up to 6): pad_before[d] elements are added in front of
 * dimension d; what is added behind follows from the output shape.  For quantized outputs pad_value is the
 * stored code (rounded, saturated), not a real number. */
int orc_pad(const orc_tensor* in, const orc_tensor* out, const uint32_t* pad_before, float pad_value);

const char* orc_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
