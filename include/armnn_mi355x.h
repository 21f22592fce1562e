/*
 * armnn_mi355x.h -- C ABI of the MI355X (gfx950) device library behind the Arm NN "Mi355x" backend.
 *
 * This is the only door to the GPU: the C++17 backend (IBackendInternal / IWorkloadFactory / ITensorHandle /
 * IMemoryManager implementations) calls nothing but these functions, and so can any other host
 * (ctypes, JNI, cgo ...).  Plain pointers, sizes and POD structs only; no C++ or framework types.
 *
 * Conventions
 *   - every function returns 0 on success, otherwise a non-zero code (a hipError_t value when the
 *     failure came from HIP, MI355X_ERR_* otherwise); mi355x_last_error() returns a thread-local message.
 *     Nothing throws across this boundary.
 *   - pointers named *_dev are device pointers obtained from mi355x_malloc(); *_host are host pointers.
 *   - tensors are dense NHWC (Convolution2d / DepthwiseConvolution2d / Pooling2d) or row-major [M,K]
 *     (FullyConnected), 8-bit quantized, exactly as the reference's workloads see them.
 *   - a "plan" owns device copies of the constant operands (weights re-laid-out for the kernel, per-channel
 *     requantization multipliers, bias, zero-point corrections).  Plans are immutable after creation and may
 *     be run concurrently on different streams.
 *   - results equal the reference's CpuRef workloads to within 1 LSB (the accumulation is exact int32 where
 *     the reference accumulates in fp32); the requantization uses the reference's float formula.
 *
 * Reference interfaces each entry point stands in for (paths relative to the Arm NN 35.0.0 tree) are cited
 * at each declaration.
 */
#ifndef ARMNN_MI355X_H
#define ARMNN_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355X_ABI_VERSION 1

/* error codes outside the hipError_t range */
#define MI355X_ERR_INVALID_ARGUMENT 10001
#define MI355X_ERR_UNSUPPORTED      10002
#define MI355X_ERR_NO_DEVICE        10003
#define MI355X_ERR_OUT_OF_MEMORY    10004

/* armnn::DataType subset (include/armnn/Types.hpp:48-64) */
typedef enum {
    MI355X_QASYMM_S8 = 0,
    MI355X_QASYMM_U8 = 1,
    MI355X_QSYMM_S8  = 2,
    MI355X_SIGNED32  = 3
} mi355x_dtype;

/* armnn::ActivationFunction subset that the backend fuses (include/armnn/Types.hpp:86-101) */
typedef enum {
    MI355X_ACT_NONE         = 0,
    MI355X_ACT_RELU         = 1,   /* max(0, x)            */
    MI355X_ACT_BOUNDED_RELU = 2    /* min(a, max(b, x))    */
} mi355x_activation;

/* kernel selection; AUTO picks the fastest kernel whose preconditions hold */
typedef enum {
    MI355X_ALGO_AUTO      = 0,
    MI355X_ALGO_DIRECT    = 1,   /* one thread per output element; accepts every supported configuration      */
    MI355X_ALGO_MFMA      = 2,   /* implicit-GEMM on v_mfma_i32_32x32x32_i8 (conv / FC; symmetric int8 weights) */
    MI355X_ALGO_DEPTHWISE = 3,   /* channel-vectorised VALU kernels (depthwise, multiplier 1); 3x3 uses v_dot4 + LDS halo */
    MI355X_ALGO_DOT4      = 4    /* v_dot4 kernel with an LDS halo tile for layers with <= 4 input channels (stems) */
} mi355x_algo;

typedef struct mi355x_stream_s* mi355x_stream_t;   /* NULL = the default stream */
typedef struct mi355x_event_s*  mi355x_event_t;
typedef struct mi355x_graph_s*  mi355x_graph_t;
typedef struct mi355x_conv2d_s* mi355x_conv2d_t;
typedef struct mi355x_fc_s*     mi355x_fc_t;

/* Quantization of one activation tensor: armnn::TensorInfo scale/offset (include/armnn/Tensor.hpp:203-217). */
typedef struct {
    int32_t dtype;      /* MI355X_QASYMM_S8 or MI355X_QASYMM_U8 */
    float   scale;
    int32_t offset;
} mi355x_quant;

/* Quantization of a constant tensor: per-tensor (n_scales == 1) or per-axis (one scale per output channel). */
typedef struct {
    int32_t      dtype;      /* weights: QSYMM_S8 / QASYMM_S8 / QASYMM_U8 ; bias: SIGNED32 */
    int32_t      offset;     /* must be 0 for per-axis weights and for bias (WorkloadData.cpp:180-205,353-393) */
    uint32_t     n_scales;   /* 1 or the number of output channels */
    const float* scales;     /* host pointer, n_scales entries */
} mi355x_const_quant;

/* ------------------------------------------------------------------------------------------------------
 * Runtime: device, memory, streams, events, graphs.
 * Used by the backend's IBackendContext / IMemoryManager / ITensorHandle implementations; the CpuRef
 * counterparts are RefMemoryManager (src/backends/reference/RefMemoryManager.cpp:20-101) and
 * RefTensorHandle::Map/CopyInFrom/CopyOutTo (src/backends/reference/RefTensorHandle.cpp:45-133).
 * ---------------------------------------------------------------------------------------------------- */
const char* mi355x_last_error(void);
int  mi355x_abi_version(void);
/* Process-wide switches, read when a plan or a layer call is set up.
 *   "exact_division_epilogue" = 1: requantize every output with the fp32 division of armnn::Quantize
 *   (src/armnn/TypesUtils.cpp:40) instead of the reciprocal fast path that falls back to the division near
 *   rounding ties.  Both give identical bytes; the switch exists so that tests can prove it.
 *   "stem_dot4" = 1: convolutions with at most 4 input channels run on the v_dot4 kernel instead of the MFMA one
 *   (identical bytes; lets tests compare the two).
 *   "igemm_tile" = 0 | 64 | 96 | 128 | 256 | 512: plans created while it is set run on the LDS-tiled implicit-GEMM
 *   kernel with 64x64, 128x64, 128x128, 256x128 or 256x256 tiles instead of the automatic choice (the two largest only
 *   where the direct-to-LDS kernel applies; identical bytes; tests and tuning).  Further values force the other MFMA
 *   kernels where their shape rules allow them: 2256 | 2128 | 1256 the large-tile GEMM at 256x256, 256x128, 128x256;
 *   2064 | 4064 64x64 tiles with K split over 2 or 4 groups of waves inside the block; 3000 | 3001 the convolution that
 *   keeps its input tile resident in on-chip memory (3001: half-height tiles).
 *   "igemm_lds" = 2 | 3 | 0: LDS stages of the implicit-GEMM kernel that loads its k-tiles from global memory straight
 *   into LDS (input channels a multiple of 128); 0 selects the register-staged kernel instead (identical bytes).
 *   "dw_rows" = 0 | 1 | 2: output rows per thread of the 3x3 depthwise kernel (0: chosen from the feature-map height;
 *   identical bytes).
 *   "pw_slab" = 0 | 32 | 64 | 128: output channels per weight slab of the weight-stationary kernel for 1x1 convolutions
 *   with at most 128 input channels (0: 128 with 128 input channels and more than 64 outputs, else 64 or 32 by the layer's
 *   width; a value wider than the layer is ignored; identical bytes; tests and tuning).
 *   "dw_cb" = 0 | 32: channels per block of the 3x3 depthwise kernels (0: as many as the channel count and the kernel
 *   allow: 64 on the matrix cores, 128 on the VALU kernel; 32: always 32; identical bytes).
 *   "dw_mfma" = 1 | 0 | 7 | 8 | 14 | 16: 3x3 depthwise layers (multiplier 1, channels a multiple of 16) compute on the
 *   matrix cores (1, with the tile chosen from the feature map; 7, 8, 14 or 16: that tile height where the stride allows
 *   it) or on the VALU kernel (0).  Identical bytes.
 *   "igemm_xcd_cols" = 0 | 1 | 2: how the direct-to-LDS implicit GEMM deals its tiles to the 8 XCDs (each has an L2 of its
 *   own): 1 every XCD takes a range of row blocks over all output channels (each fetches every weight), 2 XCDs 0-3 take
 *   the lower half of the output channels and XCDs 4-7 the upper half (half the weights per XCD, every activation row
 *   fetched twice), 0 chooses 2 where the weights outweigh a quarter of the activations of a launch.  Identical bytes.
 *   "dwpw_stream" = 1 | 0: mi355x_conv2d_run_fused may (1) or may not (0) run a depthwise layer of 32, 64 (stride 2) or
 *   128 channels and the pointwise layer behind it (64, 128, 128 / 256 output channels) on the persistent kernel that keeps the
 *   pointwise weights in on-chip memory (identical bytes; lets tests compare it with the older fused kernel).
 *   "pwdw_auto" = 1 | 0: mi355x_conv2d_fusion_pays may (1) or may not (0) recommend a 1x1 convolution + the depthwise layer
 *   behind it (tests and tuning).
 *   "pwdw_mf" = 0 | 2 | 4 | 7: rows per block, in units of 32 pixels, of the kernels that keep whole images of a 1x1
 *   convolution's output on chip for the depthwise layer or the global pooling behind it (0: 7 with the depthwise layer, 4
 *   with the pooling where two images fit; a value too small for one image is ignored; identical bytes; tests and tuning).
 *   "pool_small" = 1 | 0: a pooling over a whole image of at most 64 pixels runs on the kernel that gives a thread one
 *   channel and requests all its taps at once (1), or on the kernel that stages the image in on-chip memory (0).  Identical
 *   bytes.
 *   "pwpool_auto" = 1 | 0: mi355x_conv2d_pool_fusion_pays may (1) or may not (0) recommend a 1x1 convolution + the global
 *   pooling behind it (tests and tuning).
 *   "dwpw_panel" = 1 | 0: mi355x_conv2d_run_fused may (1) or may not (0) run a depthwise layer of 256 or 512
 *   channels and a pointwise layer of 256 or 512 output channels on the kernel that gives a block an 8 x 8 pixel tile over
 *   all channels (identical bytes; lets tests compare it with the older fused kernel).
 *   "chain_stages" = 2 | 3 | 4: LDS stages of the matrix-core tiles inside a layer chain; "chain_blocks_per_cu" = 0 .. 16:
 *   persistent blocks per CU of a layer chain (0: as many as fit); "chain_panel" = 0 | 1: 1x1 convolutions with 256 or 512
 *   input channels and at least 96 row blocks run as one work item per 64 output rows with the activation panel resident
 *   in on-chip memory; "chain_defer_signal" = 0 | 1: a tile is counted as finished behind the next tile's loads instead of
 *   after a wait for its stores.  All four are read by mi355x_chain_create and give identical bytes; they exist for
 *   tests and tuning (the defaults are the fastest measured).
 *   Every option except "exact_division_epilogue" is a test and tuning hook: the numeric codes of "igemm_tile" name
 *   kernels of this library's current build and are no stable interface.
 * Unknown names and values outside these return MI355X_ERR_INVALID_ARGUMENT. */
int  mi355x_set_option(const char* name, int value);
int  mi355x_device_count(int* count);                 /* 0 devices is success with *count == 0 */
int  mi355x_init(int device);                         /* select + warm up the device; idempotent */
int  mi355x_device_name(char* buf, size_t buf_len);   /* e.g. "gfx950:sramecc+:xnack-" */
int  mi355x_device_props(int* compute_units, int* clock_khz, size_t* total_mem, size_t* lds_per_cu);

int  mi355x_malloc(void** ptr_dev, size_t bytes);
int  mi355x_free(void* ptr_dev);
int  mi355x_host_alloc(void** ptr_host, size_t bytes);          /* pinned host memory (hipHostMalloc) */
/* Device address of caller memory the device reaches directly: memory from mi355x_host_alloc (pinned; *is_device_memory
 * = 0) or device memory itself (*is_device_memory = 1).  Fails with MI355X_ERR_UNSUPPORTED for pageable host memory.
 * Lets a tensor handle adopt caller memory instead of copying it through a staging buffer (RefTensorHandle::CanBeImported /
 * Import, src/backends/reference/RefTensorHandle.cpp:135-165). */
int  mi355x_host_device_pointer(const void* ptr, void** device_ptr, int* is_device_memory);
int  mi355x_host_free(void* ptr_host);
int  mi355x_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, mi355x_stream_t stream);
int  mi355x_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, mi355x_stream_t stream);
/* The two above return when the transfer is complete (the host buffer may be pageable and is the caller's again at
 * once).  The _async forms only queue the transfer in stream order and return; the host buffer must be memory the
 * device reaches directly (mi355x_host_alloc / what mi355x_host_device_pointer accepts) and must stay untouched
 * (h2d) or unread (d2h) until the stream has passed the transfer.  Pageable memory is refused with
 * MI355X_ERR_UNSUPPORTED. */
int  mi355x_memcpy_h2d_async(void* dst_dev, const void* src_pinned, size_t bytes, mi355x_stream_t stream);
int  mi355x_memcpy_d2h_async(void* dst_pinned, const void* src_dev, size_t bytes, mi355x_stream_t stream);
int  mi355x_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, mi355x_stream_t stream);
int  mi355x_fill_u8(void* dst_dev, uint8_t value, size_t bytes, mi355x_stream_t stream);  /* fill kernel, graph-safe */

int  mi355x_stream_create(mi355x_stream_t* stream);
int  mi355x_stream_destroy(mi355x_stream_t stream);
int  mi355x_stream_synchronize(mi355x_stream_t stream);
int  mi355x_device_synchronize(void);

int  mi355x_event_create(mi355x_event_t* event);
int  mi355x_event_destroy(mi355x_event_t event);
int  mi355x_event_record(mi355x_event_t event, mi355x_stream_t stream);
/* Work queued on `stream` after this call starts only when the work recorded by `event` is done. Inside a graph
 * capture this is how a second stream joins the capture (fork) and how its work is joined back. */
int  mi355x_stream_wait_event(mi355x_stream_t stream, mi355x_event_t event);
int  mi355x_event_synchronize(mi355x_event_t event);
int  mi355x_event_elapsed_ms(mi355x_event_t start, mi355x_event_t stop, float* ms);

/* Capture everything launched on `stream` between begin and end into an executable graph, then replay it
 * with one launch (removes per-kernel launch latency from a network's steady-state loop). */
int  mi355x_graph_capture_begin(mi355x_stream_t stream);
int  mi355x_graph_capture_end(mi355x_stream_t stream, mi355x_graph_t* graph);
int  mi355x_graph_launch(mi355x_graph_t graph, mi355x_stream_t stream);
int  mi355x_graph_destroy(mi355x_graph_t graph);

/* ------------------------------------------------------------------------------------------------------
 * Convolution2d / DepthwiseConvolution2d
 *
 * Stands in for RefConvolution2dWorkload::Execute (workloads/RefConvolution2dWorkload.cpp:38-58) and
 * RefDepthwiseConvolution2dWorkload::Execute (workloads/RefDepthwiseConvolution2dWorkload.cpp:38-62), i.e.
 * Convolve() (workloads/ConvImpl.cpp:68-233) between MakeDecoder/MakeEncoder (Decoders.hpp:63-126,
 * Encoders.hpp:19-91), optionally followed by the Activation layer the backend fused into it
 * (workloads/Activation.cpp:33-42 via RefActivationWorkload.cpp:23-36).
 *
 * Fields mirror armnn::Convolution2dDescriptor / DepthwiseConvolution2dDescriptor
 * (include/armnn/Descriptors.hpp:534-585,659-711) and the tensor infos in WorkloadInfo.  As in Convolve(),
 * only pad_top / pad_left are inputs; bottom / right padding is implied by the output shape.
 * ---------------------------------------------------------------------------------------------------- */
typedef struct {
    uint32_t in_h, in_w, in_c;            /* input  [N, in_h, in_w, in_c]                      */
    uint32_t out_h, out_w, out_c;         /* output [N, out_h, out_w, out_c]                   */
    uint32_t kernel_h, kernel_w;
    uint32_t pad_top, pad_left;
    uint32_t stride_x, stride_y;
    uint32_t dilation_x, dilation_y;
    uint32_t depthwise;                   /* 0: weights [out_c, kh, kw, in_c]; 1: weights [1, kh, kw, out_c], out_c = in_c * M */
    uint32_t bias_enabled;
    mi355x_quant input;
    mi355x_quant output;
    int32_t  activation;                  /* mi355x_activation */
    float    activation_a, activation_b;  /* ActivationDescriptor::m_A / m_B */
    int32_t  algo;                        /* mi355x_algo */
} mi355x_conv2d_desc;

/* weights_host / bias_host are read once and may be released after the call returns.
 * Weight scales index the OUTPUT channel (quantization dim 0 for conv, 3 for depthwise); bias scales index
 * the output channel; with n_scales == 1 the single scale applies to all channels.  bias quantization is
 * NOT assumed to equal input_scale * weight_scale.
 * Limit: the kernels accumulate sum (x - zx)(w - zw) exactly in 32 bits; a plan whose K taps per output could overflow
 * that (K * max|x - zx| * max|w - zw| >= 2^31 with the given zero points and weights; never below K = 33 026) is refused
 * with MI355X_ERR_UNSUPPORTED.  The same holds for mi355x_fc_create with K = input features.
 * Filters of more than 32 taps over a multiple of 128 channels never run on the 256-row tiles (they take smaller ones). */
int mi355x_conv2d_create(const mi355x_conv2d_desc* desc,
                         const void* weights_host, const mi355x_const_quant* weights_quant,
                         const int32_t* bias_host, const mi355x_const_quant* bias_quant,
                         mi355x_conv2d_t* plan);
int mi355x_conv2d_run(mi355x_conv2d_t plan, uint32_t batch, const void* input_dev, void* output_dev,
                      mi355x_stream_t stream);
int mi355x_conv2d_destroy(mi355x_conv2d_t plan);
/* How many launches of the network this plan belongs to run side by side on the device (a batch split into lanes on
 * streams of their own); 1 after creation.  With more than one the plan prefers kernels whose blocks are small and
 * many, which share a CU with a neighbour's blocks better than the kernels that are fastest alone (identical bytes
 * either way).  No counterpart in the reference, whose workloads run one after the other on the calling thread. */
int mi355x_conv2d_set_concurrency(mi355x_conv2d_t plan, uint32_t lanes);
/* A Convolution2d and the Addition that consumes its output (a residual connection), run as one launch where the kernel
 * the plan resolves to can do it (the matrix-core kernels with 16-byte row stores), else as the convolution followed by
 * the Addition in place.  other_dev / other_quant: the Addition's other input, same shape as the convolution's output;
 * sum_quant, activation, a, b: the Addition's output quantization and the activation fused into it.  The convolution's
 * own output codes are formed first and then added exactly as the Addition layer adds (dequantize both inputs, one
 * fp32 addition, quantize), so the bytes are those of mi355x_conv2d_run followed by mi355x_add_run -- in the reference
 * these are two workloads in sequence (RefConvolution2dWorkload.cpp:38-58, then RefElementwiseBinaryWorkload.cpp:27-107).
 * output_dev may share no byte with input_dev or other_dev (one launch reads both while it writes the sum): overlapping
 * buffers are refused with MI355X_ERR_INVALID_ARGUMENT. */
int mi355x_conv2d_run_add(mi355x_conv2d_t plan, uint32_t batch, const void* input_dev, const void* other_dev,
                          const mi355x_quant* other_quant, const mi355x_quant* sum_quant, int32_t activation, float a, float b,
                          void* output_dev, mi355x_stream_t stream);
/* A 3x3 depthwise plan and the plan of the unpadded 1x1 stride-1 Convolution2d that consumes its output, run as one
 * kernel: the depthwise result is requantized to its own int8 codes in on-chip memory and fed to the pointwise GEMM
 * there, so the intermediate tensor is never written.  The bytes produced equal mi355x_conv2d_run(depthwise) followed
 * by mi355x_conv2d_run(pointwise) -- in the reference these are two workloads in sequence
 * (RefDepthwiseConvolution2dWorkload.cpp:38-62, then RefConvolution2dWorkload.cpp:38-58).
 * mi355x_conv2d_fusable returns 0 when the pair qualifies (3x3 depthwise with channels % 32 == 0, multiplier 1,
 * stride 1 or 2; pointwise with output channels % 64 == 0; chaining shapes and identical quantization of the shared
 * tensor), else MI355X_ERR_UNSUPPORTED / MI355X_ERR_INVALID_ARGUMENT with the reason in mi355x_last_error().
 * The other order is accepted as well: first = the unpadded 1x1 stride-1 Convolution2d, second = the 3x3 depthwise layer
 * that consumes it (stride 1 or 2, multiplier 1).  A block then computes whole images of the intermediate tensor for 64
 * of its channels, keeps them on chip and runs the depthwise filter there; it qualifies when one image has at most 224
 * pixels (14 x 14, 7 x 7 ...), the 1x1 layer's input channels are a multiple of 128, its weights have no zero point and
 * the shared channel count is a multiple of 64.  Same contract: the bytes of the two layers run one after the other. */
int mi355x_conv2d_fusable(mi355x_conv2d_t first, mi355x_conv2d_t second);
/* 1 when running the pair as one launch is what the library recommends at this batch, else 0; never an error.  Today:
 * a depthwise layer over 32, 64 (stride 2) or 128 channels and the pointwise layer behind it (64, 128, 128 or -- at stride
 * 2 -- 256 output channels) in launches of at least 1024 tiles of 8 x 8 output pixels, which run on the persistent kernel
 * that keeps the pointwise weights on chip; and a depthwise layer over 256 or 512 channels (stride 1, or stride 2 from 256
 * to 512 channels) and the pointwise layer of 256 or 512 output channels behind it in launches of at least 100 such tiles,
 * which run on the kernel that gives a block an 8 x 8 pixel tile over all channels; and, in the other order, a 1x1
 * convolution and the depthwise layer behind it on maps of at most 7 x 7 pixels in launches of at least 64 images (option
 * "pwdw_auto" = 0 turns this one off).  No counterpart in the reference, which has no fused workloads on CpuRef. */
int mi355x_conv2d_fusion_pays(mi355x_conv2d_t first, mi355x_conv2d_t second, uint32_t batch);
int mi355x_conv2d_run_fused(mi355x_conv2d_t first, mi355x_conv2d_t second, uint32_t batch,
                            const void* input_dev, void* output_dev, mi355x_stream_t stream);
/* A run of consecutive layers as one persistent launch ("chain").  plans[k] reads the output of plans[k - 1] (plans[0]
 * reads input_dev) and writes outputs_dev[k]; all for `batch` images.  One kernel executes the whole run: its blocks draw
 * (layer, tile) work items in layer order, and a tile starts as soon as the images it reads are complete in the layer
 * before -- there is no kernel boundary and no device-wide barrier between the layers, so tiles of neighbouring layers
 * overlap on every CU.  The tiles are those of mi355x_conv2d_run's kernels: the bytes written to every outputs_dev[k]
 * equal the bytes of running the plans one after the other with mi355x_conv2d_run -- in the reference the workloads of a
 * network run in sequence on the calling thread (LoadedNetwork::Execute, src/armnn/LoadedNetwork.cpp:845-1100, each
 * RefDepthwiseConvolution2dWorkload.cpp:38-62 / RefConvolution2dWorkload.cpp:38-58).
 *   Accepted members (mi355x_chain_accepts: 0, else MI355X_ERR_UNSUPPORTED with the reason): 3x3 depthwise plans of
 * multiplier 1, stride 1 or 2, a channel count that is a multiple of 128 and weights that fit one int8 each; unpadded 1x1
 * stride-1 Convolution2d plans with more than 128 input channels that are a multiple of 128, output channels a multiple of
 * 16 and weights without a zero point.  Tensors stay below 2 GiB.
 *   The addresses are bound at creation (a captured graph replays them).  input_dev and all outputs must not overlap each
 * other: every tensor of the run is written once per launch and read by other blocks as soon as an image is complete.
 * Outputs are 128-byte aligned, the input 16-byte aligned.  The chain owns a few KB of device memory (work queue head and
 * one counter per layer and image), so two launches of ONE chain object must not run at the same time; launches of
 * different chain objects may.  The plans must outlive the chain.
 *   mi355x_chain_status waits for nothing: call it after synchronizing the stream.  *gave_up is the number of blocks
 * whose bounded wait for a producer ran out (2 s; never in normal operation): if it is not 0 the outputs of that launch
 * are invalid; the call clears the condition. */
typedef struct mi355x_chain_s* mi355x_chain_t;
int mi355x_chain_accepts(mi355x_conv2d_t plan, uint32_t batch);
int mi355x_chain_create(uint32_t n_layers, const mi355x_conv2d_t* plans, uint32_t batch, const void* input_dev,
                        void* const* outputs_dev, mi355x_chain_t* chain);
int mi355x_chain_run(mi355x_chain_t chain, mi355x_stream_t stream);
/* The same run as mi355x_chain_create + mi355x_chain_run in one call that allocates nothing: the layer records, the work
 * queue heads and the per-image counters live in a device array that is part of the library (about 300 KB on every GPU
 * the library runs on, held until the process ends).  It has no counterpart in the reference; it is for callers that
 * cannot allocate device memory where they launch: code under graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Limits: at most 32 layers and 64 images, else MI355X_ERR_UNSUPPORTED (use mi355x_chain_create).  Same
 * members, same rules for the tensors, same bytes.  All calls on one GPU share the one array: two calls whose launches
 * could run at the same time on that GPU race (order them on one stream or with events); the array keeps the last call's
 * contents, and each call first sets what must start at zero with a fill kernel.  The two small host-to-device copies of
 * the call read the calling thread's own buffers; wait for the stream before the same thread calls again with other
 * arguments.  mi355x_chain_status does not apply: synchronize and compare, or use the chain object where a report is needed. */
int mi355x_chain_run_noalloc(uint32_t n_layers, const mi355x_conv2d_t* plans, uint32_t batch, const void* input_dev,
                             void* const* outputs_dev, mi355x_stream_t stream);
int mi355x_chain_status(mi355x_chain_t chain, uint32_t* gave_up);
/* work items (tiles) of one launch and the number of persistent blocks it uses */
int mi355x_chain_info(mi355x_chain_t chain, uint32_t* work_items, uint32_t* blocks);
/* Measurement support (not for graph capture: allocates, synchronizes the stream and uses the default stream for the
 * read-back): one launch of the chain whose blocks add up shader-clock cycles per phase; sums[0..4] = cycles, summed over
 * all blocks, spent taking an item from the queue, waiting for producers, inside matrix-core tiles, inside depthwise
 * tiles, and waiting for the tile's stores plus the hand-over; sums[5], sums[6] = matrix-core and depthwise tiles run,
 * sums[7] = tiles that found their producer unfinished.  The reference's counterpart is its per-workload profiler
 * (src/armnn/Profiling.hpp:227-236). */
int mi355x_chain_run_stamped(mi355x_chain_t chain, mi355x_stream_t stream, uint64_t* sums);
int mi355x_chain_destroy(mi355x_chain_t chain);
/* which kernel a plan resolved to (mi355x_algo) and its tile configuration, for logs and tests */
int mi355x_conv2d_algo(mi355x_conv2d_t plan, int32_t* algo, char* desc_buf, size_t desc_len);
/* Name of the device kernel the calling thread's last *_run call launched, with its template arguments, as a profiler
 * lists it (without namespace and argument list); "" before the first launch.  The reference reports what a workload
 * resolved to through its profiler the same way (ARMNN_REPORT_PROFILING_WORKLOAD_DESC, src/armnn/Profiling.hpp:227-236;
 * ClConvolution2dWorkload reports its ConvolutionMethod, src/backends/cl/workloads/ClConvolution2dWorkload.cpp:135-161). */
const char* mi355x_last_kernel(void);

/* ------------------------------------------------------------------------------------------------------
 * FullyConnected
 *
 * Stands in for RefFullyConnectedWorkload::Execute (workloads/RefFullyConnectedWorkload.cpp:39-67) ->
 * FullyConnected() (workloads/FullyConnected.cpp:13-65).  K is the product of the input's dimensions after
 * the first (GetNumActivations, RefFullyConnectedWorkload.cpp:16-24).
 * Fields mirror armnn::FullyConnectedDescriptor (include/armnn/Descriptors.hpp:507-531).
 * ---------------------------------------------------------------------------------------------------- */
typedef struct {
    uint32_t k;                           /* inputs per row                                        */
    uint32_t out_features;                /* outputs per row                                       */
    uint32_t transpose_weights;           /* 1: weights [out_features, k]; 0: weights [k, out_features] */
    uint32_t bias_enabled;
    mi355x_quant input;
    mi355x_quant output;
    int32_t  activation;
    float    activation_a, activation_b;
    int32_t  algo;
} mi355x_fc_desc;

int mi355x_fc_create(const mi355x_fc_desc* desc,
                     const void* weights_host, const mi355x_const_quant* weights_quant,
                     const int32_t* bias_host, const mi355x_const_quant* bias_quant,
                     mi355x_fc_t* plan);
int mi355x_fc_run(mi355x_fc_t plan, uint32_t batch, const void* input_dev, void* output_dev,
                  mi355x_stream_t stream);
int mi355x_fc_destroy(mi355x_fc_t plan);
int mi355x_fc_algo(mi355x_fc_t plan, int32_t* algo, char* desc_buf, size_t desc_len);

/* ------------------------------------------------------------------------------------------------------
 * Bandwidth-bound layers that keep a whole network on the device (no bounce through CpuRef).
 * ---------------------------------------------------------------------------------------------------- */

/* Standalone Activation layer, ReLu / BoundedReLu, same quantization in and out or different:
 * RefActivationWorkload::Execute (workloads/RefActivationWorkload.cpp:23-36). */
int mi355x_activation_run(size_t n_elements, const mi355x_quant* in_q, const mi355x_quant* out_q,
                          int32_t activation, float a, float b,
                          const void* input_dev, void* output_dev, mi355x_stream_t stream);

/* Pooling2d, NHWC: Pooling2d() (workloads/Pooling2d.cpp:142-303).  Fields mirror armnn::Pooling2dDescriptor
 * (include/armnn/Descriptors.hpp:371-418). pool_type: 0 Max, 1 Average.  padding_method: 0 IgnoreValue, 1 Exclude. */
typedef struct {
    uint32_t in_h, in_w, channels, out_h, out_w;
    uint32_t pool_w, pool_h, stride_x, stride_y;
    uint32_t pad_left, pad_right, pad_top, pad_bottom;
    int32_t  pool_type, padding_method;
    mi355x_quant input, output;
} mi355x_pool2d_desc;
int mi355x_pool2d_run(const mi355x_pool2d_desc* desc, uint32_t batch, const void* input_dev, void* output_dev,
                      mi355x_stream_t stream);
/* An unpadded 1x1 stride-1 Convolution2d and the Pooling2d over its whole output image (Max or Average, no padding,
 * one output pixel) as one launch: a block computes whole images of the convolution's output for 64 of its channels,
 * keeps them on chip and pools them there in the order of Pooling2d.cpp:186-300, so output_dev [batch][channels] holds
 * the bytes of mi355x_conv2d_run followed by mi355x_pool2d_run -- two workloads in sequence in the reference
 * (RefConvolution2dWorkload.cpp:38-58, then RefPooling2dWorkload.cpp:18-36) -- and the convolution's output tensor is
 * never written: the caller must have no other reader of it.  mi355x_conv2d_pool_fusable returns 0 when the pair
 * qualifies: a matrix-core plan whose input channels are a multiple of 128 and whose weights have no zero point, output
 * channels % 64 == 0, an image of at most 196 pixels, the pooling's input quantization equal to the convolution's
 * output quantization; else MI355X_ERR_UNSUPPORTED / MI355X_ERR_INVALID_ARGUMENT with the reason in mi355x_last_error().
 * mi355x_conv2d_pool_fusion_pays: 1 when the library recommends the one launch at this batch (at least 32 blocks of
 * whole images x 64 channels; option "pwpool_auto" = 0 turns the recommendation off), else 0; never an error.
 * input_dev 16-byte aligned; output_dev may share no byte with input_dev (one launch reads the one while it writes the
 * other: MI355X_ERR_INVALID_ARGUMENT). */
int mi355x_conv2d_pool_fusable(mi355x_conv2d_t conv, const mi355x_pool2d_desc* pool);
int mi355x_conv2d_pool_fusion_pays(mi355x_conv2d_t conv, const mi355x_pool2d_desc* pool, uint32_t batch);
int mi355x_conv2d_run_pooled(mi355x_conv2d_t conv, const mi355x_pool2d_desc* pool, uint32_t batch, const void* input_dev,
                             void* output_dev, mi355x_stream_t stream);

/* ElementwiseBinary Add of two equally-shaped tensors (dequantize, add, requantize) with an optional fused
 * ReLu / BoundedReLu: RefElementwiseBinaryWorkload (workloads/RefElementwiseBinaryWorkload.cpp:27-107). */
int mi355x_add_run(size_t n_elements, const mi355x_quant* in0_q, const mi355x_quant* in1_q,
                   const mi355x_quant* out_q, int32_t activation, float a, float b,
                   const void* input0_dev, const void* input1_dev, void* output_dev, mi355x_stream_t stream);

/* Softmax over the last axis of a [rows, cols] tensor: Softmax() (workloads/Softmax.cpp:16-69). */
int mi355x_softmax_run(uint32_t rows, uint32_t cols, float beta, const mi355x_quant* in_q,
                       const mi355x_quant* out_q, const void* input_dev, void* output_dev,
                       mi355x_stream_t stream);

/* The tail of a classifier as ONE launch: global pooling (the window is the whole unpadded image, at most 196 pixels,
 * channels % 4 == 0) -> FullyConnected (a matrix-core plan: k % 16 == 0, k >= 128, at most 2048 outputs) -> Softmax over
 * each row of logits.  Every stage computes exactly what mi355x_pool2d_run, mi355x_fc_run and mi355x_softmax_run compute
 * (Pooling2d.cpp:142-303, FullyConnected.cpp:13-65, Softmax.cpp:16-69) and writes the same bytes to pooled_dev
 * [batch][channels], logits_dev [batch][out_features] and output_dev [batch][out_features]; the stages hand over inside the
 * kernel through two counters in a few hundred bytes of device memory the object owns, so two launches of ONE object must
 * not run at the same time (launches of different objects may).  `fc` must outlive the object; its input quantization
 * must be the pooling's output quantization, its output quantization is the Softmax's input quantization.  The four
 * tensors must not overlap; pooled_dev 16-byte, input_dev and logits_dev 4-byte aligned; at most 1024 rows per launch.
 * What the object does not take (MI355X_ERR_UNSUPPORTED) runs as the three calls.  On an MI355X the one launch takes
 * about 16 us for 64 rows of 1024 channels against about 13 us for the three calls back to back (each hand-over inside the
 * kernel costs what a kernel boundary costs: stores written through, a counter, a poll, reads that miss), so the callers
 * here launch the three; the entry point is for callers whose cost is the number of launches.
 *   Every wait inside the kernel is bounded (2 s by default; mi355x_tail_set_wait_limit, for tests of the give-up path);
 * mi355x_tail_status waits for nothing (call it after synchronizing the stream): *gave_up is the number of waits that ran
 * out in runs since the last call, and a run that gave up leaves its outputs undefined. */
typedef struct mi355x_tail_s* mi355x_tail_t;
int mi355x_tail_create(const mi355x_pool2d_desc* pool, mi355x_fc_t fc, float beta, const mi355x_quant* output_quant,
                       mi355x_tail_t* tail);
int mi355x_tail_run(mi355x_tail_t tail, uint32_t batch, const void* input_dev, void* pooled_dev, void* logits_dev,
                    void* output_dev, mi355x_stream_t stream);
int mi355x_tail_status(mi355x_tail_t tail, uint32_t* gave_up);
int mi355x_tail_set_wait_limit(mi355x_tail_t tail, uint64_t microseconds);
int mi355x_tail_destroy(mi355x_tail_t tail);

/* Pad with a constant, rank 1..4: Pad() (workloads/Pad.cpp:39-236) as RefPadWorkload::Execute calls it
 * (workloads/RefPadWorkload.cpp:18-40).  Fields mirror armnn::PadDescriptor (include/armnn/Descriptors.hpp:1196-1229):
 * pad_before[d] / pad_after[d] are m_PadList[d].first / .second.  pad_value is the stored code of the padding
 * (rounded half away from zero and saturated to the type), not a real number: the reference encodes it with scale 1
 * and offset 0 (Pad.cpp:77-84).  Elements of the input are decoded with `input` and encoded with `output`; with equal
 * quantizations they are copied. */
typedef struct {
    uint32_t rank;
    uint32_t in_shape[4];
    uint32_t pad_before[4], pad_after[4];
    float    pad_value;
    mi355x_quant input, output;
} mi355x_pad_desc;
int mi355x_pad_run(const mi355x_pad_desc* desc, const void* input_dev, void* output_dev, mi355x_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ARMNN_MI355X_H */
