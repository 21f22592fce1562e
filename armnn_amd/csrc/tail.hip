// Global pooling -> FullyConnected -> Softmax as one launch (mi355x_tail_*): host side of TailKernel.
#include "common.h"
#include "plan.h"
#include "tail_kernel.h"

#include <algorithm>
#include <cmath>

using namespace mi355x;

struct mi355x_tail_s
{
    mi355x_pool2d_desc pool{};
    const mi355x_conv2d_s* fc = nullptr;      // owned by the caller's FullyConnected plan
    float beta = 1.0f;
    mi355x_quant out_q{};
    uint32_t* d_sync = nullptr;
    long long timeout_ticks = 200000000ll;    // 2 s of the 100 MHz wall clock
    int cus = 256;
    ~mi355x_tail_s() { (void)hipFree(d_sync); }
};

namespace
{

struct OwnStream
{
    hipStream_t s = nullptr;
    ~OwnStream() { if (s) (void)hipStreamDestroy(s); }
};

// a stream of the library's own: the legacy default stream may not be touched while any thread captures a graph
int OwnStreamGet(hipStream_t* out)
{
    thread_local OwnStream own;
    if (!own.s) MI355X_HIP(hipStreamCreateWithFlags(&own.s, hipStreamNonBlocking));
    *out = own.s;
    return 0;
}

bool SameQuant(const mi355x_quant& a, const mi355x_quant& b) { return a.dtype == b.dtype && a.scale == b.scale && a.offset == b.offset; }

int CheckQuant(const mi355x_quant& q, const char* what)
{
    if (!IsActivationDtype(q.dtype)) return SetError(MI355X_ERR_UNSUPPORTED, "tail: %s: data type %d is not QAsymmS8/QAsymmU8", what, q.dtype);
    if (!(q.scale > 0.0f) || !std::isfinite(q.scale)) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: %s: scale must be positive and finite", what);
    return 0;
}

template <int UN, int V>
int LaunchTail(const TailArgs& a, unsigned grid, hipStream_t stream)
{
    NoteKernel("TailKernel<%d, %d>", UN, V);
    hipLaunchKernelGGL((TailKernel<UN, V>), dim3(grid), dim3(256), 0, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

} // namespace

extern "C" {

int mi355x_tail_create(const mi355x_pool2d_desc* pool, mi355x_fc_t fc, float beta, const mi355x_quant* output_quant, mi355x_tail_t* tail)
{
    if (!tail) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail pointer is null");
    *tail = nullptr;
    if (!pool || !fc || !fc->conv || !output_quant) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: descriptor / plan / quantization is null");
    const mi355x_conv2d_s* p = fc->conv;
    if (int rc = CheckQuant(pool->input, "pooling input")) return rc;
    if (int rc = CheckQuant(pool->output, "pooling output")) return rc;
    if (int rc = CheckQuant(*output_quant, "output")) return rc;
    if (pool->pool_type != 0 && pool->pool_type != 1) return SetError(MI355X_ERR_UNSUPPORTED, "Unsupported pooling algorithm %d", pool->pool_type);
    const bool global = pool->out_h == 1 && pool->out_w == 1 && pool->pad_top == 0 && pool->pad_left == 0 && pool->pad_bottom == 0 &&
                        pool->pad_right == 0 && pool->pool_h == pool->in_h && pool->pool_w == pool->in_w && pool->in_h * pool->in_w >= 1 &&
                        pool->in_h * pool->in_w <= static_cast<uint32_t>(kGlobalPoolMaxTaps);
    if (!global) return SetError(MI355X_ERR_UNSUPPORTED, "tail: the pooling window must be the whole unpadded image, at most %d pixels", kGlobalPoolMaxTaps);
    if (pool->channels == 0 || (pool->channels % 4) != 0) return SetError(MI355X_ERR_UNSUPPORTED, "tail: channels must be a multiple of 4 (got %u)", pool->channels);
    const ConvGeom& g = p->geom;
    if (static_cast<uint32_t>(g.Ci) != pool->channels)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: FullyConnected reads %d inputs per row, the pooling gives %u", g.Ci, pool->channels);
    if (!SameQuant(pool->output, p->d.input))
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: the pooling's output quantization is not the FullyConnected's input quantization");
    if (p->algo != MI355X_ALGO_MFMA || (g.Ci % 16) != 0 || g.Ci < 128 || p->tile_override != 0 || p->Co_pad < (g.Co + 31) / 32 * 32)
        return SetError(MI355X_ERR_UNSUPPORTED, "tail: the FullyConnected plan must be a matrix-core plan with k %% 16 == 0 and k >= 128");
    if (g.Co > 2048) return SetError(MI355X_ERR_UNSUPPORTED, "tail: at most 2048 outputs per row (got %d)", g.Co);
    if (!std::isfinite(beta)) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: beta must be finite");
    auto* t = new mi355x_tail_s;
    t->pool = *pool;
    t->fc = p;
    t->beta = beta;
    t->out_q = *output_quant;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) t->cus = prop.multiProcessorCount;
    if (hipMalloc(reinterpret_cast<void**>(&t->d_sync), kTailSyncWords * 4) != hipSuccess)
    {
        delete t;
        return SetError(MI355X_ERR_OUT_OF_MEMORY, "tail: out of device memory");
    }
    const uint32_t zeros[kTailSyncWords] = {};
    if (const int rc = UploadNow(t->d_sync, zeros, sizeof(zeros))) { delete t; return rc; }
    *tail = t;
    return 0;
}

int mi355x_tail_run(mi355x_tail_t tail, uint32_t batch, const void* input_dev, void* pooled_dev, void* logits_dev, void* output_dev,
                    mi355x_stream_t stream)
{
    if (!tail) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail is null");
    if (batch == 0) return 0;
    if (!input_dev || !pooled_dev || !logits_dev || !output_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "null tensor pointer");
    if (batch > 1024) return SetError(MI355X_ERR_UNSUPPORTED, "tail: at most 1024 rows per launch (got %u)", batch);
    const mi355x_conv2d_s* p = tail->fc;
    const ConvGeom& g = p->geom;
    if ((reinterpret_cast<uintptr_t>(input_dev) & 3) != 0 || (reinterpret_cast<uintptr_t>(pooled_dev) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(logits_dev) & 3) != 0)
        return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: input and logits must be 4-byte aligned, the pooled tensor 16-byte aligned");
    // the three written tensors must not overlap each other or the input: blocks of one launch read what others wrote
    const size_t n_in = static_cast<size_t>(batch) * tail->pool.in_h * tail->pool.in_w * tail->pool.channels;
    const size_t n_pool = static_cast<size_t>(batch) * tail->pool.channels, n_out = static_cast<size_t>(batch) * g.Co;
    const struct { const uint8_t* p; size_t n; } span[4] = {{static_cast<const uint8_t*>(input_dev), n_in},
                                                            {static_cast<const uint8_t*>(pooled_dev), n_pool},
                                                            {static_cast<const uint8_t*>(logits_dev), n_out},
                                                            {static_cast<const uint8_t*>(output_dev), n_out}};
    for (int i = 0; i < 4; ++i)
        for (int j = i + 1; j < 4; ++j)
            if (span[i].p < span[j].p + span[j].n && span[j].p < span[i].p + span[i].n)
                return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail: the tensors of a run must not overlap");
    TailArgs a{};
    const mi355x_pool2d_desc& d = tail->pool;
    a.pool.H = d.in_h; a.pool.W = d.in_w; a.pool.C = d.channels; a.pool.Ho = 1; a.pool.Wo = 1;
    a.pool.pool_w = d.pool_w; a.pool.pool_h = d.pool_h; a.pool.stride_x = d.stride_x; a.pool.stride_y = d.stride_y;
    a.pool.is_max = d.pool_type == 0;
    a.pool.exclude = d.padding_method == 1;
    a.pool_in = MakeQIn(d.input);
    a.pool_rq = MakeRequant(d.output, MI355X_ACT_NONE, 0.0f, 0.0f);
    a.x = static_cast<const uint8_t*>(input_dev);
    a.pooled = static_cast<uint8_t*>(pooled_dev);
    a.fc.x = a.pooled; a.fc.w = p->w_mfma; a.fc.ct = ChanTab{p->chan, p->Co_pad}; a.fc.corr = p->corr; a.fc.y = static_cast<uint8_t*>(logits_dev);
    a.fc.M = static_cast<int>(batch); a.fc.K = g.Ci; a.fc.N = g.Co; a.fc.w_stride = p->K_pad; a.fc.xor_mask = p->xor_mask; a.fc.zw_neg = p->zw_neg;
    a.fc.rq = p->rq;
    a.cols = g.Co;
    a.beta = tail->beta;
    a.sm_in = MakeQIn(p->d.output);
    a.sm_rq = MakeRequant(tail->out_q, MI355X_ACT_NONE, 0.0f, 0.0f);
    a.out = static_cast<uint8_t*>(output_dev);
    a.batch = static_cast<int>(batch);
    a.pool_items = static_cast<int>(batch) * ((g.Ci + 255) / 256);
    a.fc_tiles_n = (g.Co + 31) / 32;
    a.fc_tiles = a.fc_tiles_n * ((static_cast<int>(batch) + 31) / 32);
    a.sync = tail->d_sync;
    a.timeout_ticks = tail->timeout_ticks;
    const unsigned grid = static_cast<unsigned>(std::max(1, std::min(tail->cus, std::max(a.pool_items, std::max(a.fc_tiles, a.batch)))));
    hipStream_t s = ToHip(stream);
    const bool wide = g.Co > 1024;
    if (g.Ci <= 512) return wide ? LaunchTail<4, 8>(a, grid, s) : LaunchTail<4, 4>(a, grid, s);
    return wide ? LaunchTail<8, 8>(a, grid, s) : LaunchTail<8, 4>(a, grid, s);
}

int mi355x_tail_status(mi355x_tail_t tail, uint32_t* gave_up)
{
    if (!tail || !gave_up) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail / result pointer is null");
    hipStream_t s = nullptr;
    if (const int rc = OwnStreamGet(&s)) return rc;
    uint32_t words[2] = {0, 0};
    MI355X_HIP(hipMemcpyAsync(words, tail->d_sync + kTailAbort, sizeof(words), hipMemcpyDeviceToHost, s));
    MI355X_HIP(hipStreamSynchronize(s));
    *gave_up = words[1] + (words[0] != 0 && words[1] == 0 ? 1u : 0u);
    if (words[0] != 0 || words[1] != 0)
    {
        // a run that gave up leaves its flag standing and may have left counters behind: clear everything
        const uint32_t zeros[kTailSyncWords] = {};
        MI355X_HIP(hipMemcpyAsync(tail->d_sync, zeros, sizeof(zeros), hipMemcpyHostToDevice, s));
        MI355X_HIP(hipStreamSynchronize(s));
    }
    return 0;
}

int mi355x_tail_set_wait_limit(mi355x_tail_t tail, uint64_t microseconds)
{
    if (!tail) return SetError(MI355X_ERR_INVALID_ARGUMENT, "tail is null");
    tail->timeout_ticks = static_cast<long long>(std::min<uint64_t>(microseconds, 3600ull * 1000000ull)) * 100;
    return 0;
}

int mi355x_tail_destroy(mi355x_tail_t tail)
{
    delete tail;
    return 0;
}

} // extern "C"
