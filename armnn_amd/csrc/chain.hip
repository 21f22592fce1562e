// mi355x_chain_*: a run of consecutive convolution plans executed by one persistent launch (chain_kernel.h).
#include "chain_kernel.h"
#include "plan.h"

#include <algorithm>
#include <mutex>
#include <string>
#include <vector>

using namespace mi355x;

// mi355x_chain_run_noalloc: the memory mi355x_chain_create would allocate (layer records, per-image tile counts, queue heads
// and counters), as one file-scope device array.  Every GPU the library runs on holds its own copy until the process
// ends.  In host code the array's name is only a stand-in: its address on the current device comes from
// hipGetSymbolAddress, once per device, and only that pointer is handed to kernels and copies.
constexpr uint32_t kNoallocMaxLayers = 32, kNoallocMaxBatch = 64;
constexpr size_t kNoallocSyncBytes = (static_cast<size_t>(kChainCounterSlot) + kNoallocMaxLayers * kNoallocMaxBatch) * kChainSlot * 4;   // 264 320
constexpr size_t kNoallocNeedBytes = static_cast<size_t>(kNoallocMaxLayers) * kNoallocMaxBatch * 4;                                        //   8 192
constexpr size_t kNoallocLayerBytes = static_cast<size_t>(kNoallocMaxLayers) * sizeof(ChainLayer);
constexpr size_t kNoallocBytes = kNoallocSyncBytes + kNoallocNeedBytes + kNoallocLayerBytes;
static __device__ __align__(256) unsigned char scratch[kNoallocBytes];

struct mi355x_chain_s
{
    std::vector<ChainLayer> layers;
    ChainLayer* d_layers = nullptr;
    uint32_t*   d_need = nullptr;
    uint32_t*   d_sync = nullptr;
    int batch = 0, total_items = 0, grid = 0, stages = 2;
    int qtotal[kChainQueues] = {};
    int smem = 0;
    int defer_signal = 0;
    long long timeout_ticks = 200000000ll;     // 2 s of the 100 MHz wall clock
    ~mi355x_chain_s()
    {
        (void)hipFree(d_layers);
        (void)hipFree(d_need);
        (void)hipFree(d_sync);
    }
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

// What a plan contributes to a chain at this batch: fills `L` (without first_item / src) or says why not.
int Describe(const mi355x_conv2d_s* p, uint32_t batch, const void* x, void* y, ChainLayer* L)
{
    if (!p) return SetError(MI355X_ERR_INVALID_ARGUMENT, "plan is null");
    if (batch == 0) return SetError(MI355X_ERR_INVALID_ARGUMENT, "batch is 0");
    const ConvGeom& g = p->geom;
    *L = ChainLayer{};
    const long long in_bytes = static_cast<long long>(batch) * g.H * g.W * g.Ci;
    const long long out_bytes = static_cast<long long>(batch) * g.Ho * g.Wo * g.Co;
    if (in_bytes >= (1ll << 31) || out_bytes >= (1ll << 31)) return SetError(MI355X_ERR_UNSUPPORTED, "chain: tensors of 2 GiB and more");
    if (p->algo == MI355X_ALGO_DEPTHWISE && p->variant == 1)
    {
        int rows = 1, cbw = 32;
        if (const int rc = FillDw3x3Args(p, batch, x, y, &L->dw, &rows, &cbw)) return rc;
        if (cbw != 128) return SetError(MI355X_ERR_UNSUPPORTED, "chain: depthwise layers need a channel count that is a multiple of 128 (%d)", g.Co);
        if (p->w_dot4b) return SetError(MI355X_ERR_UNSUPPORTED, "chain: depthwise weights that need two int8 halves");
        L->kind = kChainDw3x3;
        L->variant = (g.stride_x == 2 ? 2 : 0) + (rows == 1 ? 1 : 0);
        L->items_per_image = L->dw.tiles_x * L->dw.tiles_y * L->dw.cblocks;
        L->group = L->dw.cblocks;
        L->n_items = L->dw.total_blocks;
        L->out_rows = g.Ho * g.Wo;
        return 0;
    }
    if (p->algo == MI355X_ALGO_MFMA && p->bk128 && (g.Ci % 128) == 0 && p->pw_bn == 0 && p->zw_neg == 0 && (g.Co % 16) == 0 && p->w_mfma)
    {
        bool unit_fast = false;
        if (const int rc = FillIgemmLdsArgs(p, 64, 64, batch, x, y, &L->ig, &unit_fast)) return rc;
        if (!unit_fast) return SetError(MI355X_ERR_UNSUPPORTED, "chain: only 1x1 stride-1 unpadded convolutions run on the matrix cores here");
        L->tiles_n = L->ig.tiles_n;
        L->M = L->ig.M;
        L->out_rows = g.Ho * g.Wo;
        // Enough row blocks to go round: one work item per row block over all channels, the activation panel resident in LDS.
        const int nk = p->K_pad / 128;
        if (GlobalOptions().chain_panel != 0 && (nk == 2 || nk == 4) && L->ig.tiles_n * 64 <= kGemmPanelMaxCols && L->ig.tiles_m >= 96)
        {
            L->kind = kChainGemmPanel;
            L->variant = nk;
            L->n_items = L->ig.tiles_m;
            L->group = 1;
            return 0;
        }
        L->kind = kChainIgemm64;
        L->n_items = L->ig.tiles_m * L->ig.tiles_n;
        L->group = L->ig.tiles_n;
        return 0;
    }
    return SetError(MI355X_ERR_UNSUPPORTED, "chain: layer kind not supported (algo %d)", p->algo);
}

template <int ST>
int LaunchChain(const mi355x_chain_s* c, hipStream_t stream)
{
    const int smem = c->smem;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&LayerChainKernel<ST>), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    MI355X_HIP(attr);
    ChainArgs a;
    a.layers = c->d_layers; a.need = c->d_need; a.sync = c->d_sync;
    a.n_layers = static_cast<int>(c->layers.size()); a.batch = c->batch;
    for (int q = 0; q < kChainQueues; ++q) a.qtotal[q] = c->qtotal[q];
    a.timeout_ticks = c->timeout_ticks;
    a.defer_signal = c->defer_signal;
    a.stamps = nullptr;
    NoteKernel("LayerChainKernel<%d>", ST);
    hipLaunchKernelGGL((LayerChainKernel<ST>), dim3(c->grid), dim3(256), smem, stream, a);
    MI355X_HIP(hipGetLastError());
    return 0;
}

template <int ST>
int ChainOccupancy(int smem, int* blocks_per_cu)
{
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&LayerChainKernel<ST>), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    MI355X_HIP(attr);
    MI355X_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, reinterpret_cast<const void*>(&LayerChainKernel<ST>), 256, smem));
    return 0;
}

// Everything mi355x_chain_create and mi355x_chain_run_noalloc derive from the caller's arguments: layer records, queue
// sizes, the per-image tile counts, LDS size and grid.  Fills `c` (no device memory is touched) and `need_out`.
int DescribeRun(uint32_t n_layers, const mi355x_conv2d_t* plans, uint32_t batch, const void* input_dev, void* const* outputs_dev,
                mi355x_chain_s* c, std::vector<uint32_t>* need_out)
{
    if (n_layers == 0 || !plans || !outputs_dev || !input_dev) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: no layers / null pointers");
    if (batch == 0 || batch > 65535) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: batch must be 1 .. 65535");
    c->batch = static_cast<int>(batch);
    c->layers.resize(n_layers);
    struct Range { uintptr_t lo, hi; };
    std::vector<Range> ranges;
    long long items = 0;
    for (uint32_t k = 0; k < n_layers; ++k)
    {
        const mi355x_conv2d_s* p = plans[k];
        void* y = outputs_dev[k];
        const void* x = k == 0 ? input_dev : outputs_dev[k - 1];
        if (!p || !y) { return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: layer %u has a null plan or output", k); }
        if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(y) & 127) != 0)
        {
            return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: layer %u needs a 16-byte aligned input and a 128-byte aligned output", k);
        }
        ChainLayer& L = c->layers[k];
        if (const int rc = Describe(p, batch, x, y, &L)) { return rc; }
        const ConvGeom& g = p->geom;
        if (k > 0)
        {
            const ConvGeom& q = plans[k - 1]->geom;
            if (q.Ho != g.H || q.Wo != g.W || q.Co != g.Ci) { return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: layer %u does not consume layer %u's output shape", k, k - 1); }
            const mi355x_quant& a = plans[k - 1]->d.output; const mi355x_quant& b = p->d.input;
            if (a.dtype != b.dtype || a.scale != b.scale || a.offset != b.offset) { return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: layer %u reads another quantization than layer %u writes", k, k - 1); }
        }
        L.src = static_cast<int>(k) - 1;
        // queue q takes the layer's groups q, q + 8, ...: their items follow those of the layers before
        const int n_groups = L.n_items / L.group;
        for (int q = 0; q < kChainQueues; ++q)
        {
            L.qfirst[q] = c->qtotal[q];
            c->qtotal[q] += (n_groups > q ? (n_groups - q + kChainQueues - 1) / kChainQueues : 0) * L.group;
        }
        items += L.n_items;
        if (items > 0x3fffffffll) { return SetError(MI355X_ERR_UNSUPPORTED, "chain: too many work items"); }
        if (k == 0) ranges.push_back(Range{reinterpret_cast<uintptr_t>(x), reinterpret_cast<uintptr_t>(x) + static_cast<uintptr_t>(batch) * g.H * g.W * g.Ci});
        ranges.push_back(Range{reinterpret_cast<uintptr_t>(y), reinterpret_cast<uintptr_t>(y) + static_cast<uintptr_t>(batch) * g.Ho * g.Wo * g.Co});
    }
    // every tensor of the run is written once and read only when complete: none may share bytes with another
    for (size_t i = 0; i < ranges.size(); ++i)
        for (size_t j = i + 1; j < ranges.size(); ++j)
            if (ranges[i].lo < ranges[j].hi && ranges[j].lo < ranges[i].hi)
            {
                    return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain: tensors %zu and %zu of the run overlap (0 = the input, k = output of layer k - 1)", i, j);
            }
    c->total_items = static_cast<int>(items);

    // tiles of layer l that touch image n
    std::vector<uint32_t>& need = *need_out;
    need.assign(static_cast<size_t>(n_layers) * batch, 0u);
    for (uint32_t k = 0; k < n_layers; ++k)
    {
        const ChainLayer& L = c->layers[k];
        for (uint32_t n = 0; n < batch; ++n)
        {
            if (L.kind == kChainDw3x3) need[static_cast<size_t>(k) * batch + n] = static_cast<uint32_t>(L.items_per_image);
            else
            {
                // row blocks of 64 that intersect rows [n * out_rows, (n + 1) * out_rows), times the column tiles
                const long long r0 = static_cast<long long>(n) * L.out_rows, r1 = r0 + L.out_rows - 1;
                need[static_cast<size_t>(k) * batch + n] = static_cast<uint32_t>((r1 / 64 - r0 / 64 + 1) * (L.kind == kChainGemmPanel ? 1 : L.tiles_n));
            }
        }
    }
    const Options& opt = GlobalOptions();
    c->stages = opt.chain_stages == 3 ? 3 : opt.chain_stages == 4 ? 4 : 2;
    c->defer_signal = opt.chain_defer_signal;
    // LDS per block: the largest any work item of this run needs
    c->smem = c->stages == 3 ? ChainSmemBytes<3>() : c->stages == 4 ? ChainSmemBytes<4>() : ChainSmemBytes<2>();
    for (const ChainLayer& L : c->layers)
        if (L.kind == kChainGemmPanel)
            c->smem = std::max(c->smem, L.variant == 2 ? GemmPanelSmemBytes<kChainPanelStages, 2>(L.tiles_n * 64) : GemmPanelSmemBytes<kChainPanelStages, 4>(L.tiles_n * 64));
    int per_cu = 0;
    int rc = c->stages == 3 ? ChainOccupancy<3>(c->smem, &per_cu) : c->stages == 4 ? ChainOccupancy<4>(c->smem, &per_cu) : ChainOccupancy<2>(c->smem, &per_cu);
    if (rc) { return rc; }
    if (per_cu < 1) { return SetError(MI355X_ERR_UNSUPPORTED, "chain: the kernel does not fit a CU"); }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
    {
        return SetError(MI355X_ERR_NO_DEVICE, "chain: cannot read the device's CU count");
    }
    if (opt.chain_blocks_per_cu > 0) per_cu = std::min(per_cu, opt.chain_blocks_per_cu);
    // at least one block per queue; never more blocks than the device holds at once
    c->grid = std::max(kChainQueues, std::min(c->total_items, per_cu * cus));

    return 0;
}

} // namespace

extern "C" {

int mi355x_chain_accepts(mi355x_conv2d_t plan, uint32_t batch)
{
    ChainLayer L;
    // addresses do not matter for the answer
    return Describe(plan, batch, nullptr, nullptr, &L);
}

int mi355x_chain_create(uint32_t n_layers, const mi355x_conv2d_t* plans, uint32_t batch, const void* input_dev, void* const* outputs_dev,
                        mi355x_chain_t* chain)
{
    if (!chain) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain pointer is null");
    *chain = nullptr;
    auto c = new mi355x_chain_s;
    std::vector<uint32_t> need;
    int rc = DescribeRun(n_layers, plans, batch, input_dev, outputs_dev, c, &need);
    if (rc) { delete c; return rc; }
    const size_t sync_words = (static_cast<size_t>(kChainCounterSlot) + need.size()) * kChainSlot;
    const std::vector<uint32_t> zeros(sync_words, 0u);
    if (hipMalloc(reinterpret_cast<void**>(&c->d_layers), c->layers.size() * sizeof(ChainLayer)) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&c->d_need), need.size() * 4) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&c->d_sync), sync_words * 4) != hipSuccess)
    {
        delete c;
        return SetError(MI355X_ERR_OUT_OF_MEMORY, "chain: out of device memory");
    }
    rc = UploadNow(c->d_layers, c->layers.data(), c->layers.size() * sizeof(ChainLayer));
    if (!rc) rc = UploadNow(c->d_need, need.data(), need.size() * 4);
    if (!rc) rc = UploadNow(c->d_sync, zeros.data(), sync_words * 4);
    if (rc) { delete c; return rc; }
    *chain = c;
    return 0;
}

int mi355x_chain_run(mi355x_chain_t chain, mi355x_stream_t stream)
{
    if (!chain) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain is null");
    if (chain->stages == 3) return LaunchChain<3>(chain, ToHip(stream));
    if (chain->stages == 4) return LaunchChain<4>(chain, ToHip(stream));
    return LaunchChain<2>(chain, ToHip(stream));
}

int mi355x_chain_run_noalloc(uint32_t n_layers, const mi355x_conv2d_t* plans, uint32_t batch, const void* input_dev, void* const* outputs_dev,
                             mi355x_stream_t stream)
{
    if (n_layers > kNoallocMaxLayers || batch > kNoallocMaxBatch)
        return SetError(MI355X_ERR_UNSUPPORTED, "chain without allocation: at most %u layers and %u images (got %u and %u); use mi355x_chain_create",
                        kNoallocMaxLayers, kNoallocMaxBatch, n_layers, batch);
    // the array's address on the current device, looked up once per device
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static unsigned char* base_of[kMaxDevices] = {};
    int dev = 0;
    MI355X_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return SetError(MI355X_ERR_UNSUPPORTED, "chain without allocation: device index %d", dev);
    unsigned char* base = nullptr;
    {
        std::lock_guard<std::mutex> lock(mutex);
        if (!base_of[dev])
        {
            void* p = nullptr;
            MI355X_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            base_of[dev] = static_cast<unsigned char*>(p);
        }
        base = base_of[dev];
    }
    // the description lives in the calling thread's own storage, which keeps its capacity from call to call
    thread_local mi355x_chain_s host;
    thread_local std::vector<uint32_t> need;
    host.layers.clear();
    host.total_items = 0;
    for (int q = 0; q < kChainQueues; ++q) host.qtotal[q] = 0;
    if (const int rc = DescribeRun(n_layers, plans, batch, input_dev, outputs_dev, &host, &need)) return rc;
    host.d_sync = reinterpret_cast<uint32_t*>(base);
    host.d_need = reinterpret_cast<uint32_t*>(base + kNoallocSyncBytes);
    host.d_layers = reinterpret_cast<ChainLayer*>(base + kNoallocSyncBytes + kNoallocNeedBytes);
    hipStream_t s = ToHip(stream);
    // The array keeps what the call before left there.  Queue heads and counters must start at zero (a launch leaves them so,
    // but one that gave up, or a larger run before, may not have): a fill kernel, which a captured graph can hold.
    const size_t sync_bytes = (static_cast<size_t>(kChainCounterSlot) + need.size()) * kChainSlot * 4;
    int rc = mi355x_fill_u8(host.d_sync, 0, sync_bytes, stream);
    if (!rc) rc = hipMemcpyAsync(host.d_need, need.data(), need.size() * 4, hipMemcpyHostToDevice, s) == hipSuccess ? 0 : SetError(MI355X_ERR_INVALID_ARGUMENT, "chain without allocation: copy of the tile counts failed");
    if (!rc) rc = hipMemcpyAsync(host.d_layers, host.layers.data(), host.layers.size() * sizeof(ChainLayer), hipMemcpyHostToDevice, s) == hipSuccess ? 0 : SetError(MI355X_ERR_INVALID_ARGUMENT, "chain without allocation: copy of the layer records failed");
    if (!rc) rc = host.stages == 3 ? LaunchChain<3>(&host, s) : host.stages == 4 ? LaunchChain<4>(&host, s) : LaunchChain<2>(&host, s);
    // the thread-local object must not free the static array
    host.d_sync = nullptr; host.d_need = nullptr; host.d_layers = nullptr;
    return rc;
}

int mi355x_chain_status(mi355x_chain_t chain, uint32_t* gave_up)
{
    if (!chain || !gave_up) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain / result pointer is null");
    hipStream_t s = nullptr;
    if (const int rc = OwnStreamGet(&s)) return rc;
    uint32_t words[4] = {0, 0, 0, 0};
    MI355X_HIP(hipMemcpyAsync(words, chain->d_sync + kChainMiscSlot * kChainSlot, sizeof(words), hipMemcpyDeviceToHost, s));
    MI355X_HIP(hipStreamSynchronize(s));
    const uint32_t abort = words[kChainAbort - kChainMiscSlot * kChainSlot], timeouts = words[kChainTimeouts - kChainMiscSlot * kChainSlot];
    *gave_up = timeouts + (abort != 0 && timeouts == 0 ? 1u : 0u);
    if (abort != 0 || timeouts != 0)
    {
        // a run that gave up leaves its flag standing; clear it so that the chain can be used again
        const uint32_t z[2] = {0u, 0u};
        MI355X_HIP(hipMemcpyAsync(chain->d_sync + kChainAbort, z, sizeof(z), hipMemcpyHostToDevice, s));
        MI355X_HIP(hipStreamSynchronize(s));
    }
    return 0;
}

int mi355x_chain_run_stamped(mi355x_chain_t chain, mi355x_stream_t stream, uint64_t* sums)
{
    if (!chain || !sums) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain / result pointer is null");
    if (chain->stages != 2) return SetError(MI355X_ERR_UNSUPPORTED, "stamped runs exist for two LDS stages only");
    const int smem = chain->smem;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&LayerChainKernel<2, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    MI355X_HIP(attr);
    unsigned long long* d = nullptr;
    const size_t words = static_cast<size_t>(chain->grid) * kChainStampWords;
    MI355X_HIP(hipMalloc(reinterpret_cast<void**>(&d), words * 8));
    ChainArgs a;
    a.layers = chain->d_layers; a.need = chain->d_need; a.sync = chain->d_sync;
    a.n_layers = static_cast<int>(chain->layers.size()); a.batch = chain->batch;
    for (int q = 0; q < kChainQueues; ++q) a.qtotal[q] = chain->qtotal[q];
    a.timeout_ticks = chain->timeout_ticks;
    a.defer_signal = chain->defer_signal;
    a.stamps = d;
    hipLaunchKernelGGL((LayerChainKernel<2, true>), dim3(chain->grid), dim3(256), smem, ToHip(stream), a);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(ToHip(stream));
    std::vector<unsigned long long> h(words, 0ull);
    if (e == hipSuccess) e = hipMemcpy(h.data(), d, words * 8, hipMemcpyDeviceToHost);
    (void)hipFree(d);
    if (e != hipSuccess) return HipFail(e, "stamped chain run");
    for (int w = 0; w < kChainStampWords; ++w) sums[w] = 0;
    for (size_t i = 0; i < words; ++i) sums[i % kChainStampWords] += h[i];
    return 0;
}

int mi355x_chain_info(mi355x_chain_t chain, uint32_t* work_items, uint32_t* blocks)
{
    if (!chain) return SetError(MI355X_ERR_INVALID_ARGUMENT, "chain is null");
    if (work_items) *work_items = static_cast<uint32_t>(chain->total_items);
    if (blocks) *blocks = static_cast<uint32_t>(chain->grid);
    return 0;
}

int mi355x_chain_destroy(mi355x_chain_t chain)
{
    delete chain;
    return 0;
}

} // extern "C"
