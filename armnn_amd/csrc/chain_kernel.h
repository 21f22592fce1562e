// A run of consecutive layers as ONE persistent launch: blocks draw (layer, tile) work items from queues in layer
// order and a tile starts as soon as the images it reads are complete in the producing layer -- no kernel boundary, no
// device-wide barrier between layers.  The tiles are the ones the per-layer kernels compute (same device functions,
// same bytes); what changes is that tiles of neighbouring layers, in different phases (staging, v_dot4, MFMA k-loop,
// requantization, stores), share a CU at the same time, and that the dispatch / ramp / drain / write-back cost of a
// launch is paid once per run instead of once per layer.
//
// Hand-over between blocks, which run on 8 XCDs with private L2s:
//   producer  every output store is written through L2 as it is issued (sc1); after its tile the block waits for its
//             stores (s_waitcnt vmcnt(0)), meets at a barrier, and adds 1 to the counter of every image the tile touched
//             (agent-scope atomics, executed at the memory side; every counter has a cache line to itself).
//   consumer  one wave looks at the counters of the images its tile reads (agent-scope atomic loads) until each has
//             reached the number of tiles the host counted for that image, then the block reads with ordinary loads.
//   No cache is ever stale for such a read: every address is written once per launch, a line is read only after its
//   image is complete, and no L2 or L1 holds lines of the run's tensors from before (the launch itself starts with
//   invalidated caches).  Fences are not used: a release fence writes back the whole L2 (tens of microseconds each).
//   The host checks that the run's tensors do not overlap.
// Queues: one per XCD (blocks with id q modulo 8 pop queue q), because atomics on ONE address execute one after the other,
//   about 11 ns each on this device -- a single queue head delivers 90 tiles per microsecond, a third of what these
//   tiles need.  A layer's items are dealt to the queues in groups (the column tiles of a row block, the channel blocks
//   of a depthwise tile), so tiles that read the same lines run on one XCD.
// Progress: within a queue, positions are in dependency order and handed out in that order, and an item depends only on
//   items of earlier layers; so the earliest unfinished item of the whole run is always held by a running block that
//   waits for nothing.  Every wait is bounded by a wall-clock limit all the same: a block that exceeds it raises the run's
//   abort flag, and every block leaves at its next wait.
// The queue heads, the exit counts and the per-image counters live in device memory owned by the chain object; the last
// block to leave sets them back to zero for the next launch.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "conv_kernels.h"
#include "device_math.h"
#include "dw_stem_kernels.h"
#include "igemm_lds_kernel.h"
#include "gemm_panel_task.h"

namespace mi355x
{

enum ChainKind : int
{
    kChainIgemm64 = 1,     // IgemmLdsTile<64, 64, 2, 2, ST, true, false, true>: 1x1 stride-1 unpadded convolution, 64 x 64 tiles
    kChainDw3x3   = 2,     // Depthwise3x3Block<S, R, false, 128, true>
    kChainGemmPanel = 3,   // GemmPanelTask<3, NK, true>: the same convolutions, one work item per 64 output rows over all channels
};
constexpr int kChainPanelStages = 3;

constexpr int kChainQueues = 8;      // one work queue per XCD: blocks whose id is q modulo 8 (the XCD the hardware deals them to) pop queue q

struct ChainLayer
{
    // header words, read by index in the kernel (kChainHdr*)
    int kind;
    int variant;           // kChainDw3x3: (stride == 2 ? 2 : 0) + (rows per thread == 1 ? 1 : 0); kChainGemmPanel: k-tiles (K / 128)
    int group;             // consecutive work items that stay together on one queue: the column tiles of a row block
                           // (they read the same activation rows), the channel blocks of a depthwise tile
    int n_items;
    int src;               // layer whose output this one reads; -1: the run's input, complete before the launch
    int out_rows;          // output pixels per image (igemm: rows of the GEMM per image)
    int items_per_image;   // depthwise: work items per image
    int tiles_n;           // igemm: column tiles per row block
    int M;                 // igemm: rows of the GEMM
    int reserved[7];
    int qfirst[kChainQueues];   // position in queue q of the layer's first item there (groups q, q + 8, ... of the layer, in order)
    IgemmArgs ig;
    Dw3x3Args dw;
};
enum { kChainHdrKind = 0, kChainHdrVariant, kChainHdrGroup, kChainHdrItems, kChainHdrSrc, kChainHdrOutRows, kChainHdrPerImage, kChainHdrTilesN, kChainHdrM,
       kChainHdrQFirst = 16 };

// ChainArgs::sync, in 32-dword (128-byte) slots so that no two counters share a cache line: atomics on one line are
// executed one after the other (about 11 ns each on this device, whichever words they touch).
//   slot q (0..7): head of queue q            slot 8 + q: blocks of queue q that have left
//   slot 16: word 0 queues whose blocks have all left, word 1 abort flag, word 2 waits that ran out
//   slot kChainCounterSlot + l * batch + n: tiles of layer l finished for image n
constexpr int kChainSlot = 32;
constexpr int kChainExitSlot = 8, kChainMiscSlot = 16, kChainCounterSlot = 17;
constexpr int kChainAbort = kChainMiscSlot * kChainSlot + 1, kChainTimeouts = kChainMiscSlot * kChainSlot + 2;

struct ChainArgs
{
    const ChainLayer* layers;
    const uint32_t*   need;     // [n_layers][batch]: tiles of layer l that touch image n
    uint32_t*         sync;     // (kChainCounterSlot + n_layers * batch) slots, zero between launches
    int n_layers, batch;
    int qtotal[kChainQueues];   // items in queue q
    long long timeout_ticks;    // of the 100 MHz wall clock
    int defer_signal;           // 1: a tile is counted as finished behind the next tile's loads instead of right after its stores have been waited for
    unsigned long long* stamps; // STAMPS instances: [blocks][kChainStampWords] shader-clock sums per phase, else null
};

// words of a block's stamp record: cycles spent popping, waiting for producers, in matrix-core tiles, in depthwise tiles,
// draining stores + barrier; then the number of matrix-core tiles, of depthwise tiles, and of tiles that had to wait
constexpr int kChainStampWords = 8;

template <typename T>
__device__ __forceinline__ T LoadUniformStruct(const T* p)
{
    // wave-uniform address in memory nobody writes during the launch: scalar loads
    static_assert(sizeof(T) % 4 == 0, "whole dwords");
    T v;
    const uint32_t MI355X_CONST_AS* s = (const uint32_t MI355X_CONST_AS*)p;
    uint32_t* d = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 4; ++i) d[i] = s[i];
    return v;
}

template <int ST>
constexpr int ChainSmemBytes()
{
    constexpr int ig = IgemmLdsSmemBytes<64, 64, ST>();
    constexpr int d0 = Dw3x3Tile<1, 2, 128>::SMEM, d1 = Dw3x3Tile<1, 1, 128>::SMEM, d2 = Dw3x3Tile<2, 2, 128>::SMEM, d3 = Dw3x3Tile<2, 1, 128>::SMEM;
    int m = ig;
    m = d0 > m ? d0 : m; m = d1 > m ? d1 : m; m = d2 > m ? d2 : m; m = d3 > m ? d3 : m;
    return m;
}

// The tile kinds as functions of their own (not inlined): a kernel that inlines them all needs the sum of their
// registers rather than the maximum, and the persistent blocks then fit a CU two at a time instead of four.
// Arguments arrive in vector registers; the uniform ones are made scalar again so that the layer record is read with
// scalar loads.
typedef __attribute__((address_space(3))) uint8_t* ChainLdsPtr;

template <typename T>
__device__ __forceinline__ T* UniformPointer(T* p)
{
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return reinterpret_cast<T*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// What a block does behind a tile's last load, while the tile's own write-out is still to come:
//   * it counts the tile BEFORE as finished.  That tile's stores were issued before this tile's loads, a wave's vector
//     memory operations complete in issue order, and every wave has waited for this tile's loads and met the others at a
//     barrier since: all of them are written through.  (Waiting for them right after the tile cost a tenth of the time.)
//   * lane 0 takes the block's next position from the queue, so that the answer is there when the tile is done.
struct ChainHook
{
    uint32_t* sig;         // this lane's counter of the tile before; null: none
    uint32_t* queue;       // queue head; null: no pop
    int* popped;
    __device__ __forceinline__ void operator()() const
    {
        if (threadIdx.x < 64)
        {
            if (sig) __hip_atomic_fetch_add(sig, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (threadIdx.x == 0 && queue) *popped = static_cast<int>(__hip_atomic_fetch_add(queue, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        }
    }
};

template <int ST>
__device__ __attribute__((noinline)) int ChainIgemmTile(const ChainLayer* L, int local, ChainLdsPtr lds, uint32_t* sig, uint32_t* queue)
{
    L = UniformPointer(L);
    local = __builtin_amdgcn_readfirstlane(local);
    queue = UniformPointer(queue);
    int popped = 0;
    const IgemmArgs a = LoadUniformStruct(&L->ig);
    IgemmLdsTile<64, 64, 2, 2, ST, true, false, true>(a, local, (uint8_t*)lds, ChainHook{sig, queue, &popped});
    return popped;
}

template <int NK>
__device__ __attribute__((noinline)) int ChainPanelTask(const ChainLayer* L, int local, ChainLdsPtr lds, uint32_t* sig, uint32_t* queue)
{
    L = UniformPointer(L);
    local = __builtin_amdgcn_readfirstlane(local);
    queue = UniformPointer(queue);
    int popped = 0;
    const IgemmArgs a = LoadUniformStruct(&L->ig);
    GemmPanelTask<kChainPanelStages, NK, true>(a, local, (uint8_t*)lds);
    ChainHook{sig, queue, &popped}();        // the task's k-loops have waited for loads and met at barriers many times
    return popped;
}

template <int S, int R>
__device__ __attribute__((noinline)) int ChainDwTile(const ChainLayer* L, int local, ChainLdsPtr lds, uint32_t* sig, uint32_t* queue)
{
    L = UniformPointer(L);
    local = __builtin_amdgcn_readfirstlane(local);
    queue = UniformPointer(queue);
    int popped = 0;
    const Dw3x3Args a = LoadUniformStruct(&L->dw);
    Depthwise3x3Block<S, R, false, 128, true>(a, local, (uint8_t*)lds, ChainHook{sig, queue, &popped});
    return popped;
}

#ifndef MI355X_CHAIN_WAVES_PER_SIMD
#define MI355X_CHAIN_WAVES_PER_SIMD 4
#endif

// Blocks draw work items from the queue of their XCD, in order; queue q holds, layer after layer, the item groups
// q, q + 8, ... of each layer.  A single queue head would bound the whole run: the device executes atomics on one
// address at about 90 million per second, a quarter of the rate at which these tiles finish.
template <int ST, bool STAMPS = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MI355X_CHAIN_WAVES_PER_SIMD, MI355X_CHAIN_WAVES_PER_SIMD)))
void LayerChainKernel(ChainArgs c)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int s_pos, s_flag;
    [[maybe_unused]] unsigned long long st_sum[kChainStampWords] = {};
    [[maybe_unused]] long long st_t = STAMPS ? clock64() : 0;
    auto stamp = [&](int word) {
        if constexpr (STAMPS)
        {
            const long long now = clock64();
            st_sum[word] += static_cast<unsigned long long>(now - st_t);
            st_t = now;
        }
    };
    const int tid = threadIdx.x;
    const int q = static_cast<int>(blockIdx.x) & (kChainQueues - 1);
    const int qtotal = c.qtotal[q];
    uint32_t* const queue = c.sync + q * kChainSlot;
    const int MI355X_CONST_AS* lw = (const int MI355X_CONST_AS*)c.layers;
    constexpr int LW = sizeof(ChainLayer) / 4;           // dwords per layer record
    static_assert(sizeof(ChainLayer) % 4 == 0, "whole dwords");

    struct Item { int l, kind, variant, local, src, i0, i1; };
    // positions come in increasing order, so the search for a position's layer starts at the layer of the one before
    auto decode = [&](int pos, int l) {
        Item it;
        while (l + 1 < c.n_layers && pos >= lw[(l + 1) * LW + kChainHdrQFirst + q]) ++l;
        it.l = l;
        it.kind = lw[l * LW + kChainHdrKind];
        it.variant = lw[l * LW + kChainHdrVariant];
        it.src = lw[l * LW + kChainHdrSrc];
        const int group = lw[l * LW + kChainHdrGroup];
        const int in_layer = pos - lw[l * LW + kChainHdrQFirst + q];
        it.local = (q + kChainQueues * (in_layer / group)) * group + in_layer % group;
        // images this tile reads (and writes: every tile kind maps image n of the input to image n of the output)
        if (it.kind != kChainDw3x3)
        {
            const int out_rows = lw[l * LW + kChainHdrOutRows];
            const int m0 = (it.kind == kChainIgemm64 ? it.local / lw[l * LW + kChainHdrTilesN] : it.local) * 64;
            const int m1 = min(m0 + 64, lw[l * LW + kChainHdrM]) - 1;
            it.i0 = m0 / out_rows;
            it.i1 = m1 / out_rows;
        }
        else
        {
            it.i0 = it.i1 = it.local / lw[l * LW + kChainHdrPerImage];
        }
        return it;
    };
    // the tile before, not yet counted as finished (its stores may still be on their way)
    bool owed = false;
    int owed_l = 0, owed_i0 = 0, owed_i1 = 0;
    // all of the block: wait for every store issued so far, then count the owed tile
    auto settle = [&]() {
        __builtin_amdgcn_s_waitcnt(0);           // vmcnt(0) expcnt(0) lgkmcnt(0): this wave's stores have been written through
        __syncthreads();
        if (owed && tid <= owed_i1 - owed_i0)
            __hip_atomic_fetch_add(c.sync + (kChainCounterSlot + owed_l * c.batch + owed_i0 + tid) * kChainSlot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        owed = false;
    };

    int popped = 0;
    if (tid == 0) popped = static_cast<int>(__hip_atomic_fetch_add(queue, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    int l = 0;
    for (;;)
    {
        // ---- wave 0: the position lane 0 holds, and a first look at the counters of the images that tile reads ----------
        if (tid < 64)
        {
            const int pos = __builtin_amdgcn_readfirstlane(popped);
            int ready = 1;
            if (pos < qtotal)
            {
                const Item it = decode(pos, l);
                if (it.src >= 0)
                {
                    const int slot = it.src * c.batch + min(it.i0 + tid, it.i1);
                    const uint32_t seen = __hip_atomic_load(c.sync + (kChainCounterSlot + slot) * kChainSlot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ready = __builtin_amdgcn_ballot_w64(seen < c.need[slot]) == 0;
                }
            }
            if (tid == 0) { s_pos = pos; s_flag = ready; }
        }
        __syncthreads();
        const int pos = __builtin_amdgcn_readfirstlane(s_pos);
        const bool ready = __builtin_amdgcn_readfirstlane(s_flag) != 0;
        stamp(0);
        if (pos >= qtotal) break;
        const Item it = decode(pos, l);
        l = it.l;
        // ---- wait for the producer's images (only when the first look found them incomplete) ---------------------------
        if (!ready)
        {
            // first pay what this block owes: the tile it has not yet counted may be what a producer of this one waits for
            if (owed) settle();
            else __syncthreads();                // s_flag is rewritten below: everyone has read it
            if (tid < 64)
            {
                const int slot = it.src * c.batch + min(it.i0 + tid, it.i1);
                const uint32_t want = c.need[slot];
                const uint32_t* ctr = c.sync + (kChainCounterSlot + slot) * kChainSlot;
                int flag = 0;
                if constexpr (STAMPS) st_sum[7] += 1;
                const long long t0 = wall_clock64();
                while (__builtin_amdgcn_ballot_w64(__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) != 0)
                {
                    __builtin_amdgcn_s_sleep(8);
                    if (__hip_atomic_load(c.sync + kChainAbort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { flag = 1; break; }
                    if (wall_clock64() - t0 > c.timeout_ticks)
                    {
                        if (tid == 0)
                        {
                            __hip_atomic_fetch_add(c.sync + kChainTimeouts, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            __hip_atomic_store(c.sync + kChainAbort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                        flag = 1;
                        break;
                    }
                }
                if (tid == 0) s_flag = flag;
            }
            __syncthreads();
            if (s_flag != 0) break;
        }
        stamp(1);
        // ---- the tile; behind its loads the tile before is counted and the next position taken ---------------------------
        uint32_t* sig = nullptr;
        if (owed && tid <= owed_i1 - owed_i0) sig = c.sync + (kChainCounterSlot + owed_l * c.batch + owed_i0 + tid) * kChainSlot;
        const ChainLayer* L = c.layers + it.l;
        ChainLdsPtr lds = (ChainLdsPtr)smem;
        if (it.kind == kChainIgemm64) popped = ChainIgemmTile<ST>(L, it.local, lds, sig, queue);
        else if (it.kind == kChainGemmPanel)
        {
            if (it.variant == 2) popped = ChainPanelTask<2>(L, it.local, lds, sig, queue);
            else popped = ChainPanelTask<4>(L, it.local, lds, sig, queue);
        }
        else if (it.variant == 0) popped = ChainDwTile<1, 2>(L, it.local, lds, sig, queue);
        else if (it.variant == 1) popped = ChainDwTile<1, 1>(L, it.local, lds, sig, queue);
        else if (it.variant == 2) popped = ChainDwTile<2, 2>(L, it.local, lds, sig, queue);
        else popped = ChainDwTile<2, 1>(L, it.local, lds, sig, queue);
        owed = true; owed_l = it.l; owed_i0 = it.i0; owed_i1 = it.i1;
        stamp(it.kind != kChainDw3x3 ? 2 : 3);
        if constexpr (STAMPS) st_sum[it.kind != kChainDw3x3 ? 5 : 6] += 1;
        if (!c.defer_signal)
        {
            settle();
            stamp(4);
        }
        // (the next iteration's barrier also separates this tile's last LDS reads from the next tile's first LDS writes)
    }
    if (owed) settle();
    stamp(4);
    if constexpr (STAMPS)
    {
        if (tid == 0 && c.stamps)
            for (int w = 0; w < kChainStampWords; ++w) c.stamps[static_cast<size_t>(blockIdx.x) * kChainStampWords + w] = st_sum[w];
    }
    // ---- leave; the last block out zeroes the queues and the counters for the next launch ------------------------------
    __syncthreads();
    if (tid == 0)
    {
        int last = 0;
        const uint32_t mine = (gridDim.x - static_cast<uint32_t>(q) + kChainQueues - 1) / kChainQueues;      // blocks on this queue
        if (__hip_atomic_fetch_add(c.sync + (kChainExitSlot + q) * kChainSlot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == mine)
        {
            const uint32_t queues = gridDim.x < static_cast<uint32_t>(kChainQueues) ? gridDim.x : static_cast<uint32_t>(kChainQueues);
            last = __hip_atomic_fetch_add(c.sync + kChainMiscSlot * kChainSlot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == queues;
        }
        s_flag = last;
    }
    __syncthreads();
    if (s_flag != 0)
    {
        const int n = c.n_layers * c.batch;
        for (int i = tid; i < n; i += 256) __hip_atomic_store(c.sync + (kChainCounterSlot + i) * kChainSlot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid < 2 * kChainQueues) __hip_atomic_store(c.sync + tid * kChainSlot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0) __hip_atomic_store(c.sync + kChainMiscSlot * kChainSlot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

} // namespace mi355x
