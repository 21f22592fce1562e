// The tail of a classifier -- global pooling -> FullyConnected -> Softmax -- as ONE launch.  Each stage needs all of the
// stage before (every pooled vector before a 32-row tile of the logits, whose weights are read once per tile and not once
// per image; all logits of a row before its Softmax), so the stages hand over through two device-wide counters:
//   producer  writes its outputs through L2 as it stores them (sc1), waits for its stores, meets at a barrier and adds
//             the number of items it finished to the stage's counter (agent-scope atomic, executed at the memory side);
//   consumer  one lane polls the counter (agent-scope atomic loads) until it has reached the stage's item count, then the
//             block reads with ordinary loads.  No cache holds a stale line: the pooled vectors and the logits are
//             written once per launch, read only after ALL of them are complete (so a line shared by two rows is never
//             fetched half-written), and the launch starts with invalidated caches.  No fences (a release fence writes
//             back the whole L2).
// Blocks: at most one per CU and never more than the device holds at once, so every block is resident or becomes so
// without waiting for a block of this launch; every wait is bounded by a wall-clock limit and raises an abort flag the
// other blocks see.  Work is dealt statically: block b pools items b, b + G, ...; computes tiles b, b + G, ... of the
// logits; rows are dealt from the other end of the grid (G - 1 - b), so that at the usual sizes no block holds two
// dependent items in a row.  The last block to leave sets the counters back to zero for the next launch.
// The item bodies are the per-layer kernels' own (GlobalPoolItem, SmallMGemmTile, SoftmaxRowItem): same bytes.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "device_math.h"
#include "pool_softmax_items.h"
#include "pw_gemm_kernel.h"

namespace mi355x
{

// TailArgs::sync in 32-dword slots (no two counters share a cache line; atomics on one line execute one after the other,
// about 11 ns each, so each stage counts in eight slots -- block b adds to slot b % 8 -- and a waiting block sums them):
// slots 0..7 pooling items finished, 8..15 tiles of the logits finished, 16 blocks that have left, 17 word 0 abort flag,
// word 1 waits that ran out.
constexpr int kTailSlot = 32, kTailWays = 8;
constexpr int kTailPoolDone = 0, kTailFcDone = kTailWays * kTailSlot, kTailExit = 2 * kTailWays * kTailSlot, kTailAbort = kTailExit + kTailSlot,
              kTailTimeouts = kTailAbort + 1;
constexpr int kTailSyncWords = kTailAbort + kTailSlot;

struct TailArgs
{
    PoolArgs pool;
    QIn pool_in;
    Requant pool_rq;
    const uint8_t* x;          // [batch][H][W][C]
    uint8_t* pooled;           // [batch][C]
    GemvArgs fc;               // x = pooled, y = logits [batch][N], M = batch
    int cols;                  // = fc.N
    float beta;
    QIn sm_in;
    Requant sm_rq;
    uint8_t* out;              // [batch][N]
    int batch, pool_items, fc_tiles_n, fc_tiles;
    uint32_t* sync;
    long long timeout_ticks;   // of the 100 MHz wall clock
};

template <int UN, int V>
__global__ __launch_bounds__(256) void TailKernel(TailArgs t)
{
    // pooling: taps * 64 dwords; logits: 4 x 16 x 64 + 4 x 64 ints; Softmax: 8 floats
    __shared__ __align__(16) uint32_t smem[kGlobalPoolMaxTaps * 64];
    __shared__ int s_flag;
    const int tid = threadIdx.x;
    const int G = static_cast<int>(gridDim.x);
    const int b = static_cast<int>(blockIdx.x);

    // all of the block: wait for this wave's stores, meet, and count `n` finished items on `ctr`
    auto publish = [&](uint32_t* ctr, int n) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) __hip_atomic_fetch_add(ctr + (b % kTailWays) * kTailSlot, static_cast<uint32_t>(n), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    // all of the block: true once the stage's slots add up to `want`, false when the run has been given up
    auto wait_for = [&](const uint32_t* ctr, uint32_t want) -> bool {
        if (tid < 64)
        {
            int flag = 0;
            const long long t0 = wall_clock64();
            for (;;)
            {
                uint32_t seen = tid < kTailWays ? __hip_atomic_load(ctr + tid * kTailSlot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
#pragma unroll
                for (int o = 1; o < kTailWays; o <<= 1) seen += __shfl_xor(seen, o);
                if (__builtin_amdgcn_readfirstlane(seen) >= want) break;
                __builtin_amdgcn_s_sleep(2);
                if (__hip_atomic_load(t.sync + kTailAbort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { flag = 1; break; }
                if (wall_clock64() - t0 > t.timeout_ticks)
                {
                    if (tid == 0)
                    {
                        __hip_atomic_fetch_add(t.sync + kTailTimeouts, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(t.sync + kTailAbort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    flag = 1;
                    break;
                }
            }
            if (tid == 0) s_flag = flag;
        }
        __syncthreads();
        const bool ok = s_flag == 0;
        __syncthreads();                 // s_flag may be rewritten by the next wait
        return ok;
    };

    // ---- pooling -------------------------------------------------------------------------------------------------------
    int done = 0;
    for (int item = b; item < t.pool_items; item += G)
    {
        if (done) __syncthreads();       // the item before still read its taps from LDS
        GlobalPoolItem<true>(t.pool, t.pool_in, t.pool_rq, t.x, t.pooled, item, smem);
        ++done;
    }
    if (done) publish(t.sync + kTailPoolDone, done);

    // ---- logits --------------------------------------------------------------------------------------------------------
    bool alive = true;
    done = 0;
    for (int tile = b; tile < t.fc_tiles && alive; tile += G)
    {
        if (done == 0) alive = wait_for(t.sync + kTailPoolDone, static_cast<uint32_t>(t.pool_items));
        else __syncthreads();            // the tile before still read its partial sums from LDS
        if (!alive) break;
        int (*part)[16][64] = reinterpret_cast<int (*)[16][64]>(smem);
        int (*rowpart)[64] = reinterpret_cast<int (*)[64]>(smem + 4 * 16 * 64);
        SmallMGemmTile<UN, true>(t.fc, (tile % t.fc_tiles_n) * 32, (tile / t.fc_tiles_n) * 32, part, rowpart);
        ++done;
    }
    if (done) publish(t.sync + kTailFcDone, done);

    // ---- Softmax -------------------------------------------------------------------------------------------------------
    done = 0;
    for (int row = G - 1 - b; row < t.batch && alive; row += G)
    {
        if (done == 0) alive = wait_for(t.sync + kTailFcDone, static_cast<uint32_t>(t.fc_tiles));
        else __syncthreads();
        if (!alive) break;
        SoftmaxRowItem<V>(t.cols, t.beta, t.sm_in, t.sm_rq, t.fc.y + static_cast<long long>(row) * t.cols,
                          t.out + static_cast<long long>(row) * t.cols, reinterpret_cast<float*>(smem));
        ++done;
    }

    // ---- leave; the last block out zeroes the counters for the next launch (every block has passed its waits by then) ----
    if (tid == 0)
    {
        if (__hip_atomic_fetch_add(t.sync + kTailExit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == static_cast<uint32_t>(G))
        {
            for (int w = 0; w < 2 * kTailWays; ++w) __hip_atomic_store(t.sync + w * kTailSlot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(t.sync + kTailExit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

} // namespace mi355x
