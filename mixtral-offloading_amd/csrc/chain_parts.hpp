// Chained launches: the work of several dependent launches placed in ONE grid, so that the later parts can request
// their weights while the earlier parts still run.  Blocks are ordered by role -- all blocks of the first role have
// lower block indices than those of the middle role, and those lower than the last role's -- and a block only ever
// waits for blocks of a lower index.  Workgroups are dispatched in index order, so whenever a waiting block is
// resident every block it waits for is resident or finished: the chain cannot deadlock whatever share of the chip the
// grid gets.  As a second line of defence every wait is bounded: after kChainSpinLimit polls the block gives up,
// records it in the chain's error word and carries on (with wrong data), so every wave always reaches its end.
//
// Hand-over: the producer writes its results with device-scope stores (written through its XCD's L2, which is not
// coherent with the other XCDs'), waits until they are acknowledged, and only then counts itself with a device-scope
// atomic; the consumer, once told to go, reads the results with device-scope loads.  No cache-wide write-back or
// invalidate is used.
//
// The words of a chain live in the workspace head, zero between launches, each on a 128-byte line of its own (device-
// scope operations on one line are served one after the other, and hundreds of pollers on the line the producers
// count on delayed both by microseconds): the count of first-role blocks done, of middle-role blocks done, of
// last-role blocks past their wait, an error word, and two sets of "go" words.  The producer whose count completes a
// role raises that role's go words; a waiting block polls ONE of them, chosen by its block index, so a line has a
// handful of pollers and nobody polls a line that is counted on.  The block of the last role that is the last to pass
// its wait clears everything: by then every wait of the launch is over.
#pragma once
#include "hqq_common.hpp"

namespace hqq {

enum { CHAIN_NONE = 0, CHAIN_FIRST = 1, CHAIN_MID = 2, CHAIN_LAST = 3 };
constexpr int kChainLine = 32; // ints per 128-byte line
constexpr int kChainGoFirst = 8, kChainGoMid = 16; // go words per hand-over
enum {
    CHAIN_FIRST_DONE = 0,
    CHAIN_MID_DONE = kChainLine,
    CHAIN_LAST_PASSED = 2 * kChainLine,
    CHAIN_ERROR = 3 * kChainLine,
    CHAIN_GO_FIRST = 4 * kChainLine,
    CHAIN_GO_MID = (4 + kChainGoFirst) * kChainLine,
    CHAIN_WORDS = (4 + kChainGoFirst + kChainGoMid) * kChainLine
};
constexpr int kChainSpinLimit = 1 << 19; // polls of about half a microsecond each: a quarter of a second, then give up

#ifdef HQQ_CHAIN_STAMPS
// timing build only: four time stamps per block at the start of the workspace (the tile counters, unused by chains)
__device__ __forceinline__ void chain_stamp(int *chain, int slot)
{
    if (threadIdx.x == 0) {
        unsigned long long *base = reinterpret_cast<unsigned long long *>(chain + CHAIN_WORDS - 16384);
        base[blockIdx.x * 4 + slot] = __builtin_amdgcn_s_memrealtime();
    }
}
#define CHAIN_STAMP(chain, slot) chain_stamp(chain, slot)
#else
#define CHAIN_STAMP(chain, slot)
#endif

// every thread of the block has stored its results at device scope: count the block once they are acknowledged, and
// raise the go words when this block completes the role (`blocks` of them)
__device__ __forceinline__ void chain_signal(int *chain, int count_at, int blocks, int go_at, int go_words)
{
    __builtin_amdgcn_s_waitcnt(0); // vmcnt(0) expcnt(0) lgkmcnt(0): every store of this thread is acknowledged
    __syncthreads();
    if (threadIdx.x == 0) {
        const int prev = __hip_atomic_fetch_add(chain + count_at, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == blocks - 1)
            for (int i = 0; i < go_words; ++i)
                __hip_atomic_store(chain + go_at + i * kChainLine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// the whole block waits for its go word: one lane polls, the other waves sleep at the barrier
__device__ __forceinline__ void chain_wait(int *chain, int go_at, int go_words)
{
    if (threadIdx.x == 0) {
        const int *word = chain + go_at + ((int)blockIdx.x % go_words) * kChainLine;
        int spins = 0;
        while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
            if (++spins > kChainSpinLimit) {
                __hip_atomic_store(chain + CHAIN_ERROR, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(8);
        }
    }
    __syncthreads();
}

// one thread of a block of the last role, after its wait: the last block to get here leaves every word at zero
__device__ __forceinline__ void chain_passed(int *chain, int blocks)
{
    const int prev = __hip_atomic_fetch_add(chain + CHAIN_LAST_PASSED, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (prev == blocks - 1) {
        __hip_atomic_store(chain + CHAIN_FIRST_DONE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(chain + CHAIN_MID_DONE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(chain + CHAIN_LAST_PASSED, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int i = 0; i < kChainGoFirst + kChainGoMid; ++i)
            __hip_atomic_store(chain + CHAIN_GO_FIRST + i * kChainLine, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// device-scope stores and loads of fp16 vectors (32- and 64-bit words)
__device__ __forceinline__ void chain_store(f16 *dst, f16x2 v)
{
    __hip_atomic_store(reinterpret_cast<uint32_t *>(dst), __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void chain_store(f16 *dst, f16x4 v)
{
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(dst), __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t chain_load4(const f16 *src)
{
    return __hip_atomic_load(reinterpret_cast<const uint32_t *>(src), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u32x4 chain_load16(const f16 *src)
{
    const unsigned long long *p = reinterpret_cast<const unsigned long long *>(src);
    const unsigned long long a = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long b = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return (u32x4){(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
}

} // namespace hqq
