// A barrier across the workgroups of ONE launch, for kernels whose phases are separated by "every workgroup has finished the
// previous phase" instead of a kernel boundary (cq_layer.hip).  The launch is COOP_GRID workgroups that are all resident at
// once (one per CU; the host checks the CU count), so a workgroup that waits is waiting for workgroups that are running.
//
// Arrival is counted in a tree: COOP_GROUPS counters of COOP_GRID / COOP_GROUPS workgroups each, one top counter over the
// groups; the last arriver of the top counter writes the barrier's number into COOP_GROUPS release words, and a waiting wave
// polls the release word of its group only.  (256 arrivals on one word serialize, and waves polling a word that is being
// incremented slow the increments down: 15 us per barrier; the tree takes 1.4 us from the last arrival to the release.)
// Counters only ever grow, so nothing has to be reset between barriers or launches: the n-th arrival at a 16-way counter is
// the last of its barrier when n is a multiple of 16.
//
// No fence anywhere.  What one phase hands to the next goes out as device-scope (write-through) stores, the wave waits until
// they are acknowledged (vmcnt = 0) and only then arrives; readers of the next phase use plain loads, which is sound because
// every such buffer is written once and read only afterwards within a launch (no cache of another XCD can hold an older copy
// of a line: the caches were invalidated when the kernel started, and nothing has read the line since).
//
// Every wait is bounded: after COOP_TIMEOUT_TICKS of the 100 MHz clock a wave gives up, sets the error word and runs on
// without waiting again (its results are then garbage, but every workgroup still arrives everywhere and the kernel ends).
// The host must treat a set error word as a failed step and clear all sync words before the next cooperative launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

constexpr int COOP_GRID = 256;
constexpr int COOP_GROUPS = 16;
constexpr int COOP_LINE = 32;                                   // words per 128-byte line: every counter has a line to itself
constexpr int COOP_TOP = COOP_GROUPS * COOP_LINE;
constexpr int COOP_RELEASE = (COOP_GROUPS + 1) * COOP_LINE;
constexpr int COOP_ERR = (2 * COOP_GROUPS + 1) * COOP_LINE;
constexpr int COOP_SYNC_BYTES = (2 * COOP_GROUPS + 2) * COOP_LINE * 4;
constexpr uint64_t COOP_TIMEOUT_TICKS = 400000;                 // 4 ms

struct Coop {
    uint32_t *sync;
    uint32_t release0;      // the release words' value when the launch began
    uint32_t done;          // barriers this wave has arrived at
    bool dead;
    int block;
};

__device__ __forceinline__ uint32_t coop_ld(const uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ void coop_init(Coop &c, uint32_t *sync, int block) {
    c.sync = sync; c.done = 0; c.dead = false; c.block = block;
    c.release0 = coop_ld(sync + COOP_RELEASE + (block & (COOP_GROUPS - 1)) * COOP_LINE);      // read before this wave's first arrival
}

// One wave arrives (its stores of the phase are acknowledged: the caller has waited for vmcnt = 0).  The last of the
// workgroup's `nwaves` waves arrives for the workgroup.  lds_cnt: a zero-initialised word of LDS shared by the workgroup.
__device__ __forceinline__ void coop_arrive(Coop &c, uint32_t *lds_cnt, int nwaves, int lane) {
    c.done++;
    if (lane == 0) {
        const uint32_t old = __hip_atomic_fetch_add(lds_cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (old + 1 == c.done * (uint32_t)nwaves) {
            const uint32_t v = __hip_atomic_fetch_add(c.sync + (c.block & (COOP_GROUPS - 1)) * COOP_LINE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (((v + 1) & (COOP_GRID / COOP_GROUPS - 1)) == 0) {
                const uint32_t t = __hip_atomic_fetch_add(c.sync + COOP_TOP, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (((t + 1) & (COOP_GROUPS - 1)) == 0) {
#pragma unroll
                    for (int q = 0; q < COOP_GROUPS; q++)
                        __hip_atomic_store(c.sync + COOP_RELEASE + q * COOP_LINE, c.release0 + c.done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    }
}

// The wave waits until every workgroup has arrived at the barrier this wave arrived at last.
__device__ __forceinline__ void coop_wait(Coop &c) {
    if (!c.dead) {
        const uint32_t want = c.release0 + c.done;
        const uint32_t *p = c.sync + COOP_RELEASE + (c.block & (COOP_GROUPS - 1)) * COOP_LINE;
        const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
        while (__builtin_amdgcn_readfirstlane((int)coop_ld(p)) != (int)want) {
            if (__builtin_amdgcn_s_memrealtime() - t0 > COOP_TIMEOUT_TICKS) {
                c.dead = true;
                __hip_atomic_fetch_or(c.sync + COOP_ERR, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    asm volatile("" ::: "memory");        // nothing that reads the previous phase's results may move in front of the wait
}

}  // namespace
