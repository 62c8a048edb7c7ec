// Device-wide barrier for persistent launches (one workgroup per compute unit, all resident at once) and the
// device-scope loads and stores that carry data across it.
//
// What crosses workgroups is written with device-scope stores and read with device-scope loads, which is all
// the coherence the barrier needs -- no cache write-back or invalidate.  Two-level arrival counters (16
// workgroups per first-level counter, every counter on its own 256-byte line) and a generation word that the
// waiters poll; counters return to zero by themselves.  A waiter gives up after a bounded time and raises a
// failure flag that every other waiter sees, so the launch always drains; the host reports the flag as an error.
// Words of the sync buffer: [0] second-level counter, [64] generation, [128] failure flag, [(4 + g) * 64]
// first-level counter of group g.
#pragma once

#include "common.h"

namespace mq {

constexpr int kSyncLine = 64;   // uint32 words between counters
constexpr int kSyncGroup = 16;  // workgroups per first-level counter

#if defined(__HIPCC__)
__device__ __forceinline__ float ld_dev(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_dev(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Device-wide barrier.  Every thread's device-scope stores are acknowledged (vmcnt) before its workgroup is
// counted.  `ahead()` runs in every thread once that is so and before the wait: the place to request weights
// of the next phase, whose latency then overlaps the barrier's.  Returns false when the barrier was abandoned.
// kWaitStores = false: the caller has already waited for the stores of every wavefront that made any (a
// wavefront that only has loads in flight need not drain them here).
template <bool kWaitStores = true, typename Ahead>
__device__ __forceinline__ bool grid_barrier(uint32_t* sync, uint32_t& my_gen, int* ok, long long spin_ticks, Ahead ahead) {
    if (kWaitStores) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    ahead();
    if (threadIdx.x == 0) {
        uint32_t* top = sync;
        uint32_t* gen = sync + kSyncLine;
        uint32_t* fail = sync + 2 * kSyncLine;
        const uint32_t n_wg = gridDim.x;
        const uint32_t grp = blockIdx.x / kSyncGroup;
        const uint32_t n_grp = (n_wg + kSyncGroup - 1) / kSyncGroup;
        const uint32_t grp_size = (grp + 1) * kSyncGroup <= n_wg ? kSyncGroup : n_wg - grp * kSyncGroup;
        uint32_t* gc = sync + (4 + grp) * kSyncLine;
        bool released = false, good = true;
        if (__hip_atomic_fetch_add(gc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == grp_size - 1) {
            __hip_atomic_store(gc, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (__hip_atomic_fetch_add(top, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == n_grp - 1) {
                __hip_atomic_store(top, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // the two resets above are acknowledged before anybody is let go
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __hip_atomic_fetch_add(gen, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                released = true;
            }
        }
        if (!released) {
            const long long t0 = wall_clock64();
            while (ld_dev(gen) == my_gen) {
                if (ld_dev(fail) != 0u || wall_clock64() - t0 > spin_ticks) {
                    __hip_atomic_store(fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    good = false;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        *ok = good ? 1 : 0;
    }
    my_gen += 1;
    __syncthreads();
    return *ok != 0;
}
#endif

}  // namespace mq
