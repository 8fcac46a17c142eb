// Communication between the workgroups of one launch: device-coherent accesses and
// a grid-wide rendezvous for grids that are resident all at once.
//
// Data that workgroups of one launch hand to each other goes through relaxed
// agent-scope atomics: the L2 of an XCD is not coherent with the other seven, and
// the fences that would make ordinary accesses visible write back and invalidate
// a whole L2 per workgroup, which costs several times the streaming pass itself.
#pragma once

#include "ts_common.h"

namespace ts {

__device__ __forceinline__ float2 load_coherent(const float2* p) {
  const uint64_t v =
      __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_float2(__uint_as_float((uint32_t)v), __uint_as_float((uint32_t)(v >> 32)));
}
// Publishing goes through read-modify-write operations whose old value is waited
// for: the value comes back once the operation has been performed (a tenth of a
// microsecond), whereas the acknowledgement of a plain store or of an atomic
// without return value takes several microseconds.
__device__ __forceinline__ void await(uint64_t old) { asm volatile("" ::"v"(old)); }
__device__ __forceinline__ void await(uint32_t old) { asm volatile("" ::"v"(old)); }
__device__ __forceinline__ void store_coherent(float2* p, float x, float y) {
  const uint64_t v = (uint64_t)__float_as_uint(x) | ((uint64_t)__float_as_uint(y) << 32);
  await(__hip_atomic_exchange((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ uint2 load_coherent(const uint2* p) {
  const uint64_t v =
      __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_uint2((uint32_t)v, (uint32_t)(v >> 32));
}
__device__ __forceinline__ void store_coherent(uint2* p, uint32_t x, uint32_t y) {
  await(__hip_atomic_exchange((uint64_t*)p, (uint64_t)x | ((uint64_t)y << 32), __ATOMIC_RELAXED,
                              __HIP_MEMORY_SCOPE_AGENT));
}
// Old value of a coherent add / max; several can be summed up and waited for once.
__device__ __forceinline__ uint32_t fetch_add_coherent(uint32_t* p, uint32_t v) {
  return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t fetch_max_coherent(uint32_t* p, uint32_t v) {
  return __hip_atomic_fetch_max(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t load_coherent(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The workgroups of a grid that take part in its rendezvous.
struct GridTeam {
  uint32_t size;   // participating workgroups
  uint32_t index;  // this workgroup among them
};

// Rendezvous area, in 32-bit words: kSyncSlots + 1 slots, kSyncSlotWords apart so
// that the slots fall into different memory channels, the first kSyncLiveWords of
// each zero at launch.
//   slot 0:     [0] fault flag, [1 + r] groups that completed round r (r = 1, 2, ...)
//   slot 1 + i: [0] highest completed round, replica i, polled by the workgroups
//               with index % kSyncSlots == i
//               [1 + r] arrivals of round r in group i
constexpr int kSyncSlots = 64;
constexpr int kSyncSlotWords = 1024;
constexpr int kSyncLiveWords = 16;
constexpr int kSyncMaxRounds = kSyncLiveWords - 2;
constexpr size_t kSyncWords = (size_t)(kSyncSlots + 1) * kSyncSlotWords;

// One thread polls the replica of its workgroup until `round` is complete.
__device__ __forceinline__ void grid_poll(uint32_t* sync, uint32_t round, uint64_t ticks,
                                          uint32_t index) {
  const uint32_t* flag = &sync[(size_t)(index % kSyncSlots + 1) * kSyncSlotWords];
  const uint64_t t0 = wall_clock64();
  for (uint32_t polls = 1; load_coherent(flag) < round; ++polls) {
    if ((polls & 15u) == 0) {
      // Some workgroup has given up already: the launch is lost, do not wait again.
      if (load_coherent(&sync[0]) != 0u) break;
      if (wall_clock64() - t0 > ticks) {
        __hip_atomic_store(&sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
    // About 0.16 us between polls.  (Every rendezvous of the fused kernels comes after the
    // statistics exchange, when no workgroup of the request streams keys any more: the polls
    // compete with nothing.  The statistics are polled for more sparsely, see there.)
    __builtin_amdgcn_s_sleep(6);
  }
}

// Every participating workgroup arrives exactly once per round and waits for the round to
// complete (a workgroup that needs no more rounds arrives at the rest with grid_arrive_rest).  Each thread first waits for its
// outstanding memory operations (what it published has been performed by then);
// thread 0 then counts the workgroup in.  Arrivals are counted in two levels,
// about sqrt(workgroups) groups of as many members: read-modify-writes of one
// address are performed one after the other, some 10 ns each, so that a single
// counter would cost 5 us per round with 500 workgroups.  The workgroup that
// completes the count raises the round number in every replica, and the waiting
// ones poll the replica of their own index: hundreds of early workgroups polling
// one word would saturate the memory channel it lives in, which the workgroups
// still streaming need for 1/128 of their data.  The wait is bounded: if the
// round does not complete within `ticks` of the 100 MHz clock the fault word is
// set and the workgroup carries on, so the kernel always drains.
// `workgroups` of the grid take part, this one as number `index` among them.
__device__ __forceinline__ void grid_arrive(uint32_t* sync, uint32_t round, uint64_t ticks,
                                            uint32_t workgroups, uint32_t index) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x < 64) {  // the first wavefront; lane 0 counts, all lanes raise the flags
    uint32_t last = 0;
    if (threadIdx.x == 0) {
      uint32_t groups = 1;
      while (groups * groups < workgroups && groups < (uint32_t)kSyncSlots) ++groups;
      const uint32_t group = index % groups;
      const uint32_t members = workgroups / groups + (group < workgroups % groups ? 1u : 0u);
      if (__hip_atomic_fetch_add(&sync[(size_t)(group + 1) * kSyncSlotWords + 1 + round], 1u,
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == members)
        last = __hip_atomic_fetch_add(&sync[1 + round], 1u, __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT) + 1 == groups ? 1u : 0u;
    }
    last = __shfl(last, 0);
    if (last) {
      static_assert(kSyncSlots == 64, "one replica per lane");
      __hip_atomic_fetch_max(&sync[(size_t)(threadIdx.x + 1) * kSyncSlotWords], round,
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if (threadIdx.x == 0) {
      grid_poll(sync, round, ticks, index);
    }
  }
  __syncthreads();
}

// Arrival at the rounds first..last (at most 64 of them) at once, waiting for none: for a
// workgroup that is through with its rendezvous while others of the launch still need
// rounds.  Lane r counts the workgroup in for round first + r, so the rounds cost one chain of
// two dependent read-modify-writes instead of one chain each.  A later round may complete
// before an earlier one does (the counts of different rounds interleave); that is
// harmless, since whoever arrives at a later round has published all it ever will, and a
// waiter of round r may proceed as soon as any round >= r is complete.
__device__ __forceinline__ void grid_arrive_rest(uint32_t* sync, uint32_t first, uint32_t last,
                                                 uint32_t workgroups, uint32_t index) {
  if (first > last) return;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x < 64) {
    const uint32_t round = first + threadIdx.x;
    uint32_t completes = 0;
    if (round <= last) {
      uint32_t groups = 1;
      while (groups * groups < workgroups && groups < (uint32_t)kSyncSlots) ++groups;
      const uint32_t group = index % groups;
      const uint32_t members = workgroups / groups + (group < workgroups % groups ? 1u : 0u);
      if (__hip_atomic_fetch_add(&sync[(size_t)(group + 1) * kSyncSlotWords + 1 + round], 1u,
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == members)
        completes = __hip_atomic_fetch_add(&sync[1 + round], 1u, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT) + 1 == groups ? 1u : 0u;
    }
    const uint64_t which = __ballot(completes != 0u);
    if (which) {  // the highest round this workgroup completed, raised in every replica
      static_assert(kSyncSlots == 64, "one replica per lane");
      const uint32_t highest = first + 63u - (uint32_t)__builtin_clzll(which);
      __hip_atomic_fetch_max(&sync[(size_t)(threadIdx.x + 1) * kSyncSlotWords], highest,
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// One lane waits until the 64-bit word at `p` is no longer zero and returns it; 0 when
// the wait ran into its bound (the fault word is then set) or another one did.  SLEEP
// spaces the polls (in units of 64 clocks): a wait that begins while other workgroups
// still stream must not compete with them.
template <int SLEEP>
__device__ __forceinline__ uint64_t poll_nonzero(const uint64_t* p, uint32_t* sync, uint64_t ticks) {
  const uint64_t t0 = wall_clock64();
  for (uint32_t polls = 1;; ++polls) {
    const uint64_t v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (v != 0ull) return v;
    if ((polls & 15u) == 0) {
      if (load_coherent(&sync[0]) != 0u) return 0ull;
      if (wall_clock64() - t0 > ticks) {
        __hip_atomic_store(&sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return 0ull;
      }
    }
    __builtin_amdgcn_s_sleep(SLEEP);
  }
}

}  // namespace ts
