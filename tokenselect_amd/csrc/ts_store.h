// The K/V store of a prefill chunk (tr.py:725-733, 332-336) as a device function: the
// store kernel runs it, and so do spare workgroups of the chunk's fingerprint launch.
#pragma once

#include "ts_common.h"

namespace ts {

// A workgroup copies blockDim / kChunkThreadsPerRow rows of the chunk (row r to pool slot
// loc[r]) and writes table[len + r] for them.  Every workgroup must read the same old
// length, and the new one must be there when the launch ends: the workgroups count
// themselves in the upper bits of the length word itself (a length stays below 2^21,
// the count below 2^10), everybody masks those bits off, and the workgroup that
// completes the count writes the new length.  No second launch, no other memory.
// Rows that would not fit the table are dropped; slots are clamped to the pool.
constexpr int kLenBits = 21;
constexpr int kLenMask = (1 << kLenBits) - 1;
constexpr int kChunkThreadsPerRow = 32;
constexpr int kChunkCountedWgs = 1023;  // more workgroups take the two-launch form

// wg: this workgroup among the cs.workgroups that store; threads: its size.
template <bool COUNTED>
__device__ __forceinline__ void store_chunk_rows(const ChunkStore& cs, int wg, int threads) {
  // Counted: the upper bits may already hold other workgroups' counts.
  const int len = COUNTED ? (__hip_atomic_load(cs.seq_len, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & kLenMask)
                          : *cs.seq_len;
  const int r = wg * (threads / kChunkThreadsPerRow) + (int)threadIdx.x / kChunkThreadsPerRow;
  const int t = threadIdx.x % kChunkThreadsPerRow;
  const int at = len + r;
  if (r < cs.rows && at >= 0 && at < cs.max_tokens) {
    int64_t slot = cs.loc[r];
    slot = slot < 0 ? 0 : (slot >= cs.pool_rows ? cs.pool_rows - 1 : slot);
    for (int i = t; i < cs.row_vec; i += kChunkThreadsPerRow) {
      cs.k_pool[(size_t)slot * cs.row_vec + i] = cs.k[(size_t)r * cs.row_vec + i];
      cs.v_pool[(size_t)slot * cs.row_vec + i] = cs.v[(size_t)r * cs.row_vec + i];
    }
    if (t == 0) cs.table[at] = (int32_t)slot;
  }
  if (COUNTED) {
    // A workgroup counts itself in when all its wavefronts have read the length, at its
    // end, where nobody waits for the answer; whoever completes the count knows that
    // every workgroup has read the old length, and writes the new one.
    __syncthreads();
    if (threadIdx.x == 0) {
      const int before = __hip_atomic_fetch_add(cs.seq_len, 1 << kLenBits, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
      if ((before >> kLenBits) + 1 == cs.workgroups)
        __hip_atomic_store(cs.seq_len, min(len + cs.rows, cs.max_tokens), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace ts
