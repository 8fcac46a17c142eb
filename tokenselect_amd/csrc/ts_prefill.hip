// Chunked prefill (patched_radix_attention_extend_forward_flashinfer, tr.py:703-775):
// the fingerprint of a chunk (mean of its rotated query rows, tr.py:380-392) and the
// causal attention of the chunk's rows over the selected KV slots (FlashInfer paged
// prefill, tr.py:759-771, page size 1, in-kernel Llama RoPE).
#include <math.h>

#include <type_traits>

#include "ts_common.h"
#include "ts_store.h"

namespace ts {

// ------------------------------------------------------------------ fingerprint
// Two workgroups per head (32 rotation pairs each), 1024 threads = 8 quads of pairs
// x 128 row groups, so that a chunk of 512 rows is one step of four independent rows
// per thread (the kernel is bound by the latency of its loads).  Row r
// is rotated with table row first_pos + r exactly like the rotation kernel (every
// product and sum rounded on its own, result rounded to bf16, tr.py:104-107); the
// bf16 values are summed in fp32, row group by row group in a fixed order, divided
// by the row count and rounded to bf16 (torch.mean on a bf16 tensor, tr.py:392).
constexpr int kFpRowGroups = 128;
constexpr int kFpInFlight = 4;  // rows per step of a row group
constexpr int kFpVec = 4;       // rotation pairs per thread
constexpr int kFpSplit = 2;     // workgroups per head

__global__ __launch_bounds__(1024) void fingerprint_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ qf, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int64_t table_rows, int first_pos, int rows, int heads,
    ZeroSet zero, ChunkStore cs) {
#pragma clang fp contract(off)
  constexpr int half = kHeadDim / 2;
  constexpr int kPairs = half / kFpSplit;   // rotation pairs of this workgroup
  constexpr int kLanes = kPairs / kFpVec;   // threads per row
  static_assert(kLanes * kFpRowGroups == 1024, "1024 threads per workgroup");
  const int h = blockIdx.x;
  const int first_pair = blockIdx.y * kPairs;
  const int i = first_pair + (threadIdx.x % kLanes) * kFpVec, rg = threadIdx.x / kLanes;
  // On the side: clear the words the selection kernel after this one counts into.
  {
    const int64_t gid = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 1024 + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * gridDim.y * 1024;
    clear_regions(zero, gid, step);
  }
  // Also on the side: the workgroups past the fingerprint's own store the chunk's K/V
  // rows (the caller's store of the chunk, which the selection after this launch must find
  // done, riding here instead of in a launch of its own).
  if ((int)blockIdx.y >= kFpSplit) {
    const int wg = ((int)blockIdx.y - kFpSplit) * (int)gridDim.x + (int)blockIdx.x;
    if (cs.k != nullptr && wg < cs.workgroups) store_chunk_rows<true>(cs, wg, 1024);
    return;
  }
  float lo_sum[kFpVec] = {0.f, 0.f, 0.f, 0.f}, hi_sum[kFpVec] = {0.f, 0.f, 0.f, 0.f};
  // Four rows per step: their loads are independent and go out together; the sums
  // are still taken in row order.
  for (int r0 = rg; r0 < rows; r0 += kFpInFlight * kFpRowGroups) {
    uint2 x1[kFpInFlight], x2[kFpInFlight];
    float4 c1[kFpInFlight], c2[kFpInFlight], s1[kFpInFlight], s2[kFpInFlight];
#pragma unroll
    for (int j = 0; j < kFpInFlight; ++j) {
      const int r = min(r0 + j * kFpRowGroups, rows - 1);
      int64_t pos = (int64_t)first_pos + r;
      pos = pos < table_rows ? pos : table_rows - 1;
      const float* c = cos_table + pos * kHeadDim;
      const float* s = sin_table + pos * kHeadDim;
      const size_t base = ((size_t)r * heads + h) * kHeadDim;
      x1[j] = *(const uint2*)(q + base + i);
      x2[j] = *(const uint2*)(q + base + i + half);
      c1[j] = *(const float4*)(c + i);
      c2[j] = *(const float4*)(c + i + half);
      s1[j] = *(const float4*)(s + i);
      s2[j] = *(const float4*)(s + i + half);
    }
#pragma unroll
    for (int j = 0; j < kFpInFlight; ++j) {
      if (r0 + j * kFpRowGroups < rows) {
        const float a1[kFpVec] = {bf16_to_f32((uint16_t)x1[j].x), bf16_to_f32((uint16_t)(x1[j].x >> 16)),
                                  bf16_to_f32((uint16_t)x1[j].y), bf16_to_f32((uint16_t)(x1[j].y >> 16))};
        const float a2[kFpVec] = {bf16_to_f32((uint16_t)x2[j].x), bf16_to_f32((uint16_t)(x2[j].x >> 16)),
                                  bf16_to_f32((uint16_t)x2[j].y), bf16_to_f32((uint16_t)(x2[j].y >> 16))};
        const float cc1[kFpVec] = {c1[j].x, c1[j].y, c1[j].z, c1[j].w};
        const float cc2[kFpVec] = {c2[j].x, c2[j].y, c2[j].z, c2[j].w};
        const float ss1[kFpVec] = {s1[j].x, s1[j].y, s1[j].z, s1[j].w};
        const float ss2[kFpVec] = {s2[j].x, s2[j].y, s2[j].z, s2[j].w};
#pragma unroll
        for (int e = 0; e < kFpVec; ++e) {
          const float lo = a1[e] * cc1[e] + (-a2[e]) * ss1[e];
          const float hi = a2[e] * cc2[e] + a1[e] * ss2[e];
          lo_sum[e] += bf16_to_f32(f32_to_bf16(lo));
          hi_sum[e] += bf16_to_f32(f32_to_bf16(hi));
        }
      }
    }
  }
  // Columns of this workgroup: its kPairs low halves, then its kPairs high halves.
  // The row groups are added in order, eight at a time and then the sixteen eights.
  __shared__ float part[kFpRowGroups][2 * kPairs];
  __shared__ float part8[kFpRowGroups / 8][2 * kPairs];
  const int col = i - first_pair;
#pragma unroll
  for (int e = 0; e < kFpVec; ++e) {
    part[rg][col + e] = lo_sum[e];
    part[rg][col + e + kPairs] = hi_sum[e];
  }
  __syncthreads();
  {
    const int c = threadIdx.x % (2 * kPairs), set = threadIdx.x / (2 * kPairs);
    float sum = 0.f;
#pragma unroll
    for (int g = 0; g < 8; ++g) sum += part[set * 8 + g][c];
    part8[set][c] = sum;
  }
  __syncthreads();
  if (threadIdx.x < 2 * kPairs) {
    float total = 0.f;
    for (int g = 0; g < kFpRowGroups / 8; ++g) total += part8[g][threadIdx.x];
    const int c = threadIdx.x;
    const int dim = c < kPairs ? first_pair + c : half + first_pair + (c - kPairs);
    qf[(size_t)h * kHeadDim + dim] = f32_to_bf16(total / (float)rows);
  }
}

// ------------------------------------------------------------ prefill attention
// Two launches.
//
// prefill_gather_kernel: the selected rows are gathered once per chunk into a
// contiguous staging area, K rotated to its index in the selected list (in fp32,
// rounded to bf16 like the queries) as kr[kvh][j][128] and V transposed as
// vt[kvh][128][S_pad], so that the attention kernel, whose 32 query tiles would
// otherwise each repeat the gather, the rotation and the transposition, only copies
// tiles.  Within every block of 32 keys a V^T row is stored in the order in which the
// attention kernel's matrix instructions want the keys (see kv_pos below).
//
// prefill_attn_kernel<G>: grid (KV heads, 16-row query tiles, quads of the G query
// heads of a KV head); 512 threads = four key groups of two wavefronts.  Key group g
// takes the 32-key tiles g, g + 4, g + 8, ...; its two wavefronts serve two query heads
// each (two 16 x 128 query blocks held in registers), so that every K and V^T operand
// read from LDS feeds two matrix instructions.  The four groups' (max, sum, acc) are
// merged through LDS at the end.
//
// Staging: a group's 128 threads bring the next tile of their group (8 KB of kr, 8 KB
// of vt) from global memory straight into LDS (global_load_lds_dwordx4: 16 bytes per
// lane, a wavefront fills 1 KB of consecutive LDS; no registers, no LDS store
// instructions) while the group computes on the tiles that arrived during the previous
// step; two LDS buffers per group, and two counters in LDS per group instead of a
// workgroup barrier per step (see the loop).  Rows are not padded in LDS;
// instead the 16-byte pieces of a row are permuted (XOR with row bits) so that the 16
// lanes the hardware serves together when a wavefront reads a matrix operand fall on
// distinct banks: which global piece a lane fetches is free, where it lands is not.
//
// A wavefront computes S^T = K Q^T with v_mfma_f32_16x16x32_bf16 (A = 16 keys x 32 dims
// from LDS, B = 16 rotated queries of one head, pre-multiplied by the softmax scale and
// log2 e), which leaves lane (query l%16, key group l/16) with base-2 logits of 8 keys of
// the tile.  The accumulator starts at minus the running maximum of the row, so the
// products come out already shifted; the running maximum is only raised when a logit
// exceeds it by more than 8 (the weights then stay below 2^8, harmless in fp32 sums
// and invisible after the final division), so the common path per logit is one
// maximum, one exp2 and half a conversion.  The 8 probabilities, rounded to bf16, are
// directly the B operand of O^T += V^T P^T (A = 16 dims x 32 keys from the V^T tile);
// a ninth product with an all-ones A operand accumulates the row sums.  fp32
// accumulation throughout.
//
// Where the time goes (512 rows over 2688 selected keys, 36.5 us): 4.6 us until the
// queries are rotated and the first tile is there, 2 us for the merge and the output, the
// rest in some 19 rounds of 2100 cycles per wavefront, of which the matrix unit of a SIMD
// is busy 1090 (its two wavefronts' 68 instructions of 16 cycles).  A round is some 250
// instructions, a wavefront issues one per four cycles at best, and every wait (for LDS
// data, for a matrix result, for the partner's counter) stalls the wavefront's whole
// stream: two wavefronts per SIMD cover each other only partly.  Four wavefronts per SIMD
// with one head each double the LDS reads and came out the same.
struct PrefillArgs {
  const uint16_t* q;  // [rows, H, 128] bf16, un-rotated
  const uint16_t* k_pool;
  const uint16_t* v_pool;
  uint32_t pool_rows;
  const int32_t* sel;      // [S] selected slots in attention order
  const int32_t* sel_len;  // device scalar S
  int max_sel_len;
  int s_pad;               // columns of a vt row: max_sel_len rounded up to kPfPadKeys
  int rows;
  int num_heads, num_kv_heads, rope_mode;
  float log2_theta, rope_rcp_scale, sm_scale, logit_cap;
  uint16_t* kr;   // [Hkv, s_pad, 128] bf16 rotated keys
  uint16_t* vt;   // [Hkv, 128, s_pad] bf16 transposed values, keys permuted within blocks of 32
  uint16_t* out;  // [rows, H, 128] bf16
};

typedef __attribute__((ext_vector_type(8))) __bf16 pf_bf16x8;
typedef __attribute__((ext_vector_type(4))) float pf_f32x4;
constexpr float kLog2e = 1.4426950408889634f;

constexpr int kPfKeys = 32;            // keys per tile: of the gather kernel and of the attention kernel
constexpr int kPfVRow = kPfKeys + 8;   // halfwords per V^T row in the gather kernel's LDS (80 B)
constexpr int kPfPadKeys = 64;         // the staging area holds whole multiples of this many keys
constexpr int kPfGroups = 4;           // key groups of an attention workgroup
constexpr int kPfTileBytes = kPfKeys * kHeadDim * 2;  // 8 KB: a K tile; a V^T tile is as large
constexpr int kPfBufBytes = 2 * kPfTileBytes;         // K tile, then V^T tile
constexpr size_t kPfLdsBytes = (size_t)kPfGroups * 2 * kPfBufBytes;  // 128 KB
constexpr int kPfHeads = 2;            // query heads per wavefront of the attention kernel
constexpr float kPfRaise = 8.0f;       // a row's maximum is raised when a logit exceeds it by this much

// Position of key kk (0..31 within its block) in a V^T row: the matrix instruction
// that made the logits left lane group g4 with keys 16 kb + 4 g4 + r (kb < 2, r < 4),
// and the next one wants those 8 as one 16-byte operand, in the order 4 kb + r.
__device__ __forceinline__ int kv_pos(int kk) { return 8 * ((kk >> 2) & 3) + 4 * (kk >> 4) + (kk & 3); }

// Grid (32-key tiles, KV heads).  Thread (key kk, chunk c) moves dims [8c, 8c+8) and
// [64+8c, +8) of key j = tile + kk.  Keys past S are written as zeros.
__global__ __launch_bounds__(256) void prefill_gather_kernel(PrefillArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t vt_lds[kHeadDim * kPfVRow];
  const int tid = threadIdx.x;
  const int kk = tid >> 3, c8 = tid & 7;
  const int kvh = blockIdx.y;
  const int j = blockIdx.x * kPfKeys + kk;
  // (the slot is asked for together with the length, not after it)
  uint32_t slot = (uint32_t)a.sel[min(j, a.max_sel_len - 1)];
  const int S = min(max(*a.sel_len, 0), a.max_sel_len);
  // Whole blocks of kPfPadKeys: the keys between S and the next multiple are written as
  // zeros too (their weights are zero, but 0 x garbage is not).
  if (blockIdx.x * kPfKeys >= (S + kPfPadKeys - 1) / kPfPadKeys * kPfPadKeys) return;
  const bool live = j < S;
  uint4 kraw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  uint4 vraw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  if (live) {
    slot = slot < a.pool_rows ? slot : a.pool_rows - 1;
    const size_t at = ((size_t)slot * a.num_kv_heads + kvh) * kHeadDim + 8 * c8;
    kraw[0] = *(const uint4*)(a.k_pool + at);
    kraw[1] = *(const uint4*)(a.k_pool + at + 64);
    vraw[0] = *(const uint4*)(a.v_pool + at);
    vraw[1] = *(const uint4*)(a.v_pool + at + 64);
  }
  const uint32_t klo[4] = {kraw[0].x, kraw[0].y, kraw[0].z, kraw[0].w};
  const uint32_t khi[4] = {kraw[1].x, kraw[1].y, kraw[1].z, kraw[1].w};
  float lo[8], hi[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    lo[2 * e] = bf16_lo(klo[e]);
    lo[2 * e + 1] = bf16_hi(klo[e]);
    hi[2 * e] = bf16_lo(khi[e]);
    hi[2 * e + 1] = bf16_hi(khi[e]);
  }
  if (a.rope_mode == TS_ROPE_LLAMA) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int pair = 8 * c8 + e;
      const float freq = a.rope_rcp_scale * exp2f(-(float)pair * (2.0f / kHeadDim) * a.log2_theta);
      float sn, cs;
      sincos_reduced((float)j * freq, sn, cs);
      const float l2 = lo[e] * cs - hi[e] * sn;
      hi[e] = hi[e] * cs + lo[e] * sn;
      lo[e] = l2;
    }
  }
  uint16_t* krow = a.kr + ((size_t)kvh * a.s_pad + j) * kHeadDim;
  *(uint4*)(krow + 8 * c8) = make_uint4(pack_bf16(lo[0], lo[1]), pack_bf16(lo[2], lo[3]),
                                        pack_bf16(lo[4], lo[5]), pack_bf16(lo[6], lo[7]));
  *(uint4*)(krow + 64 + 8 * c8) = make_uint4(pack_bf16(hi[0], hi[1]), pack_bf16(hi[2], hi[3]),
                                             pack_bf16(hi[4], hi[5]), pack_bf16(hi[6], hi[7]));
  // transpose the 32 x 128 V tile through LDS (key kk to column kv_pos(kk)), then write
  // 128 rows of 64 bytes
  const uint32_t vlo[4] = {vraw[0].x, vraw[0].y, vraw[0].z, vraw[0].w};
  const uint32_t vhi[4] = {vraw[1].x, vraw[1].y, vraw[1].z, vraw[1].w};
  const int col = kv_pos(kk);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    vt_lds[(8 * c8 + 2 * e) * kPfVRow + col] = (uint16_t)(vlo[e] & 0xffffu);
    vt_lds[(8 * c8 + 2 * e + 1) * kPfVRow + col] = (uint16_t)(vlo[e] >> 16);
    vt_lds[(64 + 8 * c8 + 2 * e) * kPfVRow + col] = (uint16_t)(vhi[e] & 0xffffu);
    vt_lds[(64 + 8 * c8 + 2 * e + 1) * kPfVRow + col] = (uint16_t)(vhi[e] >> 16);
  }
  __syncthreads();
  const int d = tid >> 1, half = tid & 1;
  uint16_t* vrow = a.vt + ((size_t)kvh * kHeadDim + d) * a.s_pad + blockIdx.x * kPfKeys + 16 * half;
  const uint4* src = (const uint4*)(vt_lds + d * kPfVRow + 16 * half);
  ((uint4*)vrow)[0] = src[0];
  ((uint4*)vrow)[1] = src[1];
}

typedef void __attribute__((address_space(3)))* pf_lds_ptr;

// 16 bytes per lane from global memory straight into LDS: lane l's piece lands at LDS
// byte address lds_dst + 16 l (lds_dst the same for the whole wavefront, passed in M0).
// Written as assembly and not through the compiler's builtin on purpose: the compiler
// makes every later LDS read wait for all such loads (it cannot tell that they fill the
// other buffer), which serialises exactly what is meant to overlap.  The waits are
// explicit instead: s_waitcnt vmcnt(0) before the barrier that hands a buffer over.
// The source is base (the same for the whole wavefront) + offset (per lane).  Four pieces per
// lane with one write of M0: the instruction's offset field moves both addresses, so piece
// i lands 1 KB after piece i - 1, and its source offset is passed 1024 i too small.
// A wavefront issues one instruction per four cycles at best, whatever its kind, and
// the loop around these loads is bound by exactly that: every scalar instruction counts.
__device__ __forceinline__ void load_to_lds16(const void* base, const uint32_t (&offset)[4], uint32_t lds_dst) {
  uint32_t saved_m0;  // M0 is the compiler's; it gets it back
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %2, %6\n\t"
      "global_load_lds_dwordx4 %3, %6 offset:1024\n\t"
      "global_load_lds_dwordx4 %4, %6 offset:2048\n\t"
      "global_load_lds_dwordx4 %5, %6 offset:3072\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0)
      : "s"(lds_dst), "v"(offset[0]), "v"(offset[1]), "v"(offset[2]), "v"(offset[3]), "s"(base)
      : "memory");
}

// One lane adds 1 to a counter in LDS.  LDS instructions of a wavefront are carried out in
// order, so the reads before it have been served when the addition is.
__device__ __forceinline__ void lds_count(uint32_t lds_at_vgpr, uint32_t one_vgpr) {
  uint64_t saved_exec;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 1\n\tds_add_u32 %1, %2\n\ts_mov_b64 exec, %0"
               : "=&s"(saved_exec)
               : "v"(lds_at_vgpr), "v"(one_vgpr)
               : "memory");
}

// Largest of three, without the NaN-quieting copies fmaxf brings along.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float d;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}

// Two wavefronts per SIMD by construction (8 per workgroup, one workgroup per CU): saying
// so lets the compiler use 256 registers.
template <int G, bool CAP>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void prefill_attn_kernel(
    PrefillArgs a) {
  constexpr int HEADS = kPfHeads;        // query heads per wavefront
  constexpr int kWaves = 4 / HEADS;      // wavefronts of a key group
  constexpr int kBlocks = 8 / kWaves;    // 1 KB blocks of a K tile (and of a V^T tile) a wavefront brings in
  static_assert(HEADS == 2 && kBlocks == 4, "the staging loads come four per wavefront");
  // Dynamic LDS: per key group two buffers, each a K tile [32 keys][256 B] followed by a
  // V^T tile [128 dims][64 B]; the merge of the groups at the end reuses the space.
  extern __shared__ __attribute__((aligned(16))) uint16_t pf_lds[];
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int group = wave / kWaves;  // which of the four tile streams this wavefront follows
  const int hp = wave % kWaves;     // which HEADS of the quad's heads it serves
  const int qc = lane & 15, g4 = lane >> 4;  // query column / key group of the matrix layouts
  // The KV head is the fastest-moving workgroup index: consecutive workgroups go to
  // consecutive XCDs, so with eight KV heads each XCD's L2 holds the keys and values of one
  // head (1.4 MB of 11 MB) and every query tile of that head finds them there.  The last
  // query tiles, which see the most keys, start first.
  const int kvh = blockIdx.x;
  const int q_row0 = (int)(gridDim.y - 1 - blockIdx.y) * 16;
  const int H = a.num_heads;
  char* const group_lds = (char*)pf_lds + group * (2 * kPfBufBytes);
  const uint32_t group_lds_at = (uint32_t)(uintptr_t)(pf_lds_ptr)pf_lds + (uint32_t)(group * (2 * kPfBufBytes));

  // ---- staging role.  K tile: wavefront hp of the group fills the 1 KB blocks kBlocks hp + i
  // (i < kBlocks; a block is 4 keys), lane l the piece (key l/16 of the block, slot l%16), which
  // holds the dims [8 c, 8 c + 8) with c = slot ^ (key & 15).  V^T tile: blocks of 16 dims,
  // lane l the piece (dim l/4 of the block, slot l%4) = keys [8 c, +8) of the tile in vt's
  // order, c = slot ^ ((dim / 4) & 3).
  uint32_t k_src[kBlocks], v_src[kBlocks];
  {
    const int key_in_block = lane >> 4, slot = lane & 15;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int key = 4 * (kBlocks * hp + i) + key_in_block;
      k_src[i] = (uint32_t)(key * kHeadDim + 8 * (slot ^ (key & 15))) * 2u - (uint32_t)(i * 1024);
    }
    const int dim_in_block = lane >> 2, vslot = lane & 3;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int dim = 16 * (kBlocks * hp + i) + dim_in_block;
      v_src[i] = (uint32_t)(dim * a.s_pad + 8 * (vslot ^ ((dim >> 2) & 3))) * 2u - (uint32_t)(i * 1024);
    }
  }
  const char* const k_base = (const char*)(a.kr + (size_t)kvh * a.s_pad * kHeadDim);
  const char* const v_base = (const char*)(a.vt + (size_t)kvh * kHeadDim * a.s_pad);
  // Tile t of this group holds the keys [(t kPfGroups + group) kPfKeys, + kPfKeys); K tile t
  // lives in K buffer t % 2, V^T tile t in V buffer t % 2.
  auto request_k = [&](int t) __attribute__((always_inline)) {
    // past the end: a harmless repeat of the last tile
    const int tile = min((t * kPfGroups + group) * kPfKeys, a.s_pad - kPfKeys);
    const uint32_t dst = group_lds_at + (uint32_t)((t & 1) * kPfBufBytes + (kBlocks * hp) * 1024);
    load_to_lds16(k_base + (size_t)tile * (kHeadDim * 2), k_src, dst);
  };
  auto request_v = [&](int t) __attribute__((always_inline)) {
    const int tile = min((t * kPfGroups + group) * kPfKeys, a.s_pad - kPfKeys);
    const uint32_t dst = group_lds_at + (uint32_t)((t & 1) * kPfBufBytes + kPfTileBytes + (kBlocks * hp) * 1024);
    load_to_lds16(v_base + (size_t)tile * 2, v_src, dst);
  };
  request_k(0);  // on its way while the queries are prepared

  const int m = a.rows;
  int head[HEADS];
  bool head_active[HEADS];
#pragma unroll
  for (int rb = 0; rb < HEADS; ++rb) {
    const int head_in_group = blockIdx.z * 4 + HEADS * hp + rb;
    head_active[rb] = head_in_group < G;
    head[rb] = kvh * G + (head_active[rb] ? head_in_group : 0);
  }
  // The queries' loads do not wait for the selection's length.
  const int q_row = min(q_row0 + qc, m - 1);
  uint4 q_raw[HEADS][4];
#pragma unroll
  for (int rb = 0; rb < HEADS; ++rb) {
    const uint16_t* qrow = a.q + ((size_t)q_row * H + head[rb]) * kHeadDim;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) q_raw[rb][ks] = *(const uint4*)(qrow + 32 * ks + 8 * g4);
  }
  const int S = min(max(*a.sel_len, 0), a.max_sel_len);
  const int shift = S - m;  // query row i sits at position shift + i and sees keys <= that
  const bool rope = a.rope_mode == TS_ROPE_LLAMA;
  const bool wave_active = head_active[0];
  if (S <= 0) {
    // No keys (a selection that reported a fault): the rows attend to nothing and the
    // output is defined as zero.  (With fewer keys than rows, 0 < S < m, the rows whose
    // position S - m + i is negative see no key either: every tile is masked for them,
    // their sums stay zero and so does their output; the others attend as usual.)
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb)
      if (head_active[rb])
        for (int i = lane; i < 16 * (kHeadDim / 8); i += 64) {
          const int row = q_row0 + i / (kHeadDim / 8);
          if (row < m)
            *(uint4*)(a.out + ((size_t)row * H + head[rb]) * kHeadDim + 8 * (i % (kHeadDim / 8))) =
                make_uint4(0u, 0u, 0u, 0u);
        }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the tile on its way lands before the LDS is given up
    return;
  }

  // ---- queries: B operand, lane (qc, g4) holds dims [32 ks + 8 g4, +8) of row q_row0 + qc
  // of each of its two heads, rotated to position shift + row (partner dims d and d + 64 are
  // k-steps ks and ks + 2; the angles are the same for both heads).
  pf_bf16x8 qb[HEADS][4];
  {
    float x[HEADS][4][8];
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const uint4 w = q_raw[rb][ks];
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[rb][ks][2 * e] = bf16_lo(ww[e]);
          x[rb][ks][2 * e + 1] = bf16_hi(ww[e]);
        }
      }
    }
    if (rope) {
      const float pos = (float)(shift + q_row);
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int pair = 32 * ks + 8 * g4 + e;
          const float freq = a.rope_rcp_scale * exp2f(-(float)pair * (2.0f / kHeadDim) * a.log2_theta);
          float sn, cs;
          sincos_reduced(pos * freq, sn, cs);
#pragma unroll
          for (int rb = 0; rb < HEADS; ++rb) {
            const float lo = x[rb][ks][e], hi = x[rb][ks + 2][e];
            x[rb][ks][e] = lo * cs - hi * sn;
            x[rb][ks + 2][e] = hi * cs + lo * sn;
          }
        }
    }
    // Without a soft cap the softmax scale and log2(e) go into the query, so that the
    // products come out as base-2 logits and every key costs one exp2 and no multiply.
    const float qs = CAP ? 1.0f : a.sm_scale * kLog2e;
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[rb][ks][e] *= qs;
        const uint4 w = make_uint4(pack_bf16(x[rb][ks][0], x[rb][ks][1]), pack_bf16(x[rb][ks][2], x[rb][ks][3]),
                                   pack_bf16(x[rb][ks][4], x[rb][ks][5]), pack_bf16(x[rb][ks][6], x[rb][ks][7]));
        qb[rb][ks] = __builtin_bit_cast(pf_bf16x8, w);
      }
  }

  // ---- reading role: where this lane's operands sit in a buffer.  K operand (kb, ks): key
  // 16 kb + qc, dims [32 ks + 8 g4, +8) = piece 4 ks + g4, in slot (4 ks + g4) ^ qc.  V^T
  // operand db: dim 16 db + qc, piece g4, in slot g4 ^ ((qc / 4) & 3).
  uint32_t k_at[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) k_at[ks] = (uint32_t)(qc * (kHeadDim * 2) + 16 * ((4 * ks + g4) ^ qc));
  const uint32_t v_at = (uint32_t)(kPfTileBytes + qc * (kPfKeys * 2) + 16 * (g4 ^ ((qc >> 2) & 3)));

  // ---- main loop over the tiles any row of this query tile can see
  const int last_visible = min(S - 1, shift + min(q_row0 + 15, m - 1));
  const int my_limit = shift + q_row;  // last key this lane's query sees
  // tiles of this group that hold a visible key
  const int n_tiles = last_visible >= group * kPfKeys
                          ? (last_visible - group * kPfKeys) / (kPfGroups * kPfKeys) + 1
                          : 0;
  // Running maximum of each head's row: m_run (kNegBig: none yet), minus that as the
  // four-register start value of the logits' accumulators (0 while there is none), and the
  // excess over it that makes the row move (-inf while there is none: any finite logit does).
  float m_run[HEADS], raise_at[HEADS];
  pf_f32x4 minus_m[HEADS];
  pf_f32x4 o[HEADS][8], row_sum[HEADS];
#pragma unroll
  for (int rb = 0; rb < HEADS; ++rb) {
    m_run[rb] = kNegBig;
    raise_at[rb] = -INFINITY;
    minus_m[rb] = pf_f32x4{0.f, 0.f, 0.f, 0.f};
    row_sum[rb] = pf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int db = 0; db < 8; ++db) o[rb][db] = pf_f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const pf_bf16x8 ones = __builtin_bit_cast(pf_bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));

  // The work on a tile comes in three parts, and the loop below is a software pipeline
  // over them, because a wavefront issues in order and the matrix unit and the vector
  // ALU only run side by side when their instructions alternate in one stream (two
  // wavefronts of a SIMD, each doing first one kind and then the other, were measured to
  // overlap in 15 % of the matrix cycles):
  //   logits(t):  S^T = K_t Q^T for both heads (16 matrix instructions), shifted by the
  //               running maximum through the accumulator's start value;
  //   settle(t):  the causal mask on the diagonal, the largest logit of a row, and, when
  //               a row outgrew its maximum by kPfRaise, the move to a new one (vector);
  //   output(t):  P = exp2 (vector, 16 exp2), O^T += V_t^T P^T and the row sums (18 matrix).
  // Iteration t runs logits(t + 1) with the exp2 of tile t in between, then output(t),
  // then settle(t + 1).
  pf_f32x4 s_cur[HEADS][2];  // logits of the tile whose output comes next: [head][key block]

  auto logits = [&](int t, pf_f32x4 (&s)[HEADS][2]) __attribute__((always_inline)) {
    const char* const base = group_lds + (t & 1) * kPfBufBytes;
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb) {
      s[rb][0] = CAP ? pf_f32x4{0.f, 0.f, 0.f, 0.f} : minus_m[rb];
      s[rb][1] = s[rb][0];
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const uint4 kw = *(const uint4*)(base + kb * (16 * kHeadDim * 2) + k_at[ks]);
#pragma unroll
        for (int rb = 0; rb < HEADS; ++rb)
          s[rb][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, kw), qb[rb][ks],
                                                             s[rb][kb], 0, 0, 0);
      }
  };

  auto settle = [&](int t, pf_f32x4 (&s)[HEADS][2]) __attribute__((always_inline)) {
    const int tile = (t * kPfGroups + group) * kPfKeys;
    // Only the tiles on the diagonal hold keys that some query of the tile must not see.
    const bool diagonal = tile + kPfKeys - 1 > shift + q_row0;
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb) {
      if (CAP) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            s[rb][kb][r] = a.logit_cap * tanhf(s[rb][kb][r] * a.sm_scale / a.logit_cap) * kLog2e + minus_m[rb][0];
      }
      if (diagonal) {
        // Masked logits are -inf: exp2 makes them 0 without a branch.  (The tile's
        // number passes through an empty asm so that the comparisons stay in here: the
        // compiler otherwise computes all of them before the branch, on every tile.)
        int tile_here = tile;
        asm volatile("" : "+s"(tile_here));
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (tile_here + 16 * kb + 4 * g4 + r > my_limit) s[rb][kb][r] = -INFINITY;
      }
      float mx = max3(s[rb][0][0], s[rb][0][1], s[rb][0][2]);
      mx = max3(mx, s[rb][0][3], s[rb][1][0]);
      mx = max3(mx, s[rb][1][1], s[rb][1][2]);
      mx = fmaxf(mx, s[rb][1][3]);
      if (__ballot(mx > raise_at[rb]) != 0ull) {
        // Some row of this head has no maximum yet, or outgrew it: agree on the row's
        // maximum over the four key groups of lanes and move to it.
        const bool unset = m_run[rb] == kNegBig;
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const bool take = unset ? mx > -INFINITY : mx > kPfRaise;
        const float delta = take ? mx : 0.f;
        // (a row without a maximum has only zeros in its accumulators)
        const float scale = unset ? 1.0f : __builtin_amdgcn_exp2f(-delta);
        if (take) {
          m_run[rb] = delta - minus_m[rb][0];
          raise_at[rb] = kPfRaise;
          const float nm = -m_run[rb];
          minus_m[rb] = pf_f32x4{nm, nm, nm, nm};
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 4; ++r) s[rb][kb][r] -= delta;
#pragma unroll
        for (int db = 0; db < 8; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[rb][db][r] *= scale;
#pragma unroll
        for (int r = 0; r < 4; ++r) row_sum[rb][r] *= scale;
      }
    }
  };

  // One iteration of the pipeline: NEXT = there is a tile t + 1.
  auto iteration = [&](int t, auto next) __attribute__((always_inline)) {
    constexpr bool NEXT = decltype(next)::value;
    const char* const vbase = group_lds + (t & 1) * kPfBufBytes;
    pf_f32x4 s_next[HEADS][2];
    // The V^T operands are asked for first: they arrive under the logits' products.
    uint4 vw[8];
#pragma unroll
    for (int db = 0; db < 8; ++db) vw[db] = *(const uint4*)(vbase + db * (16 * kPfKeys * 2) + v_at);
    if (NEXT) logits(t + 1, s_next);
    pf_bf16x8 pb[HEADS];
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb) {
      float p[2][4];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) p[kb][r] = __builtin_amdgcn_exp2f(s_cur[rb][kb][r]);
      const uint4 pw = make_uint4(pack_bf16(p[0][0], p[0][1]), pack_bf16(p[0][2], p[0][3]),
                                  pack_bf16(p[1][0], p[1][1]), pack_bf16(p[1][2], p[1][3]));
      pb[rb] = __builtin_bit_cast(pf_bf16x8, pw);
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) {
#pragma unroll
      for (int rb = 0; rb < HEADS; ++rb)
        o[rb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, vw[db]), pb[rb],
                                                           o[rb][db], 0, 0, 0);
    }
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb)
      row_sum[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[rb], row_sum[rb], 0, 0, 0);
    if (NEXT) {
      settle(t + 1, s_next);
#pragma unroll
      for (int rb = 0; rb < HEADS; ++rb) {
        s_cur[rb][0] = s_next[rb][0];
        s_cur[rb][1] = s_next[rb][1];
      }
    }
  };

  // The wavefronts of a key group keep in step through two counters in LDS and no
  // barrier, so that the four groups drift apart.  landed = requests that have arrived
  // (after each round of requests a wavefront waits for its own pieces and counts once),
  // done = rounds of reading a wavefront has finished.  Round -1 brings K tile 0 and reads
  // nothing; round t >= 0 is iteration t: it needs K tile t + 1 and V tile t, requested in
  // round t - 1, and requests K tile t + 2 and V tile t + 1 into the buffers that round
  // t - 1 read (K tile t, V tile t - 1): so it starts when landed >= kWaves (t + 2) and
  // done >= kWaves (t + 1).  Neither wait can last: a partner is at most one round behind.
  // The waits are bounded all the same, so that a mistake here would show as a wrong
  // result and not as a hang.
  __shared__ __attribute__((aligned(8))) uint32_t pf_sync[kPfGroups][2];
  if (threadIdx.x < 2 * kPfGroups) (&pf_sync[0][0])[threadIdx.x] = 0u;
  __syncthreads();
  const uint64_t* const both = (const uint64_t*)&pf_sync[group][0];  // one read for the two
  const uint32_t landed_at = (uint32_t)(uintptr_t)(pf_lds_ptr)&pf_sync[group][0], done_at = landed_at + 4u;
  const uint32_t one = 1u;
  auto await = [&](uint32_t need_landed, uint32_t need_done) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_count(landed_at, one);
    for (int spin = 0; spin < (1 << 20); ++spin) {
      const uint64_t counters = __hip_atomic_load(both, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
      if ((uint32_t)counters >= need_landed && (uint32_t)(counters >> 32) >= need_done) break;
      __builtin_amdgcn_s_sleep(1);
    }
  };
  auto finish_round = [&]() __attribute__((always_inline)) {
    lds_count(done_at, one);
  };
  if (n_tiles > 0) {
    await((uint32_t)kWaves, 0u);
    if (1 < n_tiles) request_k(1);
    request_v(0);
    if (wave_active) {
      logits(0, s_cur);
      settle(0, s_cur);
    }
    finish_round();
    for (int t = 0; t + 1 < n_tiles; ++t) {
      await((uint32_t)(kWaves * (t + 2)), (uint32_t)(kWaves * (t + 1)));
      if (t + 2 < n_tiles) request_k(t + 2);
      request_v(t + 1);
      if (wave_active) iteration(t, std::true_type{});
      finish_round();
    }
    // the last tile: nothing follows it
    await((uint32_t)(kWaves * (n_tiles + 1)), (uint32_t)(kWaves * n_tiles));
    if (wave_active) iteration(n_tiles - 1, std::false_type{});
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- merge of the four key groups (the barrier that ended the last step also freed
  // the tiles' space): groups 1..3 hand their partial results to group 0 (same heads,
  // same lane), per head 9 vectors of four floats per lane: 8 of acc and (max, sum).
  constexpr int kVecs = 9 * HEADS;
  pf_f32x4* const merge = (pf_f32x4*)pf_lds;  // [(group - 1) * kWaves + hp][kVecs][64 lanes]
  static_assert(3 * kWaves * kVecs * 64 * 16 <= kPfLdsBytes, "the merge area fits the tiles");
  if (group != 0) {
    pf_f32x4* const mine = merge + ((group - 1) * kWaves + hp) * (kVecs * 64) + lane;
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb) {
#pragma unroll
      for (int db = 0; db < 8; ++db) mine[(9 * rb + db) * 64] = o[rb][db];
      mine[(9 * rb + 8) * 64] = pf_f32x4{m_run[rb], row_sum[rb][0], 0.f, 0.f};
    }
  }
  __syncthreads();
  if (group != 0 || !wave_active) return;
  float l_run[HEADS];
#pragma unroll
  for (int rb = 0; rb < HEADS; ++rb) l_run[rb] = row_sum[rb][0];
#pragma unroll
  for (int g = 1; g < kPfGroups; ++g) {
    const pf_f32x4* const other = merge + ((g - 1) * kWaves + hp) * (kVecs * 64) + lane;
#pragma unroll
    for (int rb = 0; rb < HEADS; ++rb) {
      const pf_f32x4 ml = other[(9 * rb + 8) * 64];
      const float m_new = fmaxf(m_run[rb], ml[0]);
      const float e0 = __builtin_amdgcn_exp2f(m_run[rb] - m_new), e1 = __builtin_amdgcn_exp2f(ml[0] - m_new);
      m_run[rb] = m_new;
      l_run[rb] = l_run[rb] * e0 + ml[1] * e1;
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        const pf_f32x4 od = other[(9 * rb + db) * 64];
#pragma unroll
        for (int r = 0; r < 4; ++r) o[rb][db][r] = o[rb][db][r] * e0 + od[r] * e1;
      }
    }
  }

  // o[rb][db][r] = O[query qc][dim 16 db + 4 g4 + r] of head rb; the row sum is complete in every lane.
  if (q_row0 + qc >= m) return;
#pragma unroll
  for (int rb = 0; rb < HEADS; ++rb) {
    if (!head_active[rb]) continue;
    const float inv = l_run[rb] > 0.f ? 1.0f / l_run[rb] : 0.f;
    uint16_t* orow = a.out + ((size_t)(q_row0 + qc) * H + head[rb]) * kHeadDim;
#pragma unroll
    for (int db = 0; db < 8; ++db)
      *(uint2*)(orow + 16 * db + 4 * g4) = make_uint2(pack_bf16(o[rb][db][0] * inv, o[rb][db][1] * inv),
                                                      pack_bf16(o[rb][db][2] * inv, o[rb][db][3] * inv));
  }
}

int launch_fingerprint(const ts_config* cfg, const void* q, int32_t rows, const float* cos_table,
                       const float* sin_table, int64_t table_rows, void* qf, const ZeroSet& zero,
                       hipStream_t stream, const ChunkStore* store) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(!zero.overflow, TS_EINVAL, "internal: more than %d regions to clear in one launch", kZeroRegions);
  TS_REQUIRE(q && cos_table && sin_table && qf, TS_EINVAL, "ts_fingerprint: NULL tensor argument");
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(cos_table, 16, "cos_table");
  TS_REQUIRE_ALIGNED(sin_table, 16, "sin_table");
  TS_REQUIRE(rows >= 1, TS_EINVAL, "ts_fingerprint: rows %d < 1", rows);
  TS_REQUIRE(table_rows >= (int64_t)cfg->n_local + rows, TS_EINVAL,
             "ts_fingerprint: cos/sin tables have %lld rows, need n_local + rows = %lld",
             (long long)table_rows, (long long)cfg->n_local + rows);
  ChunkStore cs{};
  unsigned grid_y = kFpSplit;
  if (store) {  // rows of 32 threads: 32 rows per workgroup of 1024
    cs = *store;
    cs.workgroups = (int)ceil_div(cs.rows, 1024 / kChunkThreadsPerRow);
    TS_REQUIRE(cs.workgroups <= kChunkCountedWgs && cs.max_tokens <= kLenMask, TS_EINVAL,
               "internal: a chunk store of %d rows does not ride in the fingerprint launch", cs.rows);
    grid_y += (unsigned)ceil_div(cs.workgroups, cfg->num_heads);
  }
  hipLaunchKernelGGL(fingerprint_kernel, dim3((unsigned)cfg->num_heads, grid_y), dim3(1024), 0, stream,
                     (const uint16_t*)q, (uint16_t*)qf, cos_table, sin_table, table_rows,
                     cfg->n_local, rows, cfg->num_heads, zero, cs);
  return check_launch("fingerprint_kernel");
}

static int prefill_s_pad(int max_sel_len) { return (int)ceil_div(max_sel_len, kPfPadKeys) * kPfPadKeys; }

}  // namespace ts

using namespace ts;

extern "C" {

int ts_fingerprint(const ts_config* cfg, const void* q, int32_t rows, const float* cos_table,
                   const float* sin_table, int64_t table_rows, void* qf, ts_stream_t stream) {
  return launch_fingerprint(cfg, q, rows, cos_table, sin_table, table_rows, qf, ZeroSet{},
                            (hipStream_t)stream);
}

size_t ts_prefill_attn_workspace_bytes(const ts_config* cfg, int32_t max_sel_len) {
  if (validate_config(cfg) != TS_OK || max_sel_len < 1) return 0;
  return 2 * align_up((size_t)cfg->num_kv_heads * prefill_s_pad(max_sel_len) * kHeadDim * 2, 256);
}

int ts_sparse_prefill_attn(const ts_config* cfg, const void* q, int32_t rows, const void* k_pool,
                           const void* v_pool, int64_t pool_rows, const int32_t* sel,
                           const int32_t* sel_len, int32_t max_sel_len, void* out, void* workspace,
                           size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(q && k_pool && v_pool && sel && sel_len && out, TS_EINVAL,
             "ts_sparse_prefill_attn: NULL tensor argument");
  TS_REQUIRE(rows >= 1 && rows <= 65535 * 16, TS_EINVAL, "rows %d out of range", rows);
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const size_t need = ts_prefill_attn_workspace_bytes(cfg, max_sel_len);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= need, TS_EWORKSPACE,
             "ts_sparse_prefill_attn: workspace %zu bytes < required %zu", workspace_bytes, need);
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_REQUIRE_ALIGNED(out, 16, "out");
  PrefillArgs a;
  a.q = (const uint16_t*)q;
  a.k_pool = (const uint16_t*)k_pool;
  a.v_pool = (const uint16_t*)v_pool;
  a.pool_rows = (uint32_t)pool_rows;
  a.sel = sel;
  a.sel_len = sel_len;
  a.max_sel_len = max_sel_len;
  a.s_pad = prefill_s_pad(max_sel_len);
  a.rows = rows;
  a.num_heads = cfg->num_heads;
  a.num_kv_heads = cfg->num_kv_heads;
  a.rope_mode = cfg->rope_mode;
  a.log2_theta = cfg->rope_mode == TS_ROPE_LLAMA ? (float)log2((double)cfg->rope_theta) : 0.f;
  a.rope_rcp_scale = cfg->rope_mode == TS_ROPE_LLAMA ? 1.0f / cfg->rope_scale : 1.0f;
  a.sm_scale = cfg->sm_scale;
  a.logit_cap = cfg->logit_cap;
  a.kr = (uint16_t*)workspace;
  a.vt = (uint16_t*)((char*)workspace + need / 2);
  a.out = (uint16_t*)out;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(prefill_gather_kernel, dim3((unsigned)(a.s_pad / kPfKeys), (unsigned)cfg->num_kv_heads),
                     dim3(256), 0, st, a);
  TS_TRY(check_launch("prefill_gather_kernel"));
  const int group = cfg->num_heads / cfg->num_kv_heads;
  const dim3 grid((unsigned)cfg->num_kv_heads, (unsigned)ceil_div(rows, 16),
                  (unsigned)ceil_div(group, 4));
  const bool cap = cfg->logit_cap > 0.f;
#define TS_PF_LAUNCH(G_, C_)                                                                  \
  {                                                                                           \
    static const hipError_t lds_ok = hipFuncSetAttribute(                                     \
        (const void*)prefill_attn_kernel<G_, C_>, hipFuncAttributeMaxDynamicSharedMemorySize, \
        (int)kPfLdsBytes);                                                                    \
    if (lds_ok != hipSuccess) return fail(TS_EHIP, "prefill attention: %zu bytes of LDS refused", kPfLdsBytes); \
    hipLaunchKernelGGL((prefill_attn_kernel<G_, C_>), grid, dim3(512), kPfLdsBytes, st, a); \
  }
#define TS_PF_CASE(G_)               \
  case G_:                           \
    if (cap) TS_PF_LAUNCH(G_, true)  \
    else TS_PF_LAUNCH(G_, false)     \
    break;
  switch (group) {
    TS_PF_CASE(1)
    TS_PF_CASE(2)
    TS_PF_CASE(3)
    TS_PF_CASE(4)
    TS_PF_CASE(5)
    TS_PF_CASE(6)
    TS_PF_CASE(7)
    TS_PF_CASE(8)
    default: return fail(TS_ESHAPE, "unsupported head group %d", group);
  }
#undef TS_PF_CASE
#undef TS_PF_LAUNCH
  return check_launch("prefill_attn_kernel");
}

}  // extern "C"
