// Decode attention over the selected KV slots: the FlashInfer paged decode the
// reference calls at tr.py:815-823 (page size 1, in-kernel Llama RoPE).
//
// Split-K in one launch: grid (splits, Hkv, B).  A workgroup owns a contiguous range of
// the request's selected list for one KV head and all G = H/Hkv query heads that read it;
// its four wavefronts walk a quarter of the range each, in tiles of 32 tokens, on the
// matrix cores (see attn_kernel).  Keys are rotated to their index in the selected list,
// the query to S-1; softmax is online in fp32.  Partial (max, sum, acc) triples are merged
// across the wavefronts, written with device-coherent stores, and the workgroup that draws
// the last ticket of its (request, KV head) merges the splits and writes the bf16 output.
#include <math.h>

#include <mutex>
#include <type_traits>

#include "ts_common.h"

namespace ts {

struct AttnArgs {
  const uint16_t* q;  // [B,H,128] bf16, un-rotated
  const uint16_t* k_pool;
  const uint16_t* v_pool;
  uint32_t pool_rows;
  const int32_t* sel;
  int64_t sel_stride;
  const int32_t* sel_len;
  int num_heads, num_kv_heads;
  int group;          // query heads per KV head
  int rope_mode;
  float log2_theta, rope_rcp_scale, sm_scale, logit_cap;
  int nsplit, max_sel_len;
  float* part_acc;    // [B,H,nsplit,128]
  float* part_ml;     // [B,H,nsplit,2]
  uint32_t* tickets;  // [B,Hkv], zero at launch and again when the kernel ends
  uint16_t* out;      // [B,H,128] bf16
  ZeroSet zero;       // cleared on the side (counters of the stream's next selection)
};

// A workgroup's share of the regions to clear, at the start of an attention kernel.
__device__ __forceinline__ void attn_clear_on_the_side(const AttnArgs& a) {
  if (a.zero.used == 0) return;
  const int64_t wg = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
  clear_regions(a.zero, wg * 256 + threadIdx.x, (int64_t)gridDim.x * gridDim.y * gridDim.z * 256);
}

__device__ __forceinline__ float2 load_coherent2(const float* p) {
  const uint64_t v =
      __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_float2(__uint_as_float((uint32_t)v), __uint_as_float((uint32_t)(v >> 32)));
}
// (Plain stores, waited for before the ticket is drawn: exchanges whose old value is
// awaited, the faster way to publish a few words elsewhere, are slower for a
// workgroup's 2 KB of partials.)
__device__ __forceinline__ void store_coherent2(float* p, float x, float y) {
  const uint64_t v = (uint64_t)__float_as_uint(x) | ((uint64_t)__float_as_uint(y) << 32);
  __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The end of an attention workgroup: its four wavefronts' partial (max, sum, acc) triples
// of G head slots lie in LDS; they are merged, written with device-coherent stores, and the
// workgroup that draws the last ticket of its (request, KV head) merges the splits and
// writes the bf16 output.
template <int G>
__device__ __forceinline__ void attn_finish(const AttnArgs& a, int b, int kvh, int split,
                                            float (*sm_acc)[G][kHeadDim], float (*sm_m)[G],
                                            float (*sm_l)[G], uint32_t* s_last_ptr) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int H = a.num_heads;
  auto head_of_slot = [&](int g) { return kvh * G + g; };
  uint32_t& s_last = *s_last_ptr;
  __syncthreads();
  // A thread owns two adjacent dims of one head: one 64-bit coherent store.
  for (int idx = tid; idx < G * (kHeadDim / 2); idx += 256) {
    const int g = idx / (kHeadDim / 2), d = (idx % (kHeadDim / 2)) * 2;
    float mm = kNegBig;
#pragma unroll
    for (int w = 0; w < 4; ++w) mm = fmaxf(mm, sm_m[w][g]);
    float o0 = 0.f, o1 = 0.f, ll = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float sc = __expf(sm_m[w][g] - mm);
      o0 += sm_acc[w][g][d] * sc;
      o1 += sm_acc[w][g][d + 1] * sc;
      ll += sm_l[w][g] * sc;
    }
    const size_t ph = ((size_t)b * H + head_of_slot(g)) * a.nsplit + split;
    store_coherent2(a.part_acc + ph * kHeadDim + d, o0, o1);
    if (d == 0) store_coherent2(a.part_ml + ph * 2, mm, ll);
  }

  // Ticket: the stores above are acknowledged before the workgroup is counted.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  uint32_t* ticket = a.tickets + (size_t)b * a.num_kv_heads + kvh;
  if (tid == 0) {
    const uint32_t before =
        __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = before + 1 == (uint32_t)a.nsplit ? 1u : 0u;
  }
  __syncthreads();
  if (!s_last) return;

  // out[b,h,:] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s, rounded to bf16.
  // A wavefront per head slot (a thread owns two adjacent dims, and a head has 64 such
  // pairs): lane s fetches the (max, sum) of split s, the wave takes the maximum and
  // lane s the weight of its split, so that the accumulators, all requested at once, are
  // added up with weights that are ready (read lane by lane): no chain of dependent
  // exponentials, and one statistics load per wave instead of one per split and thread.
  // With more than four head slots a wavefront has two of them, and works on both at once:
  // one after the other they would be two chains of loads.
  static_assert(kHeadDim / 2 == 64, "one wavefront per head slot");
  constexpr int SLOTS = (G + 3) / 4;  // head slots per wavefront: wave, wave + 4
  const int wave_id = tid >> 6, d = lane * 2;
  size_t ph[SLOTS];
  float mm[SLOTS], ll[SLOTS], o0[SLOTS], o1[SLOTS];
#pragma unroll
  for (int it = 0; it < SLOTS; ++it) {
    // (a slot past the last head repeats the last one and is not written)
    ph[it] = ((size_t)b * H + head_of_slot(min(wave_id + 4 * it, G - 1))) * a.nsplit;
    mm[it] = kNegBig;
    ll[it] = o0[it] = o1[it] = 0.f;
  }
  for (int s0 = 0; s0 < a.nsplit; s0 += 32) {
    // 32 splits at a time, branch-free: loads past the last split repeat it and get
    // the weight zero.
    float2 ac[SLOTS][32], ml[SLOTS];
#pragma unroll
    for (int it = 0; it < SLOTS; ++it) {
#pragma unroll
      for (int i = 0; i < 32; ++i)
        ac[it][i] = load_coherent2(a.part_acc + (ph[it] + min(s0 + i, a.nsplit - 1)) * kHeadDim + d);
      ml[it] = (lane < 32 && s0 + lane < a.nsplit) ? load_coherent2(a.part_ml + (ph[it] + s0 + lane) * 2)
                                                   : make_float2(kNegBig, 0.f);
    }
#pragma unroll
    for (int it = 0; it < SLOTS; ++it) {
      float mx = ml[it].x;
      mx = fmaxf(mx, dpp_move<kRowRor8>(mx));
      mx = fmaxf(mx, dpp_move<kRowRor4>(mx));
      mx = fmaxf(mx, dpp_move<kRowRor2>(mx));
      mx = fmaxf(mx, dpp_move<kRowRor1>(mx));
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      const float mn = fmaxf(mm[it], __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(mx))));
      const float keep = __expf(mm[it] - mn);  // what earlier batches hold
      const float w = (lane < 32 && s0 + lane < a.nsplit) ? __expf(ml[it].x - mn) : 0.f;
      const float wl = ml[it].y * w;
      o0[it] *= keep;
      o1[it] *= keep;
      ll[it] *= keep;
      mm[it] = mn;
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        const float wi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), i));
        ll[it] += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wl), i));
        o0[it] += ac[it][i].x * wi;
        o1[it] += ac[it][i].y * wi;
      }
    }
  }
#pragma unroll
  for (int it = 0; it < SLOTS; ++it) {
    const int g = wave_id + 4 * it;
    if (g < G) {
      const uint32_t packed = (uint32_t)f32_to_bf16(ll[it] > 0.f ? o0[it] / ll[it] : 0.f) |
                              ((uint32_t)f32_to_bf16(ll[it] > 0.f ? o1[it] / ll[it] : 0.f) << 16);
      *(uint32_t*)(a.out + ((size_t)b * H + head_of_slot(g)) * kHeadDim + d) = packed;
    }
  }
  if (tid == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------
// attn_kernel<G, ROPE, CAP>: G = H / Hkv query heads per workgroup (1 to 8), on the matrix
// cores.  A wavefront walks a contiguous quarter of the workgroup's range in tiles of 32
// tokens.  v_mfma_f32_16x16x32_bf16 three times over:
//   logits   S[token][head] = K' Q'^T : A = 16 rotated keys x 32 dims (lane (token l%16,
//            l/16) loads 16 bytes of its token's row per 32 dims and rotates them in fp32 -
//            the partner dims d and d + 64 are in the same lane), B = the query heads as
//            columns (G of 16 used), rotated to S - 1 once.
//   V^T      a value row arrives like a key row (a lane holds 8 consecutive dims of one
//            token); the matrix product with a 0/1 matrix that selects 16 of 32 dims leaves
//            lane (dim l%16, l/16) with that dim of four consecutive tokens, exactly (bf16
//            values summed with zeros in fp32): the transposition, without LDS.
//   output   O^T[dim][head] += V^T P : A = 16 dims x 32 tokens from the step above, B = the
//            weights of the tile, which the logits' product left in the lanes that need them
//            (lane (head l%16, l/16): tokens 4 (l/16) + r of both 16-token halves).
// The matrix instructions take bf16, the reference's attention works in fp32 on rotated keys:
// every fp32 operand (rotated key, rotated query, softmax weight) is therefore split into a
// bf16 value and the bf16 of what the rounding left, x = hi + lo to 2^-18 of x, and the
// products are taken as hi hi + lo hi + hi lo (fp32 accumulation; the values are bf16 as
// stored).  The results match an fp32 evaluation to the rounding of the bf16 output; with
// single bf16 operands the mean error was a hundred times larger and the largest one
// exceeded 2e-2 for outputs of magnitude 2 under a peaked softmax.
// Everything of a head lives in the four lanes of its column: the running maximum moves once
// per tile (two exchanges between the lane groups), the sums stay per lane until the end.
// The loads of the next tile's keys are issued when this tile's have been rotated, those of
// its values after this tile's have been consumed: some 8 KB per wavefront are in flight at
// any time.
typedef __attribute__((ext_vector_type(8))) __bf16 at_bf16x8;
typedef __attribute__((ext_vector_type(4))) float at_f32x4;
constexpr float kAttnLog2e = 1.4426950408889634f, kAttnLn2 = 0.6931471805599453f;
constexpr int kAttnTile = 32;        // tokens per step of a wavefront
constexpr int kAttnChunkUnit = 64;   // a workgroup's range is a multiple of this (16 per wavefront)

__device__ __forceinline__ at_bf16x8 pack8(const float* x) {
  const uint4 w = make_uint4(pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(x[4], x[5]),
                             pack_bf16(x[6], x[7]));
  return __builtin_bit_cast(at_bf16x8, w);
}
__device__ __forceinline__ void unpack8(const uint4& w, float* f) {
  f[0] = bf16_lo(w.x);
  f[1] = bf16_hi(w.x);
  f[2] = bf16_lo(w.y);
  f[3] = bf16_hi(w.y);
  f[4] = bf16_lo(w.z);
  f[5] = bf16_hi(w.z);
  f[6] = bf16_lo(w.w);
  f[7] = bf16_hi(w.w);
}

// x = hi + lo with both halves in bf16: hi = x rounded, lo = the remainder rounded (the
// subtraction is exact); what is lost is 2^-18 of x.
__device__ __forceinline__ void split8(const float* x, at_bf16x8& hi, at_bf16x8& lo) {
  const uint4 h = make_uint4(pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(x[4], x[5]),
                             pack_bf16(x[6], x[7]));
  const float r[8] = {x[0] - bf16_lo(h.x), x[1] - bf16_hi(h.x), x[2] - bf16_lo(h.y), x[3] - bf16_hi(h.y),
                      x[4] - bf16_lo(h.z), x[5] - bf16_hi(h.z), x[6] - bf16_lo(h.w), x[7] - bf16_hi(h.w)};
  hi = __builtin_bit_cast(at_bf16x8, h);
  lo = pack8(r);
}

// Tokens per workgroup of the matrix-core kernel for a launch of nsplit splits.
__host__ __device__ __forceinline__ int attn_chunk(int max_sel_len, int nsplit) {
  const int even = (max_sel_len + nsplit - 1) / nsplit;
  return (even + kAttnChunkUnit - 1) / kAttnChunkUnit * kAttnChunkUnit;
}

// An index offset of zero that the compiler cannot see through, produced after `after` is:
// LDS reads addressed with it stay where they are written (inside the loop, next to their
// use) instead of being gathered at the top, where they would hold dozens of registers.
__device__ __forceinline__ int opaque_zero(uint32_t after) {
  int z = 0;
  asm volatile("" : "+v"(z) : "v"(after));
  return z;
}

template <int G, bool ROPE, bool CAP>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_kernel(AttnArgs a) {
  static_assert(G >= 1 && G <= 8, "the query heads of a KV head are columns of one tile");
  attn_clear_on_the_side(a);
  const int split = blockIdx.x, b = blockIdx.z, kvh = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, qd = lane >> 4;
  const int H = a.num_heads;
  const int chunk = attn_chunk(a.max_sel_len, a.nsplit);
  const int wlen = chunk / 4;
  const int32_t* sel = a.sel + (int64_t)b * a.sel_stride;
  const size_t row_elems = (size_t)a.num_kv_heads * kHeadDim;

  // What every wavefront reads again and again lives in LDS, not in registers (the loop
  // below needs them all): the query operand, the 0/1 matrices, the rotation of one step.
  __shared__ __attribute__((aligned(16))) uint4 sm_q[4][64];     // B operand per 32 dims, per lane
  __shared__ __attribute__((aligned(16))) uint4 sm_q_lo[4][64];  // its low halves
  __shared__ __attribute__((aligned(16))) uint4 sm_pick[2][64];  // B operand per half, per lane
  __shared__ __attribute__((aligned(16))) float2 sm_step[kHeadDim / 2];  // (cos, sin) of 16 tokens
  __shared__ float sm_acc[4][G][kHeadDim];
  __shared__ float sm_m[4][G], sm_l[4][G];
  __shared__ uint32_t s_last;

  // Column n of the logits: query head n of the KV head (zeros beyond its heads).  Wavefront
  // kb2 < 2 prepares the dims [32 kb2, +32) and their partners 64 further on.
  const bool real = n < G;
  const int head = kvh * G + min(n, G - 1);
  // (No load of the start-up sits behind a branch: where a branch joins, the compiler waits
  // for every load that either side may have issued.)
  uint4 q_raw[2];
  {
    const uint16_t* qrow = a.q + ((size_t)b * H + head) * kHeadDim + 32 * (wave & 1) + 8 * qd;
    q_raw[0] = *(const uint4*)qrow;
    q_raw[1] = *(const uint4*)(qrow + 64);
  }
  // The first tile's slots are asked for together with the list's length, not after it.
  // An entry past the wavefront's range (its token gets the weight zero) is replaced by the
  // slot of the range's first token: its row must still be one that holds numbers.
  const int wlo = split * chunk + wave * wlen;
  auto raw_slot = [&](int j) { return (uint32_t)sel[min(j, a.max_sel_len - 1)]; };
  uint32_t slot_cur[2] = {raw_slot(wlo + n), raw_slot(wlo + 16 + n)};
  uint32_t slot_next[2] = {raw_slot(wlo + kAttnTile + n), raw_slot(wlo + kAttnTile + 16 + n)};
  const int S = min(max(a.sel_len[b], 0), a.max_sel_len);
  const int whi = min(S, wlo + wlen);
  const uint32_t first_slot =
      min((uint32_t)__builtin_amdgcn_readfirstlane((int)slot_cur[0]), a.pool_rows - 1);
  auto checked = [&](uint32_t slot, int j) { return j < whi && slot < a.pool_rows ? slot : first_slot; };
  slot_cur[0] = checked(slot_cur[0], wlo + n);
  slot_cur[1] = checked(slot_cur[1], wlo + 16 + n);
  slot_next[0] = checked(slot_next[0], wlo + kAttnTile + n);
  slot_next[1] = checked(slot_next[1], wlo + kAttnTile + 16 + n);
  // ... and the first tile's rows before the set-up below, which then runs while they travel.
  uint4 kr[2][4], vr[2][4];
  auto request = [&](const uint16_t* pool, const uint32_t* slots, uint4 (&dst)[2][4]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const uint16_t* row = pool + (size_t)slots[t] * row_elems + (size_t)kvh * kHeadDim + 8 * qd;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) dst[t][kb] = *(const uint4*)(row + 32 * kb);
    }
  };
  // (a wavefront without tokens asks too: rows of some entry of the list, never used)
  request(a.k_pool, slot_cur, kr);
  request(a.v_pool, slot_cur, vr);

  if (tid < kHeadDim / 2) {
    float sn = 0.f, cs = 1.f;
    if (ROPE) {
      const float freq =
          a.rope_rcp_scale * __builtin_amdgcn_exp2f(-(float)tid * (2.0f / kHeadDim) * a.log2_theta);
      sincos_reduced(16.0f * freq, sn, cs);
    }
    sm_step[tid] = make_float2(cs, sn);
    // 0/1 matrices that pick the dims [16 h, 16 h + 16) of a 32-dim block: B operand, lane
    // (column n, qd) holds rows 8 qd .. 8 qd + 7, of which row 16 h + n is the one.
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint32_t w[4] = {0u, 0u, 0u, 0u};
      if (qd == 2 * h + (n >> 3)) w[(n & 7) >> 1] = (n & 1) ? 0x3f800000u : 0x00003f80u;
      sm_pick[h][lane] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
  if (wave < 2) {  // the query rotated to position S - 1, rounded once
    float x[8], y[8];
    unpack8(real ? q_raw[0] : make_uint4(0u, 0u, 0u, 0u), x);
    unpack8(real ? q_raw[1] : make_uint4(0u, 0u, 0u, 0u), y);
    if (ROPE) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int pair = 32 * wave + 8 * qd + e;
        const float freq =
            a.rope_rcp_scale * __builtin_amdgcn_exp2f(-(float)pair * (2.0f / kHeadDim) * a.log2_theta);
        float sn, cs;
        sincos_reduced((float)(S - 1) * freq, sn, cs);
        const float xr = x[e] * cs - y[e] * sn;
        y[e] = y[e] * cs + x[e] * sn;
        x[e] = xr;
      }
    }
    at_bf16x8 hi, lo;
    split8(x, hi, lo);
    sm_q[wave][lane] = __builtin_bit_cast(uint4, hi);
    sm_q_lo[wave][lane] = __builtin_bit_cast(uint4, lo);
    split8(y, hi, lo);
    sm_q[wave + 2][lane] = __builtin_bit_cast(uint4, hi);
    sm_q_lo[wave + 2][lane] = __builtin_bit_cast(uint4, lo);
  }
  // This lane's 16 rotation pairs: dims 32 kb2 + 8 qd + e (kb2 < 2, e < 8) and their partners
  // 64 further on; key state at token wlo + n, 16 tokens per step.
  float kc[16], ks[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    kc[i] = 1.f;
    ks[i] = 0.f;
    if (ROPE) {
      const int pair = 32 * (i >> 3) + 8 * qd + (i & 7);
      const float freq =
          a.rope_rcp_scale * __builtin_amdgcn_exp2f(-(float)pair * (2.0f / kHeadDim) * a.log2_theta);
      sincos_reduced((float)(wlo + n) * freq, ks[i], kc[i]);
    }
  }
  __syncthreads();  // sm_q, sm_pick, sm_step

  float m = kNegBig, l = 0.f;  // base-2 running maximum, this lane's share of the sum
  at_f32x4 acc[8];             // O^T: dims 16 dt + 4 qd + r of head n
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) acc[dt] = at_f32x4{0.f, 0.f, 0.f, 0.f};

  if (wlo < whi) {
    const float scale2 = a.sm_scale * kAttnLog2e;

    // One tile; `more` (a compile-time flag: the last tile is a copy of the loop's body
    // without the requests) says that another tile follows.  Its loads are unconditional:
    // behind a branch the compiler would wait for all loads where the branch joins, the ones
    // just issued included.
    // `half` (compile-time as well, last tile only): the range ends within the tile's first 16
    // tokens, and nothing is computed for the other 16.
    auto tile = [&](const int j0, auto more_flag, auto half_flag) __attribute__((always_inline)) {
      constexpr bool more = decltype(more_flag)::value;
      constexpr bool half = decltype(half_flag)::value;
      static_assert(!(more && half), "only a last tile ends early");
      // The slots of the tile after the next are asked for before the next tile's rows, so
      // that waiting for them does not mean waiting for those rows (loads return in order).
      uint32_t slot_after[2] = {0u, 0u};
      if (more) {
        slot_after[0] = raw_slot(j0 + 2 * kAttnTile + n);
        slot_after[1] = raw_slot(j0 + 2 * kAttnTile + 16 + n);
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- keys, 16 tokens at a time: rotate, round, multiply, step the rotation
      at_f32x4 s[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int t = 0; t < (half ? 1 : 2); ++t) {
        at_bf16x8 ka[4], ka_lo[4];
#pragma unroll
        for (int kb2 = 0; kb2 < 2; ++kb2) {
          float x[8], y[8];
          unpack8(kr[t][kb2], x);
          unpack8(kr[t][kb2 + 2], y);
          if (ROPE) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float c = kc[8 * kb2 + e], sn = ks[8 * kb2 + e];
              const float xr = x[e] * c - y[e] * sn;
              y[e] = y[e] * c + x[e] * sn;
              x[e] = xr;
            }
          }
          split8(x, ka[kb2], ka_lo[kb2]);
          split8(y, ka[kb2 + 2], ka_lo[kb2 + 2]);
        }
        const int zq = opaque_zero(__builtin_bit_cast(uint4, ka[3]).w);
        s[t] = at_f32x4{0.f, 0.f, 0.f, 0.f};
        // (k_hi + k_lo) (q_hi + q_lo) without the product of the two low halves: three
        // chains that do not wait for each other, added up at the end.
        at_f32x4 s_lh = {0.f, 0.f, 0.f, 0.f}, s_hl = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
          const at_bf16x8 q_hi = __builtin_bit_cast(at_bf16x8, sm_q[kb][lane + zq]);
          const at_bf16x8 q_lo = __builtin_bit_cast(at_bf16x8, sm_q_lo[kb][lane + zq]);
          s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kb], q_hi, s[t], 0, 0, 0);
          s_lh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka_lo[kb], q_hi, s_lh, 0, 0, 0);
          s_hl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kb], q_lo, s_hl, 0, 0, 0);
        }
        s[t] += s_lh + s_hl;
        __builtin_amdgcn_sched_barrier(0);
        if (ROPE && (more || (t == 0 && !half))) {  // the same rows of the next 16 tokens
#pragma unroll
          for (int kb2 = 0; kb2 < 2; ++kb2) {
            const int zs = opaque_zero(__float_as_uint(kc[8 * kb2]));
            const float4* step = (const float4*)&sm_step[32 * kb2 + 8 * qd + zs];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
              const float4 d = step[e2];
              const float dcs[2] = {d.x, d.z}, dsn[2] = {d.y, d.w};
#pragma unroll
              for (int o = 0; o < 2; ++o) {
                const int i = 8 * kb2 + 2 * e2 + o;
                const float c2 = kc[i] * dcs[o] - ks[i] * dsn[o];
                ks[i] = ks[i] * dcs[o] + kc[i] * dsn[o];
                kc[i] = c2;
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      // the next tile's keys, into the registers just read
      if (more) request(a.k_pool, slot_next, kr);
      __builtin_amdgcn_sched_barrier(0);
      // ---- weights of 32 tokens x 16 head columns
      float p[8];
      float mx = kNegBig;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (half && t == 1) {
            p[4 + r] = -INFINITY;
            continue;
          }
          float v;
          if (CAP)
            v = a.logit_cap * tanhf(s[t][r] * a.sm_scale / a.logit_cap) * kAttnLog2e;
          else
            v = s[t][r] * scale2;
          v = j0 + 16 * t + 4 * qd + r < whi ? v : -INFINITY;
          p[4 * t + r] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float mn = fmaxf(m, mx);
      const float alpha = __builtin_amdgcn_exp2f(m - mn);
      m = mn;
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p[i] = half && i >= 4 ? 0.f : __builtin_amdgcn_exp2f(p[i] - mn);
        sum += p[i];
      }
      l = l * alpha + sum;
#pragma unroll
      for (int dt = 0; dt < 8; ++dt) acc[dt] *= alpha;
      at_bf16x8 pb, pb_lo;
      split8(p, pb, pb_lo);
      // ---- values: transpose 16 dims at a time, accumulate
      const int zp = opaque_zero(__builtin_bit_cast(uint4, pb).x);
      at_bf16x8 pick[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) pick[h] = __builtin_bit_cast(at_bf16x8, sm_pick[h][lane + zp]);
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const at_f32x4 zero = {0.f, 0.f, 0.f, 0.f};
          const at_f32x4 d0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(at_bf16x8, vr[0][c]), pick[h], zero, 0, 0, 0);
          const at_f32x4 d1 = half ? zero
                                   : __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                         __builtin_bit_cast(at_bf16x8, vr[1][c]), pick[h], zero, 0, 0, 0);
          const float vt[8] = {d0[0], d0[1], d0[2], d0[3], d1[0], d1[1], d1[2], d1[3]};
          const at_bf16x8 vta = pack8(vt);
          acc[2 * c + h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vta, pb, acc[2 * c + h], 0, 0, 0);
          acc[2 * c + h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vta, pb_lo, acc[2 * c + h], 0, 0, 0);
        }
      __builtin_amdgcn_sched_barrier(0);
      if (more) {
        request(a.v_pool, slot_next, vr);
        slot_next[0] = checked(slot_after[0], j0 + 2 * kAttnTile + n);
        slot_next[1] = checked(slot_after[1], j0 + 2 * kAttnTile + 16 + n);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // (Lowering a wavefront's priority as it advances, which evens out the two workgroups of
    // a CU in the kernel above, evens them out here too and gains nothing: the rows arrive
    // as fast as the memory system delivers them either way.)
    int j0 = wlo;
    for (; j0 + kAttnTile < whi; j0 += kAttnTile) tile(j0, std::true_type{}, std::false_type{});
    if (whi - j0 <= kAttnTile / 2)
      tile(j0, std::false_type{}, std::true_type{});
    else
      tile(j0, std::false_type{}, std::false_type{});
  }

  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  if (n < G) {
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
      *(float4*)&sm_acc[wave][n][16 * dt + 4 * qd] = make_float4(acc[dt][0], acc[dt][1], acc[dt][2], acc[dt][3]);
    if (qd == 0) {
      sm_m[wave][n] = m * kAttnLn2;  // natural-log units, as the merge expects
      sm_l[wave][n] = l;
    }
  }
  attn_finish<G>(a, b, kvh, split, sm_acc, sm_m, sm_l, &s_last);
}

__global__ __launch_bounds__(256) void attn_zero_kernel(uint32_t* tickets, int count) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256) tickets[i] = 0u;
}

// Tickets per request (the words to clear): one per KV head.
int attn_tickets_per_request(const ts_config* cfg) { return cfg->num_kv_heads; }

constexpr int kAttnRange = 128;  // list entries per workgroup as long as the device has room
static int attn_splits(int batch, int num_kv_heads, int max_sel_len) {
  // One tile per wavefront (128 entries per workgroup) as long as the grid stays within the
  // 512 workgroups that are resident at once (two per CU): a second round of workgroups pays
  // the start-up and merge latencies again, which costs more than longer ranges do.
  int64_t want = ceil_div(max_sel_len, kAttnRange);
  const int64_t cap = ceil_div(512, (int64_t)batch * num_kv_heads);
  if (want > cap) want = cap;
  if (want < 1) want = 1;
  // (ranges are whole multiples of 64 entries: the last splits may have nothing left)
  return (int)ceil_div(max_sel_len, attn_chunk(max_sel_len, (int)want));
}

struct AttnWorkspace {
  size_t acc, ml, tickets, total;
};
static AttnWorkspace attn_workspace(const ts_config* cfg, int batch, int max_sel_len) {
  const size_t ns = (size_t)attn_splits(batch, attn_tickets_per_request(cfg), max_sel_len);
  const size_t heads = (size_t)batch * cfg->num_heads;
  AttnWorkspace w;
  w.acc = 0;
  w.ml = w.acc + align_up(heads * ns * kHeadDim * 4, 256);
  w.tickets = w.ml + align_up(heads * ns * 2 * 4, 256);
  w.total = w.tickets + align_up((size_t)batch * attn_tickets_per_request(cfg) * 4, 256);
  return w;
}

uint32_t* attn_tickets(const ts_config* cfg, int batch, int max_sel_len, void* workspace) {
  return (uint32_t*)((char*)workspace + attn_workspace(cfg, batch, max_sel_len).tickets);
}

int launch_attn(const ts_config* cfg, const void* q, const void* k_pool, const void* v_pool,
                int64_t pool_rows, const int32_t* sel, int64_t sel_stride, const int32_t* sel_len,
                int batch, int max_sel_len, void* out, void* workspace, bool tickets_clear,
                hipStream_t st, const ZeroSet* clear_after) {
  const AttnWorkspace w = attn_workspace(cfg, batch, max_sel_len);
  AttnArgs a;
  if (clear_after) {
    TS_REQUIRE(!clear_after->overflow, TS_EINVAL, "internal: more than %d regions to clear in one launch",
               kZeroRegions);
    a.zero = *clear_after;
  }
  a.q = (const uint16_t*)q;
  a.k_pool = (const uint16_t*)k_pool;
  a.v_pool = (const uint16_t*)v_pool;
  a.pool_rows = (uint32_t)pool_rows;
  a.sel = sel;
  a.sel_stride = sel_stride;
  a.sel_len = sel_len;
  a.num_heads = cfg->num_heads;
  a.num_kv_heads = cfg->num_kv_heads;
  a.group = cfg->num_heads / cfg->num_kv_heads;
  a.rope_mode = cfg->rope_mode;
  a.log2_theta = cfg->rope_mode == TS_ROPE_LLAMA ? (float)log2((double)cfg->rope_theta) : 0.f;
  a.rope_rcp_scale = cfg->rope_mode == TS_ROPE_LLAMA ? 1.0f / cfg->rope_scale : 1.0f;
  a.sm_scale = cfg->sm_scale;
  a.logit_cap = cfg->logit_cap;
  a.nsplit = attn_splits(batch, attn_tickets_per_request(cfg), max_sel_len);
  a.max_sel_len = max_sel_len;
  a.part_acc = (float*)((char*)workspace + w.acc);
  a.part_ml = (float*)((char*)workspace + w.ml);
  a.tickets = (uint32_t*)((char*)workspace + w.tickets);
  a.out = (uint16_t*)out;

  if (!tickets_clear) {
    const int count = batch * attn_tickets_per_request(cfg);
    hipLaunchKernelGGL(attn_zero_kernel, dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, st,
                       a.tickets, count);
    TS_TRY(check_launch("attn_zero_kernel"));
  }
  const dim3 grid((unsigned)a.nsplit, (unsigned)attn_tickets_per_request(cfg), (unsigned)batch);
  const bool rope = cfg->rope_mode == TS_ROPE_LLAMA, cap = cfg->logit_cap > 0.f;
#define TS_ATTN_LAUNCH(G_, R_, C_) hipLaunchKernelGGL((attn_kernel<G_, R_, C_>), grid, dim3(256), 0, st, a)
#define TS_ATTN_CASE(G_)                              \
  case G_:                                            \
    if (rope && cap) TS_ATTN_LAUNCH(G_, true, true);  \
    else if (rope) TS_ATTN_LAUNCH(G_, true, false);   \
    else if (cap) TS_ATTN_LAUNCH(G_, false, true);    \
    else TS_ATTN_LAUNCH(G_, false, false);            \
    break;
  switch (a.group) {
    TS_ATTN_CASE(1)
    TS_ATTN_CASE(2)
    TS_ATTN_CASE(3)
    TS_ATTN_CASE(4)
    TS_ATTN_CASE(5)
    TS_ATTN_CASE(6)
    TS_ATTN_CASE(7)
    TS_ATTN_CASE(8)
    default: return fail(TS_ESHAPE, "unsupported head group %d", a.group);
  }
#undef TS_ATTN_CASE
#undef TS_ATTN_LAUNCH
  return check_launch("attn_kernel");
}

// Scratch of ts_sparse_decode_attn_static: the split-K partials and tickets of one
// launch, held by every device the library runs on until the process ends.
constexpr size_t kStaticScratchBytes = 4u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device, looked up once per device (each
// device holds its own copy at its own address); NULL with the error set on failure.
constexpr int kMaxDevices = 64;
static void* static_scratch() {
  static std::mutex mu;
  static void* ptr_of_device[kMaxDevices] = {};
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
    (void)hipGetLastError();
    fail(TS_EHIP, "ts_sparse_decode_attn_static: no current device (%s)", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptr_of_device[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      fail(TS_EHIP, "ts_sparse_decode_attn_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    ptr_of_device[device] = ptr;
  }
  return ptr_of_device[device];
}

}  // namespace ts

using namespace ts;

extern "C" {

size_t ts_attn_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_sel_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_sel_len < 1) return 0;
  return attn_workspace(cfg, batch, max_sel_len).total;
}

int ts_sparse_decode_attn(const ts_config* cfg, const void* q, const void* k_pool,
                          const void* v_pool, int64_t pool_rows, const int32_t* sel,
                          int64_t sel_stride, const int32_t* sel_len, int32_t batch,
                          int32_t max_sel_len, void* out, void* workspace,
                          size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(q && k_pool && v_pool && sel && sel_len && out, TS_EINVAL,
             "ts_sparse_decode_attn: NULL tensor argument");
  TS_REQUIRE(batch >= 1 && batch <= 65535, TS_EINVAL, "batch %d out of range", batch);
  TS_REQUIRE(max_sel_len >= 1, TS_EINVAL, "max_sel_len %d < 1", max_sel_len);
  TS_REQUIRE(sel_stride >= max_sel_len || batch == 1, TS_EWORKSPACE,
             "sel_stride %lld < max_sel_len %d", (long long)sel_stride, max_sel_len);
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const size_t need = ts_attn_workspace_bytes(cfg, batch, max_sel_len);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= need, TS_EWORKSPACE,
             "ts_sparse_decode_attn: workspace %zu bytes < required %zu", workspace_bytes, need);
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_REQUIRE_ALIGNED(out, 16, "out");
  return launch_attn(cfg, q, k_pool, v_pool, pool_rows, sel, sel_stride, sel_len, batch, max_sel_len,
                     out, workspace, /*tickets_clear=*/false, (hipStream_t)stream);
}

size_t ts_attn_static_scratch_bytes(void) {
  // The query a caller makes at set-up also looks up the buffer's address on the current
  // device, so that a first call under graph capture makes no runtime query of its own.
  // (Without a device there is nothing to look up, and the size is still the answer.)
  int devices = 0;
  if (hipGetDeviceCount(&devices) == hipSuccess && devices > 0) (void)static_scratch();
  (void)hipGetLastError();
  return kStaticScratchBytes;
}

int ts_sparse_decode_attn_static(const ts_config* cfg, const void* q, const void* k_pool,
                                 const void* v_pool, int64_t pool_rows, const int32_t* sel,
                                 int64_t sel_stride, const int32_t* sel_len, int32_t batch,
                                 int32_t max_sel_len, void* out, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(q && k_pool && v_pool && sel && sel_len && out, TS_EINVAL,
             "ts_sparse_decode_attn_static: NULL tensor argument");
  TS_REQUIRE(batch >= 1 && batch <= 65535, TS_EINVAL, "batch %d out of range", batch);
  TS_REQUIRE(max_sel_len >= 1, TS_EINVAL, "max_sel_len %d < 1", max_sel_len);
  TS_REQUIRE(sel_stride >= max_sel_len || batch == 1, TS_EWORKSPACE,
             "sel_stride %lld < max_sel_len %d", (long long)sel_stride, max_sel_len);
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const size_t need = attn_workspace(cfg, batch, max_sel_len).total;
  TS_REQUIRE(need <= kStaticScratchBytes, TS_EWORKSPACE,
             "ts_sparse_decode_attn_static: batch %d x %d heads x %d selected needs %zu bytes of "
             "scratch, the built-in buffer holds %zu; use ts_sparse_decode_attn with a workspace",
             batch, cfg->num_heads, max_sel_len, need, kStaticScratchBytes);
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_REQUIRE_ALIGNED(out, 16, "out");
  void* ptr = static_scratch();
  if (ptr == nullptr) return TS_EHIP;
  // The tickets are cleared by a fill kernel on the caller's stream (the previous call
  // may have been interrupted), so the call can be captured into a HIP graph.
  return launch_attn(cfg, q, k_pool, v_pool, pool_rows, sel, sel_stride, sel_len, batch, max_sel_len,
                     out, ptr, /*tickets_clear=*/false, (hipStream_t)stream);
}

}  // extern "C"
