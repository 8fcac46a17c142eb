// Chunked prefill (patched_radix_attention_extend_forward_flashinfer, tr.py:703-775):
// the fingerprint of a chunk (mean of its rotated query rows, tr.py:380-392) and the
// causal attention of the chunk's rows over the selected KV slots (FlashInfer paged
// prefill, tr.py:759-771, page size 1, in-kernel Llama RoPE).
#include <math.h>

#include "ts_common.h"

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
    ZeroRegion zero, ZeroRegion zero2, ZeroRegion zero3) {
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
    for (int64_t w = gid; w < (int64_t)zero.count * zero.words; w += step)
      zero.base[(w / zero.words) * zero.stride + w % zero.words] = 0u;
    for (int64_t w = gid; w < (int64_t)zero2.count * zero2.words; w += step)
      zero2.base[(w / zero2.words) * zero2.stride + w % zero2.words] = 0u;
    for (int64_t w = gid; w < (int64_t)zero3.count * zero3.words; w += step)
      zero3.base[(w / zero3.words) * zero3.stride + w % zero3.words] = 0u;
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
// tiles.  (That repetition made the first version of this kernel bound by vector
// instructions at 5 % of the matrix peak.)
//
// prefill_attn_kernel<G>: grid (16-row query tiles, KV heads, quads of the G query
// heads of a KV head); 512 threads = two groups of four wavefronts.  The wavefronts
// of a group serve one query head each and share the K/V tiles of their KV head;
// group 0 takes the even 64-key tiles and group 1 the odd ones (two wavefronts per
// SIMD hide each other's LDS and matrix latencies), and their (max, sum, acc) are
// merged through LDS at the end.  Per tile a group copies 16 KB of kr and 16 KB of vt
// into one of its two LDS buffers (the pieces of the next two tiles already in
// registers) while the wavefronts compute on the other: one barrier per tile.  A
// wavefront computes S^T = K Q^T with v_mfma_f32_16x16x32_bf16 (A = 16 keys x 32 dims
// from LDS, B = its 16 rotated queries, held in registers, pre-multiplied by the softmax
// scale and log2 e), which leaves lane (query l%16, key group l/16) with the base-2
// logits of 16 keys; the online softmax needs two cross-lane maxima per tile; the 16
// probabilities, rounded to bf16, are directly the B operands of O^T += V^T P^T (A = 16
// dims x 32 keys from the transposed V tile, keys in the order the logits came in), so
// no data moves between the two products.  fp32 accumulation throughout.
// What the time went into, by the counters: neither the matrix units (17 % busy), nor
// the vector ALU, nor LDS bandwidth, but waiting: bank conflicts of the V^T rows (now
// padded to 34 banks), and the two barriers per tile of the single-buffered version.
struct PrefillArgs {
  const uint16_t* q;  // [rows, H, 128] bf16, un-rotated
  const uint16_t* k_pool;
  const uint16_t* v_pool;
  uint32_t pool_rows;
  const int32_t* sel;      // [S] selected slots in attention order
  const int32_t* sel_len;  // device scalar S
  int max_sel_len;
  int s_pad;               // columns of a vt row: max_sel_len rounded up to the tile
  int rows;
  int num_heads, num_kv_heads, rope_mode;
  float log2_theta, rope_rcp_scale, sm_scale, logit_cap;
  uint16_t* kr;   // [Hkv, s_pad, 128] bf16 rotated keys
  uint16_t* vt;   // [Hkv, 128, s_pad] bf16 transposed values
  uint16_t* out;  // [rows, H, 128] bf16
};

typedef __attribute__((ext_vector_type(8))) __bf16 pf_bf16x8;
typedef __attribute__((ext_vector_type(4))) float pf_f32x4;
constexpr float kLog2e = 1.4426950408889634f;

constexpr int kPfKeys = 32;               // keys per workgroup of the gather kernel
constexpr int kPfKRow = kHeadDim + 8;     // halfwords per K row in LDS (272 B: rows on different banks)
constexpr int kPfVRow = kPfKeys + 8;      // halfwords per V^T row in the gather kernel's LDS (80 B)
constexpr int kPfTile = 64;               // keys per tile of the attention kernel
constexpr int kPfPipeA = 2;               // attention tiles whose pieces are in flight
constexpr int kPfVRowA = kPfTile + 4;     // halfwords per V^T row in the attention kernel's LDS:
                                          // 136 B = 34 banks, the 16 rows a wavefront reads together
                                          // (8 bytes each) fall on distinct banks

// Two floats to packed bf16, round to nearest even, in one v_cvt_pk_bf16_f32.
typedef __attribute__((ext_vector_type(2))) __bf16 pf_bf16x2;
typedef __attribute__((ext_vector_type(2))) float pf_f32x2;
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const pf_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, pf_bf16x2));
}

// Grid (32-key tiles, KV heads).  Thread (key kk, chunk c) moves dims [8c, 8c+8) and
// [64+8c, +8) of key j = tile + kk.  Keys past S are written as zeros.
__global__ __launch_bounds__(256) void prefill_gather_kernel(PrefillArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t vt_lds[kHeadDim * kPfVRow];
  const int tid = threadIdx.x;
  const int kk = tid >> 3, c8 = tid & 7;
  const int kvh = blockIdx.y;
  const int S = min(max(*a.sel_len, 0), a.max_sel_len);
  const int j = blockIdx.x * kPfKeys + kk;
  // Whole tiles of the attention kernel: the keys between S and the next multiple of
  // its tile are written as zeros too (their weights are zero, but 0 x garbage is not).
  if (blockIdx.x * kPfKeys >= (S + kPfTile - 1) / kPfTile * kPfTile) return;
  const bool live = j < S;
  uint4 kraw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  uint4 vraw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  if (live) {
    uint32_t slot = (uint32_t)a.sel[j];
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
  // transpose the 32 x 128 V tile through LDS, then write 128 rows of 64 bytes
  const uint32_t vlo[4] = {vraw[0].x, vraw[0].y, vraw[0].z, vraw[0].w};
  const uint32_t vhi[4] = {vraw[1].x, vraw[1].y, vraw[1].z, vraw[1].w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    vt_lds[(8 * c8 + 2 * e) * kPfVRow + kk] = (uint16_t)(vlo[e] & 0xffffu);
    vt_lds[(8 * c8 + 2 * e + 1) * kPfVRow + kk] = (uint16_t)(vlo[e] >> 16);
    vt_lds[(64 + 8 * c8 + 2 * e) * kPfVRow + kk] = (uint16_t)(vhi[e] & 0xffffu);
    vt_lds[(64 + 8 * c8 + 2 * e + 1) * kPfVRow + kk] = (uint16_t)(vhi[e] >> 16);
  }
  __syncthreads();
  const int d = tid >> 1, half = tid & 1;
  uint16_t* vrow = a.vt + ((size_t)kvh * kHeadDim + d) * a.s_pad + blockIdx.x * kPfKeys + 16 * half;
  const uint4* src = (const uint4*)(vt_lds + d * kPfVRow + 16 * half);
  ((uint4*)vrow)[0] = src[0];
  ((uint4*)vrow)[1] = src[1];
}

// Two wavefronts per SIMD by construction (8 per workgroup, one workgroup per CU):
// saying so lets the compiler use 256 registers instead of spilling at 128.
template <int G, bool CAP>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void prefill_attn_kernel(
    PrefillArgs a) {
  // Dynamic LDS: per group two buffers of a K tile [kPfTile * kPfKRow] followed by a V^T
  // tile [kHeadDim * kPfVRowA]; the merge of the two groups at the end reuses the space.
  extern __shared__ __attribute__((aligned(16))) uint16_t pf_lds[];
  constexpr int kBuf = kPfTile * kPfKRow + kHeadDim * kPfVRowA;  // halfwords per buffer
  const int group = threadIdx.x >> 8;  // which of the two tile streams this wavefront follows
  uint16_t* const k_lds = pf_lds + group * (2 * kBuf);
  uint16_t* const vt_lds = k_lds + kPfTile * kPfKRow;
  float(*merge_lds)[64][34] = (float(*)[64][34])pf_lds;  // [4][64][34]
  static_assert(4 * 64 * 34 * 4 <= 4 * kBuf * 2, "the merge area fits the tiles");

  const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
  const int qc = lane & 15, g4 = lane >> 4;  // query column / key group of the MFMA layouts
  const int kvh = blockIdx.y;
  const int head_in_group = blockIdx.z * 4 + wave;
  const bool wave_active = head_in_group < G;
  const int h = kvh * G + (wave_active ? head_in_group : 0);
  const int H = a.num_heads;
  const int S = min(max(*a.sel_len, 0), a.max_sel_len);
  const int m = a.rows;
  const int q_row0 = blockIdx.x * 16;
  const int shift = S - m;  // query row i sits at position shift + i and sees keys <= that
  const bool rope = a.rope_mode == TS_ROPE_LLAMA;
  if (S < m || S <= 0) {
    // Fewer keys than rows (not a prefill chunk, or a selection that reported a
    // fault): the rows attend to nothing and the output is defined as zero.
    if (wave_active)
      for (int i = lane; i < 16 * (kHeadDim / 8); i += 64) {
        const int row = q_row0 + i / (kHeadDim / 8);
        if (row < m)
          *(uint4*)(a.out + ((size_t)row * H + h) * kHeadDim + 8 * (i % (kHeadDim / 8))) =
              make_uint4(0u, 0u, 0u, 0u);
      }
    return;
  }

  // ---- queries: B operand, lane (qc, g4) holds dims [32 ks + 8 g4, +8) of row q_row0 + qc,
  // rotated to position shift + row (partner dims d and d + 64 are k-steps ks and ks + 2).
  const int q_row = min(q_row0 + qc, m - 1);
  pf_bf16x8 qb[4];
  {
    float x[4][8];
    const uint16_t* qrow = a.q + ((size_t)q_row * H + h) * kHeadDim;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const uint4 w = *(const uint4*)(qrow + 32 * ks + 8 * g4);
      const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[ks][2 * e] = bf16_lo(ww[e]);
        x[ks][2 * e + 1] = bf16_hi(ww[e]);
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
          const float lo = x[ks][e], hi = x[ks + 2][e];
          x[ks][e] = lo * cs - hi * sn;
          x[ks + 2][e] = hi * cs + lo * sn;
        }
    }
    // Without a soft cap the softmax scale and log2(e) go into the query, so that the
    // products come out as base-2 logits and every key costs one exp2 and no multiply.
    const float qs = CAP ? 1.0f : a.sm_scale * kLog2e;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[ks][e] *= qs;
      const uint4 w = make_uint4(pack_bf16(x[ks][0], x[ks][1]), pack_bf16(x[ks][2], x[ks][3]),
                                 pack_bf16(x[ks][4], x[ks][5]), pack_bf16(x[ks][6], x[ks][7]));
      qb[ks] = __builtin_bit_cast(pf_bf16x8, w);
    }
  }

  // ---- staging role: thread t copies four 16-byte pieces of the K tile (keys t/8 and
  // t/8 + 32, dims [8 (t%8), +8) and the same 64 dims further on: consecutive lanes write
  // consecutive 16 bytes of a K row, which the LDS banks take without conflicts) and 64
  // bytes of the V^T tile (dim t/2, keys [32 (t%2), +32)).
  const uint16_t* k_src = a.kr + (size_t)kvh * a.s_pad * kHeadDim + (size_t)(tid >> 3) * kHeadDim +
                          8 * (tid & 7);
  const uint16_t* v_src = a.vt + ((size_t)kvh * kHeadDim + (tid >> 1)) * a.s_pad + 32 * (tid & 1);
  uint16_t* k_dst = k_lds + (tid >> 3) * kPfKRow + 8 * (tid & 7);
  uint16_t* v_dst = vt_lds + (tid >> 1) * kPfVRowA + 32 * (tid & 1);  // 8-byte aligned
  // Two register buffers, named rather than indexed: an indexed array of them is
  // kept in scratch memory by the compiler, and the prefetch with it.
  struct TilePiece {
    uint4 k0, k1, k2, k3, v0, v1, v2, v3;
  };
  TilePiece piece0, piece1;
  auto request_tile = [&](int tile) __attribute__((always_inline)) -> TilePiece {
    tile = min(tile, a.s_pad - kPfTile);  // past the end: harmless repeat of the last tile
    const uint4* ks = (const uint4*)(k_src + (size_t)tile * kHeadDim);
    const uint4* vs = (const uint4*)(v_src + tile);
    TilePiece piece;
    piece.k0 = ks[0];
    piece.k1 = ks[8];                      // 64 dims further on
    piece.k2 = ks[32 * kHeadDim / 8];      // 32 keys further on
    piece.k3 = ks[32 * kHeadDim / 8 + 8];
    piece.v0 = vs[0];
    piece.v1 = vs[1];
    piece.v2 = vs[2];
    piece.v3 = vs[3];
    return piece;
  };

  // ---- main loop over the tiles any row of this query tile can see
  const int last_visible = min(S - 1, shift + min(q_row0 + 15, m - 1));
  const int my_limit = shift + q_row;  // last key this lane's query sees
  float m_run = kNegBig, l_run = 0.f;
  pf_f32x4 o[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) o[db] = pf_f32x4{0.f, 0.f, 0.f, 0.f};

  // One 64-key tile of this group: logits, online softmax, output update.
  auto compute_tile = [&](int tile, int buf) __attribute__((always_inline)) {
    const uint16_t* const kt = k_lds + buf * kBuf;
    const uint16_t* const vt = vt_lds + buf * kBuf;
    // logits (base 2): s[blk][r] belongs to key tile + 16 blk + 4 g4 + r and query qc.
    // Only the tiles on the diagonal hold keys that some query of the tile must not see.
    const bool diagonal = tile + kPfTile - 1 > shift + q_row0;
    float s[4][4];
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      pf_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const uint4 kw = *(const uint4*)(kt + (16 * blk + qc) * kPfKRow + 32 * ks + 8 * g4);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, kw), qb[ks],
                                                      acc, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float x = acc[r];
        if (CAP) x = a.logit_cap * tanhf(x * a.sm_scale / a.logit_cap) * kLog2e;
        const int key = tile + 16 * blk + 4 * g4 + r;
        // Masked logits are -inf and the running maximum starts at a finite value,
        // so exp2(s - max) is 0 for them without a branch and never NaN.
        s[blk][r] = (!diagonal || key <= my_limit) ? x : -INFINITY;
      }
    }
    float mx = kNegBig;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[blk][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float p[4][4], psum = 0.f;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p[blk][r] = __builtin_amdgcn_exp2f(s[blk][r] - m_new);
        psum += p[blk][r];
      }
    l_run = l_run * alpha + psum;
    // The accumulators only need rescaling when some query's maximum moved, which
    // after the first tiles is rare: skip the 32 multiplications otherwise.
    const bool rescale = __ballot(m_new != m_run) != 0ull;
    m_run = m_new;
    pf_bf16x8 pb[2];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const uint4 pw = make_uint4(pack_bf16(p[2 * hf][0], p[2 * hf][1]),
                                  pack_bf16(p[2 * hf][2], p[2 * hf][3]),
                                  pack_bf16(p[2 * hf + 1][0], p[2 * hf + 1][1]),
                                  pack_bf16(p[2 * hf + 1][2], p[2 * hf + 1][3]));
      pb[hf] = __builtin_bit_cast(pf_bf16x8, pw);
    }
    if (rescale) {
#pragma unroll
      for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[db][r] *= alpha;
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const uint16_t* vrow = vt + (16 * db + qc) * kPfVRowA;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const uint2 v0 = *(const uint2*)(vrow + 32 * hf + 4 * g4);
        const uint2 v1 = *(const uint2*)(vrow + 32 * hf + 16 + 4 * g4);
        const uint4 vw = make_uint4(v0.x, v0.y, v1.x, v1.y);
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pf_bf16x8, vw), pb[hf],
                                                        o[db], 0, 0, 0);
      }
    }
  };

  // The LDS tiles are double-buffered: while the wavefronts compute on one buffer, the
  // next tile (its pieces already in registers) is written to the other, and one
  // barrier per tile separates "everybody has read buffer b" from its next overwrite.
  // Tile number i of this group (keys (2 i + group) * 64 ...) travels through register
  // buffer i % 2 and LDS buffer i % 2; the steps are written out for the two parities so
  // that each uses its own named registers.
  static_assert(kPfPipeA == 2, "the steps below are written out for two buffers");
#define TS_PF_STORE(u, buf)                                                                  \
  {                                                                                          \
    uint16_t* const kd = k_dst + (buf) * kBuf;                                               \
    uint16_t* const vd = v_dst + (buf) * kBuf;                                               \
    ((uint4*)kd)[0] = piece##u.k0;                                                           \
    ((uint4*)kd)[8] = piece##u.k1;                                                           \
    ((uint4*)(kd + 32 * kPfKRow))[0] = piece##u.k2;                                          \
    ((uint4*)(kd + 32 * kPfKRow))[8] = piece##u.k3;                                          \
    ((uint2*)vd)[0] = make_uint2(piece##u.v0.x, piece##u.v0.y);                              \
    ((uint2*)vd)[1] = make_uint2(piece##u.v0.z, piece##u.v0.w);                              \
    ((uint2*)vd)[2] = make_uint2(piece##u.v1.x, piece##u.v1.y);                              \
    ((uint2*)vd)[3] = make_uint2(piece##u.v1.z, piece##u.v1.w);                              \
    ((uint2*)vd)[4] = make_uint2(piece##u.v2.x, piece##u.v2.y);                              \
    ((uint2*)vd)[5] = make_uint2(piece##u.v2.z, piece##u.v2.w);                              \
    ((uint2*)vd)[6] = make_uint2(piece##u.v3.x, piece##u.v3.y);                              \
    ((uint2*)vd)[7] = make_uint2(piece##u.v3.z, piece##u.v3.w);                              \
  }
  // Step for the tile in LDS buffer `cur`: stage the following tile from register buffer
  // `nxt` into LDS buffer `nxt`, request the tile after that, compute, barrier.
#define TS_PF_STEP(cur, nxt)                                                                 \
  {                                                                                          \
    const int pair = round + 2 * kPfTile * (cur);                                            \
    if (pair > last_visible) break;                                                          \
    const int tile = pair + kPfTile * group;                                                 \
    TS_PF_STORE(nxt, nxt)                                                                    \
    piece##nxt = request_tile(tile + 3 * 2 * kPfTile);                                       \
    if (wave_active && tile <= last_visible) compute_tile(tile, cur);                        \
    __syncthreads();                                                                         \
  }
  piece0 = request_tile(kPfTile * (0 + group));
  piece1 = request_tile(kPfTile * (2 + group));
  TS_PF_STORE(0, 0)
  piece0 = request_tile(kPfTile * (4 + group));
  __syncthreads();
  for (int round = 0; round <= last_visible; round += 2 * kPfPipeA * kPfTile) {
    TS_PF_STEP(0, 1)
    TS_PF_STEP(1, 0)
  }
#undef TS_PF_STEP
#undef TS_PF_STORE
  // (the barrier that ended the last step also freed the tiles' space for the merge)
  // Group 1 hands its partial result to group 0 (same wavefront index, same lane).
  if (group == 1) {
    float* mine = merge_lds[wave][lane];
    mine[0] = m_run;
    mine[1] = l_run;
#pragma unroll
    for (int db = 0; db < 8; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[2 + 4 * db + r] = o[db][r];
  }
  __syncthreads();
  if (group == 1 || !wave_active || q_row0 + qc >= m) return;
  {
    const float* other = merge_lds[wave][lane];
    const float m_new = fmaxf(m_run, other[0]);
    const float e0 = __builtin_amdgcn_exp2f(m_run - m_new), e1 = __builtin_amdgcn_exp2f(other[0] - m_new);
    l_run = l_run * e0 + other[1] * e1;
#pragma unroll
    for (int db = 0; db < 8; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[db][r] = o[db][r] * e0 + other[2 + 4 * db + r] * e1;
  }

  // o[db][r] = O[query qc][dim 16 db + 4 g4 + r]; the row sum is spread over the 4 key groups.
  float l_tot = l_run + __shfl_xor(l_run, 16);
  l_tot += __shfl_xor(l_tot, 32);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  uint16_t* orow = a.out + ((size_t)(q_row0 + qc) * H + h) * kHeadDim;
#pragma unroll
  for (int db = 0; db < 8; ++db)
    *(uint2*)(orow + 16 * db + 4 * g4) = make_uint2(pack_bf16(o[db][0] * inv, o[db][1] * inv),
                                                    pack_bf16(o[db][2] * inv, o[db][3] * inv));
}

constexpr size_t kPfLdsBytes = 2 * 2 * (size_t)(kPfTile * kPfKRow + kHeadDim * kPfVRowA) * 2;

int launch_fingerprint(const ts_config* cfg, const void* q, int32_t rows, const float* cos_table,
                       const float* sin_table, int64_t table_rows, void* qf, const ZeroRegion& zero,
                       const ZeroRegion& zero2, hipStream_t stream, const ZeroRegion& zero3) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(q && cos_table && sin_table && qf, TS_EINVAL, "ts_fingerprint: NULL tensor argument");
  TS_REQUIRE(rows >= 1, TS_EINVAL, "ts_fingerprint: rows %d < 1", rows);
  TS_REQUIRE(table_rows >= (int64_t)cfg->n_local + rows, TS_EINVAL,
             "ts_fingerprint: cos/sin tables have %lld rows, need n_local + rows = %lld",
             (long long)table_rows, (long long)cfg->n_local + rows);
  hipLaunchKernelGGL(fingerprint_kernel, dim3((unsigned)cfg->num_heads, kFpSplit), dim3(1024), 0, stream,
                     (const uint16_t*)q, (uint16_t*)qf, cos_table, sin_table, table_rows,
                     cfg->n_local, rows, cfg->num_heads, zero, zero2, zero3);
  return check_launch("fingerprint_kernel");
}

static int prefill_s_pad(int max_sel_len) { return (int)ceil_div(max_sel_len, kPfTile) * kPfTile; }

}  // namespace ts

using namespace ts;

extern "C" {

int ts_fingerprint(const ts_config* cfg, const void* q, int32_t rows, const float* cos_table,
                   const float* sin_table, int64_t table_rows, void* qf, ts_stream_t stream) {
  return launch_fingerprint(cfg, q, rows, cos_table, sin_table, table_rows, qf, ZeroRegion{},
                            ZeroRegion{}, (hipStream_t)stream);
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
  TS_REQUIRE(max_sel_len >= rows, TS_EINVAL,
             "max_sel_len %d < rows %d: a chunk attends at least to itself", max_sel_len, rows);
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const size_t need = ts_prefill_attn_workspace_bytes(cfg, max_sel_len);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= need, TS_EWORKSPACE,
             "ts_sparse_prefill_attn: workspace %zu bytes < required %zu", workspace_bytes, need);
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
  const dim3 grid((unsigned)ceil_div(rows, 16), (unsigned)cfg->num_kv_heads,
                  (unsigned)ceil_div(group, 4));
  const bool cap = cfg->logit_cap > 0.f;
#define TS_PF_LAUNCH(G_, C_)                                                                  \
  {                                                                                           \
    static const hipError_t lds_ok = hipFuncSetAttribute(                                     \
        (const void*)prefill_attn_kernel<G_, C_>, hipFuncAttributeMaxDynamicSharedMemorySize, \
        (int)kPfLdsBytes);                                                                    \
    if (lds_ok != hipSuccess) return fail(TS_EHIP, "prefill attention: %zu bytes of LDS refused", kPfLdsBytes); \
    hipLaunchKernelGGL((prefill_attn_kernel<G_, C_>), grid, dim3(512), kPfLdsBytes, st, a);   \
  }
#define TS_PF_CASE(G_)               \
  case G_:                           \
    if (cap) TS_PF_LAUNCH(G_, true)  \
    else TS_PF_LAUNCH(G_, false)     \
    break;
  switch (group) {
    TS_PF_CASE(1)
    TS_PF_CASE(2)
    TS_PF_CASE(4)
    TS_PF_CASE(7)
    TS_PF_CASE(8)
    default: return fail(TS_ESHAPE, "unsupported head group %d", group);
  }
#undef TS_PF_CASE
#undef TS_PF_LAUNCH
  return check_launch("prefill_attn_kernel");
}

}  // extern "C"
