// Decode attention over the selected KV slots: the FlashInfer paged decode the
// reference calls at tr.py:815-823 (page size 1, in-kernel Llama RoPE).
//
// Split-K: grid (splits, Hkv, B).  A workgroup owns a contiguous range of the
// request's selected list for one KV head and keeps the G = H/Hkv query heads
// that read it in registers.  Sixteen lanes gather one K row and one V row
// (256 bytes each, 128-bit loads); sixteen such lane groups per workgroup walk
// the range with stride 16.  Keys are rotated to their index in the selected
// list, the query to S-1; softmax is online in fp32.  Partial (max, sum, acc)
// triples are merged first across the lane groups, then across splits by a
// second small kernel.
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
  int rope_mode;
  float rope_theta, rope_rcp_scale, sm_scale, logit_cap;
  int nsplit, max_sel_len;
  float* part_acc;  // [B,H,nsplit,128]
  float* part_ml;   // [B,H,nsplit,2]
  uint16_t* out;    // [B,H,128] bf16
};

__device__ __forceinline__ void unpack8(const uint4& w, float (&f)[8]) {
  f[0] = bf16_lo(w.x);
  f[1] = bf16_hi(w.x);
  f[2] = bf16_lo(w.y);
  f[3] = bf16_hi(w.y);
  f[4] = bf16_lo(w.z);
  f[5] = bf16_hi(w.z);
  f[6] = bf16_lo(w.w);
  f[7] = bf16_hi(w.w);
}

template <int G>
__global__ __launch_bounds__(256) void attn_split_kernel(AttnArgs a) {
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int S = min(max(a.sel_len[b], 0), a.max_sel_len);
  const int chunk = (S + a.nsplit - 1) / a.nsplit;
  const int lo = split * chunk;
  const int hi = min(S, lo + chunk);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lg = tid >> 4;   // lane group 0..15 inside the workgroup
  const int l16 = tid & 15;  // owns dims [8*l16, 8*l16+8)
  const bool upper = l16 >= 8;  // second half of the head dimension
  const int H = a.num_heads;
  const bool rope = a.rope_mode == TS_ROPE_LLAMA;

  // Frequencies of this lane's 8 rotation pairs (pair index = dim mod 64).
  float freq[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int pair = (l16 & 7) * 8 + e;
    freq[e] = a.rope_rcp_scale * powf(a.rope_theta, -2.0f * (float)pair / (float)kHeadDim);
  }

  // Query rows of the G heads, rotated to position S-1.
  float qv[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const uint16_t* qrow = a.q + ((size_t)b * H + (size_t)kvh * G + g) * kHeadDim;
    float mine[8], other[8];
    unpack8(*(const uint4*)(qrow + l16 * 8), mine);
    unpack8(*(const uint4*)(qrow + (l16 ^ 8) * 8), other);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (rope) {
        float sn, cs;
        sincosf((float)(S - 1) * freq[e], &sn, &cs);
        qv[g][e] = upper ? mine[e] * cs + other[e] * sn : mine[e] * cs - other[e] * sn;
      } else {
        qv[g][e] = mine[e];
      }
    }
  }

  // Key rotation state: angle of token j is j*freq; advance by 16 tokens per step.
  float kc[8], ks[8], dc[8], ds[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if (rope) {
      sincosf((float)(lo + lg) * freq[e], &ks[e], &kc[e]);
      sincosf(16.0f * freq[e], &ds[e], &dc[e]);
    } else {
      kc[e] = 1.f;
      ks[e] = 0.f;
      dc[e] = 1.f;
      ds[e] = 0.f;
    }
  }

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = kNegBig;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
  }

  const int32_t* sel = a.sel + (int64_t)b * a.sel_stride;
  const size_t row_elems = (size_t)a.num_kv_heads * kHeadDim;
  for (int j = lo + lg; j < hi; j += 16) {
    uint32_t slot = (uint32_t)sel[j];
    slot = slot < a.pool_rows ? slot : a.pool_rows - 1;
    const size_t at = (size_t)slot * row_elems + (size_t)kvh * kHeadDim + l16 * 8;
    const uint4 kraw = *(const uint4*)(a.k_pool + at);
    const uint4 vraw = *(const uint4*)(a.v_pool + at);
    float kf[8], vf[8];
    unpack8(kraw, kf);
    unpack8(vraw, vf);
    if (rope) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float partner = dpp_move<kRowRor8>(kf[e]);  // dim +-64 of the same token
        kf[e] = upper ? kf[e] * kc[e] + partner * ks[e] : kf[e] * kc[e] - partner * ks[e];
        const float c2 = kc[e] * dc[e] - ks[e] * ds[e];
        ks[e] = ks[e] * dc[e] + kc[e] * ds[e];
        kc[e] = c2;
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float p = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) p += qv[g][e] * kf[e];
      p = row16_sum(p) * a.sm_scale;
      if (a.logit_cap > 0.f) p = a.logit_cap * tanhf(p / a.logit_cap);
      const float mn = fmaxf(m[g], p);
      const float alpha = __expf(m[g] - mn);
      const float w = __expf(p - mn);
      l[g] = l[g] * alpha + w;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = acc[g][e] * alpha + w * vf[e];
      m[g] = mn;
    }
  }

  // Merge the four lane groups of a wave (rows of 16 lanes), then the four waves.
  __shared__ float sm_acc[4][G][kHeadDim];
  __shared__ float sm_m[4][G], sm_l[4][G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
      const float m2 = __shfl_xor(m[g], off), l2 = __shfl_xor(l[g], off);
      const float mn = fmaxf(m[g], m2);
      const float a1 = __expf(m[g] - mn), a2 = __expf(m2 - mn);
      l[g] = l[g] * a1 + l2 * a2;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = acc[g][e] * a1 + __shfl_xor(acc[g][e], off) * a2;
      m[g] = mn;
    }
    if (lane < 16) {
#pragma unroll
      for (int e = 0; e < 8; ++e) sm_acc[wave][g][l16 * 8 + e] = acc[g][e];
      if (lane == 0) {
        sm_m[wave][g] = m[g];
        sm_l[wave][g] = l[g];
      }
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * kHeadDim; idx += 256) {
    const int g = idx / kHeadDim, d = idx % kHeadDim;
    float mm = kNegBig;
#pragma unroll
    for (int w = 0; w < 4; ++w) mm = fmaxf(mm, sm_m[w][g]);
    float o = 0.f, ll = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float sc = __expf(sm_m[w][g] - mm);
      o += sm_acc[w][g][d] * sc;
      ll += sm_l[w][g] * sc;
    }
    const size_t ph = ((size_t)b * H + (size_t)kvh * G + g) * a.nsplit + split;
    a.part_acc[ph * kHeadDim + d] = o;
    if (d == 0) {
      a.part_ml[ph * 2] = mm;
      a.part_ml[ph * 2 + 1] = ll;
    }
  }
}

// out[b,h,:] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s, rounded to bf16.
__global__ __launch_bounds__(kHeadDim) void attn_merge_kernel(AttnArgs a) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const size_t ph = ((size_t)b * a.num_heads + h) * a.nsplit;
  float mm = kNegBig;
  for (int s = 0; s < a.nsplit; ++s) mm = fmaxf(mm, a.part_ml[(ph + s) * 2]);
  float o = 0.f, ll = 0.f;
  for (int s = 0; s < a.nsplit; ++s) {
    const float sc = __expf(a.part_ml[(ph + s) * 2] - mm);
    o += a.part_acc[(ph + s) * kHeadDim + d] * sc;
    ll += a.part_ml[(ph + s) * 2 + 1] * sc;
  }
  a.out[((size_t)b * a.num_heads + h) * kHeadDim + d] = f32_to_bf16(ll > 0.f ? o / ll : 0.f);
}

static int attn_splits(int batch, int num_kv_heads, int max_sel_len) {
  // About two workgroups per CU in total; at least 16 tokens per split.
  int64_t want = ceil_div(512, (int64_t)batch * num_kv_heads);
  int64_t cap = ceil_div(max_sel_len, 16);
  if (want > cap) want = cap;
  if (want < 1) want = 1;
  if (want > 256) want = 256;
  return (int)want;
}

}  // namespace ts

using namespace ts;

extern "C" {

size_t ts_attn_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_sel_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_sel_len < 1) return 0;
  const size_t ns = (size_t)attn_splits(batch, cfg->num_kv_heads, max_sel_len);
  const size_t heads = (size_t)batch * cfg->num_heads;
  return align_up(heads * ns * kHeadDim * 4, 256) + align_up(heads * ns * 2 * 4, 256);
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

  AttnArgs a;
  a.q = (const uint16_t*)q;
  a.k_pool = (const uint16_t*)k_pool;
  a.v_pool = (const uint16_t*)v_pool;
  a.pool_rows = (uint32_t)pool_rows;
  a.sel = sel;
  a.sel_stride = sel_stride;
  a.sel_len = sel_len;
  a.num_heads = cfg->num_heads;
  a.num_kv_heads = cfg->num_kv_heads;
  a.rope_mode = cfg->rope_mode;
  a.rope_theta = cfg->rope_theta;
  a.rope_rcp_scale = cfg->rope_mode == TS_ROPE_LLAMA ? 1.0f / cfg->rope_scale : 1.0f;
  a.sm_scale = cfg->sm_scale;
  a.logit_cap = cfg->logit_cap;
  a.nsplit = attn_splits(batch, cfg->num_kv_heads, max_sel_len);
  a.max_sel_len = max_sel_len;
  const size_t heads = (size_t)batch * cfg->num_heads;
  a.part_acc = (float*)workspace;
  a.part_ml = (float*)((char*)workspace + align_up(heads * a.nsplit * kHeadDim * 4, 256));
  a.out = (uint16_t*)out;

  const dim3 grid((unsigned)a.nsplit, (unsigned)cfg->num_kv_heads, (unsigned)batch);
  const int group = cfg->num_heads / cfg->num_kv_heads;
  hipStream_t st = (hipStream_t)stream;
  switch (group) {
    case 1: hipLaunchKernelGGL(attn_split_kernel<1>, grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL(attn_split_kernel<2>, grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL(attn_split_kernel<4>, grid, dim3(256), 0, st, a); break;
    case 7: hipLaunchKernelGGL(attn_split_kernel<7>, grid, dim3(256), 0, st, a); break;
    case 8: hipLaunchKernelGGL(attn_split_kernel<8>, grid, dim3(256), 0, st, a); break;
    default: return fail(TS_ESHAPE, "unsupported head group %d", group);
  }
  TS_TRY(check_launch("attn_split_kernel"));
  hipLaunchKernelGGL(attn_merge_kernel, dim3((unsigned)cfg->num_heads, (unsigned)batch),
                     dim3(kHeadDim), 0, st, a);
  return check_launch("attn_merge_kernel");
}

}  // extern "C"
