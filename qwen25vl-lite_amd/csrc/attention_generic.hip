// Paged attention for any head size, float32 or bfloat16 storage, float32 arithmetic.
// One wave per (token, query head).  It serves prompt portions and decoded tokens alike: a
// token at sequence index p sees keys lo..p of its request, lo = max(0, p - window + 1) with
// a window, else 0 (reference attention.py:336-402 for the mask, text.py:78 for the scale).
// Keys are walked in blocks of 64 by absolute index, so a token's result does not depend on
// how its request was cut into steps or on what else is in the batch.
#include "common.h"

#define ATTN_MAX_HD 512

template <typename T>
__global__ void attn_generic_kernel(const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
                                    const int* __restrict__ block_table, int table_width,
                                    const int* __restrict__ token_req, const int* __restrict__ token_seqpos,
                                    T* __restrict__ out, int nh, int nkv, int hd, int ps, int window, float scale) {
  __shared__ float sq[ATTN_MAX_HD];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = token_req[n], p = token_seqpos[n];
  const int kvh = h / (nh / nkv);
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const T* qr = q + ((size_t)n * nh + h) * hd;
  for (int d = lane; d < hd; d += 64) sq[d] = ldf<T>(qr + d);
  __syncthreads();
  const int* bt = block_table + (size_t)r * table_width;

  float m = -INFINITY, l = 0.f;
  float acc[ATTN_MAX_HD / 64];
#pragma unroll
  for (int i = 0; i < ATTN_MAX_HD / 64; ++i) acc[i] = 0.f;

  for (int c = lo / 64; c * 64 <= p; ++c) {
    const int j = c * 64 + lane;
    const bool valid = j >= lo && j <= p;
    float s = -INFINITY;
    if (valid) {
      const int pk = bt[j / ps];
      const size_t page = (size_t)(pk < 0 ? 0 : pk);   // a table without this page: read page 0, never out of bounds
      const T* kr = kc + ((page * nkv + kvh) * ps + (size_t)(j % ps)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot += sq[d] * ldf<T>(kr + d);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // m = -inf at first: alpha = 0
    l = l * alpha + wave_sum(pj);
#pragma unroll
    for (int i = 0; i < ATTN_MAX_HD / 64; ++i) acc[i] *= alpha;
    const int jend = (p - c * 64 < 63) ? p - c * 64 : 63;
    for (int jj = 0; jj <= jend; ++jj) {
      const float pv = __shfl(pj, jj, QVL_WAVE);
      const int ja = c * 64 + jj;
      if (ja < lo) continue;
      const int pv_page = bt[ja / ps];
      const size_t page = (size_t)(pv_page < 0 ? 0 : pv_page);
      const T* vr = vc + ((page * nkv + kvh) * hd) * ps + (size_t)(ja % ps);
#pragma unroll
      for (int i = 0; i < ATTN_MAX_HD / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < hd) acc[i] += pv * ldf<T>(vr + (size_t)d * ps);
      }
    }
    m = m_new;
  }
  T* o = out + ((size_t)n * nh + h) * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < ATTN_MAX_HD / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < hd) stf<T>(o + d, acc[i] * inv);
  }
}

extern "C" int qvl_attn_generic(const void* q, const void* kc, const void* vc, const void* block_table,
                                int table_width, const void* token_req, const void* token_seqpos, void* out, int N,
                                int nh, int nkv, int hd, int ps, int window, float scale, int dtype,
                                hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (nh <= 0 || nkv <= 0 || nh % nkv || hd <= 0 || ps <= 0 || table_width <= 0) return QVL_ERR_SHAPE;
  if (hd > ATTN_MAX_HD || nh > 65535) return QVL_ERR_LIMIT;
  const dim3 grid(N, nh);
  if (dtype == 0)
    hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(64), 0, stream, (const float*)q, (const float*)kc,
                       (const float*)vc, (const int*)block_table, table_width, (const int*)token_req,
                       (const int*)token_seqpos, (float*)out, nh, nkv, hd, ps, window, scale);
  else if (dtype == 1)
    hipLaunchKernelGGL(attn_generic_kernel<bf16_t>, grid, dim3(64), 0, stream, (const bf16_t*)q, (const bf16_t*)kc,
                       (const bf16_t*)vc, (const int*)block_table, table_width, (const int*)token_req,
                       (const int*)token_seqpos, (bf16_t*)out, nh, nkv, hd, ps, window, scale);
  else
    return QVL_ERR_DTYPE;
  return qvl_launch_status();
}
