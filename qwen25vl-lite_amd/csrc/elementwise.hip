// Row-wise kernels of the decoder step: embedding gather, residual add + RMSNorm,
// rotation + cache write, SwiGLU.  Each works for float32 and bfloat16 storage and any
// row width; all arithmetic is float32.
#include "common.h"

// ---------------------------------------------------------------------------------------
// Embedding gather: out[n, :] = float32(table[ids[n], :])       (reference text.py:213)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_gather_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                    float* __restrict__ out, int H, int V) {
  const int n = blockIdx.x;
  int id = ids[n];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);  // ids are validated on the host; never read outside the table
  const T* row = table + (size_t)id * H;
  float* o = out + (size_t)n * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = ldf<T>(row + i);
}

extern "C" int qvl_embed_gather(const void* ids, const void* table, void* out, int N, int H, int V, int dtype,
                                hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (H <= 0 || V <= 0) return QVL_ERR_SHAPE;
  if (dtype == 0)
    hipLaunchKernelGGL(embed_gather_kernel<float>, dim3(N), dim3(256), 0, stream, (const int*)ids,
                       (const float*)table, (float*)out, H, V);
  else if (dtype == 1)
    hipLaunchKernelGGL(embed_gather_kernel<bf16_t>, dim3(N), dim3(256), 0, stream, (const int*)ids,
                       (const bf16_t*)table, (float*)out, H, V);
  else
    return QVL_ERR_DTYPE;
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Residual add + RMSNorm  (reference layers.py:27-31, text.py:196-205)
//   v = h[row] + delta[row]            (delta optional; the sum is float32; delta may come as
//                                       several slabs [slab][row], partial sums of a product cut
//                                       along its inner size, which are added in slab order)
//   h[row] = v                         (unless `rows` selects rows: then h is left alone)
//   out[m] = v * (1/sqrt(mean(v^2) + eps)) * w
// One block per row; the reduction order depends on H only, so a row's result does not
// depend on what else is in the batch.
// ---------------------------------------------------------------------------------------
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, const float* __restrict__ w,
                                   TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, int nslabs,
                                   long long slab_stride) {
  __shared__ float red[17];
  const int m = blockIdx.x;
  const int row = rows ? rows[m] : m;
  float* hr = h + (size_t)row * H;
  const TD* dr = delta ? delta + (size_t)row * H : nullptr;
  auto delta_at = [&](int i) {
    float d = ldf<TD>(dr + i);
    for (int c = 1; c < nslabs; ++c) d += ldf<TD>(dr + (size_t)c * slab_stride + i);
    return d;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = hr[i];
    if (dr) v += delta_at(i);
    ss += v * v;
    if (dr && !rows) hr[i] = v;
  }
  const float total = block_sum(ss, red);
  const float rs = 1.0f / sqrtf(total / (float)H + eps);
  TO* o = out + (size_t)m * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = hr[i];
    if (dr && rows) v += delta_at(i);
    stf<TO>(o + i, (v * rs) * w[i]);
  }
}

// The same with every value held in registers between the two passes: rows whose width is a
// multiple of 4 and at most NORM_VEC_MAX * 4 * 256, read and written 4 values at a time.
#define NORM_VEC_MAX 8

template <typename T> __device__ __forceinline__ float4 ld4(const T* p);
template <> __device__ __forceinline__ float4 ld4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 ld4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                __uint_as_float(v.y & 0xffff0000u)};
}
template <typename T> __device__ __forceinline__ void st4(T* p, float4 v);
template <> __device__ __forceinline__ void st4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void st4<bf16_t>(bf16_t* p, float4 v) {
  uint2 o;
  o.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
  o.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = o;
}

template <typename TD, typename TO>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                              const float* __restrict__ w, TO* __restrict__ out,
                                                              const int* __restrict__ rows, int H, float eps) {
  __shared__ float red[17];
  const int m = blockIdx.x;
  const int row = rows ? rows[m] : m;
  float* hr = h + (size_t)row * H;
  const TD* dr = delta ? delta + (size_t)row * H : nullptr;
  const int nvec = H >> 2;
  float4 v[NORM_VEC_MAX];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NORM_VEC_MAX; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < nvec) {
      float4 x = ld4<float>(hr + 4 * i);
      if (dr) {
        const float4 d = ld4<TD>(dr + 4 * i);
        x.x += d.x; x.y += d.y; x.z += d.z; x.w += d.w;
        if (!rows) st4<float>(hr + 4 * i, x);
      }
      v[j] = x;
      ss += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
  }
  const float rs = 1.0f / sqrtf(block_sum(ss, red) / (float)H + eps);
  TO* o = out + (size_t)m * H;
#pragma unroll
  for (int j = 0; j < NORM_VEC_MAX; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < nvec) {
      const float4 g = ld4<float>(w + 4 * i);
      st4<TO>(o + 4 * i, float4{(v[j].x * rs) * g.x, (v[j].y * rs) * g.y, (v[j].z * rs) * g.z, (v[j].w * rs) * g.w});
    }
  }
}

// The addend as slabs of partial sums (float32 [slab][row][H], H a multiple of 4 and at most
// SLAB_VEC_MAX * 4096): a block of 1024 threads per row, a thread per 4 neighbouring values, the
// slabs' loads asked for sixteen at a time (they do not depend on each other, only the sum has an
// order: slab 0, 1, 2, ...).
#define SLAB_VEC_MAX 2
template <typename TO>
__global__ __launch_bounds__(1024) void add_rmsnorm_slabs_kernel(float* __restrict__ h, const float* __restrict__ delta,
                                                                 const float* __restrict__ w, TO* __restrict__ out,
                                                                 const int* __restrict__ rows, int H, float eps,
                                                                 int nslabs, long long slab_stride) {
  __shared__ float red[17];
  const int m = blockIdx.x;
  const int row = rows ? rows[m] : m;
  float* hr = h + (size_t)row * H;
  const float* dr = delta + (size_t)row * H;
  const int nvec = H >> 2;
  float4 v[SLAB_VEC_MAX], g[SLAB_VEC_MAX];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < SLAB_VEC_MAX; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < nvec) {
      // everything the thread needs is asked for before anything is waited for: the row of h, the
      // norm's weights and up to 16 slabs
      float4 x = ld4<float>(hr + 4 * i);
      g[j] = ld4<float>(w + 4 * i);
      float4 d = {0.f, 0.f, 0.f, 0.f};
      for (int c0 = 0; c0 < nslabs; c0 += 16) {
        float4 e[16];
#pragma unroll
        for (int c = 0; c < 16; ++c)
          e[c] = c0 + c < nslabs ? ld4<float>(dr + (size_t)(c0 + c) * slab_stride + 4 * i) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 16; ++c) {
          if (c0 + c < nslabs) { d.x += e[c].x; d.y += e[c].y; d.z += e[c].z; d.w += e[c].w; }
        }
      }
      x.x += d.x; x.y += d.y; x.z += d.z; x.w += d.w;
      if (!rows) st4<float>(hr + 4 * i, x);
      v[j] = x;
      ss += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
  }
  const float rs = 1.0f / sqrtf(block_sum(ss, red) / (float)H + eps);
  TO* o = out + (size_t)m * H;
#pragma unroll
  for (int j = 0; j < SLAB_VEC_MAX; ++j) {
    const int i = threadIdx.x + 1024 * j;
    if (i < nvec)
      st4<TO>(o + 4 * i, float4{(v[j].x * rs) * g[j].x, (v[j].y * rs) * g[j].y, (v[j].z * rs) * g[j].z, (v[j].w * rs) * g[j].w});
  }
}

// delta: null, or nslabs slabs of [rows of h][H], slab_stride elements apart (nslabs 1: one addend).
extern "C" int qvl_add_rmsnorm(void* h, const void* delta, const void* w, void* out, const void* rows, int M, int H,
                               float eps, int delta_dtype, int out_dtype, int nslabs, long long slab_stride,
                               hipStream_t stream) {
  if (M <= 0) return QVL_OK;
  if (H <= 0 || nslabs < 1 || (nslabs > 1 && (slab_stride < H || slab_stride % 4))) return QVL_ERR_SHAPE;
  const int threads = H >= 2048 ? 512 : 256;
  const bool vec = H % 4 == 0 && H <= NORM_VEC_MAX * 4 * 256 && nslabs == 1;
  if (nslabs > 1 && delta && delta_dtype == 0 && H % 4 == 0 && H <= SLAB_VEC_MAX * 4096) {
    if (out_dtype == 0)
      hipLaunchKernelGGL((add_rmsnorm_slabs_kernel<float>), dim3(M), dim3(1024), 0, stream, (float*)h, (const float*)delta,
                         (const float*)w, (float*)out, (const int*)rows, H, eps, nslabs, slab_stride);
    else if (out_dtype == 1)
      hipLaunchKernelGGL((add_rmsnorm_slabs_kernel<bf16_t>), dim3(M), dim3(1024), 0, stream, (float*)h, (const float*)delta,
                         (const float*)w, (bf16_t*)out, (const int*)rows, H, eps, nslabs, slab_stride);
    else
      return QVL_ERR_DTYPE;
    return qvl_launch_status();
  }
#define QVL_NORM_CASE(DD, OD, TD, TO)                                                                              \
  if (delta_dtype == DD && out_dtype == OD) {                                                                      \
    if (vec)                                                                                                       \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TO>), dim3(M), dim3(256), 0, stream, (float*)h,               \
                         (const TD*)delta, (const float*)w, (TO*)out, (const int*)rows, H, eps);                   \
    else                                                                                                           \
      hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TO>), dim3(M), dim3(threads), 0, stream, (float*)h,               \
                         (const TD*)delta, (const float*)w, (TO*)out, (const int*)rows, H, eps, nslabs,            \
                         slab_stride);                                                                             \
    return qvl_launch_status();                                                                                    \
  }
  QVL_NORM_CASE(0, 0, float, float)
  QVL_NORM_CASE(0, 1, float, bf16_t)
  QVL_NORM_CASE(1, 1, bf16_t, bf16_t)
  QVL_NORM_CASE(1, 0, bf16_t, float)
#undef QVL_NORM_CASE
  return QVL_ERR_DTYPE;
}

// ---------------------------------------------------------------------------------------
// Rotation + cache write  (reference rope.py:48-96, cache.py:440-460)
// x[n] holds nq query heads, then nkv key heads, then nkv value heads, each hd wide.
// For frequency f < rot_half the angle is float32(pos[freq_row[f]][n]) * inv_freq[f]; the pair
// is (f, f + rot_half):  out[f] = x[f] c - x[f+rot_half] s,  out[f+rot_half] = x[f+rot_half] c + x[f] s.
// Channels from 2*rot_half on pass unrotated.  Queries go to q_out; keys (rotated) and values
// go into the page slot of the token: K as [page][kv head][slot][hd], V as [page][kv head][hd][slot].
// ---------------------------------------------------------------------------------------
template <typename TI, typename T>
__global__ void rope_kv_write_kernel(const TI* __restrict__ x, int x_stride, const float* __restrict__ bias,
                                     const int* __restrict__ pos, int pos_stride,
                                     const float* __restrict__ inv_freq, const int* __restrict__ freq_row,
                                     const float2* __restrict__ cs, const int* __restrict__ slot,
                                     T* __restrict__ q_out, T* __restrict__ kc, T* __restrict__ vc, int nq, int nkv,
                                     int hd, int rot_half, int ps) {
  const int n = blockIdx.x;
  const int hh = blockIdx.y;
  const TI* src = x + (size_t)n * x_stride + (size_t)hh * hd;
  const float* b = bias ? bias + (size_t)hh * hd : nullptr;
  if (hh >= nq + nkv) {  // value head: copy
    const int s = slot[n];
    if (s < 0) return;
    const int kvh = hh - nq - nkv;
    const size_t page = (size_t)(s / ps), off = (size_t)(s % ps);
    T* dst = vc + ((page * nkv + kvh) * hd) * ps + off;
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
      float v = ldf<TI>(src + d) + (b ? b[d] : 0.f);
      stf<T>(dst + (size_t)d * ps, v);
    }
    return;
  }
  T* dst;
  if (hh < nq) {
    dst = q_out + ((size_t)n * nq + hh) * hd;
  } else {
    const int s = slot[n];
    if (s < 0) return;
    const int kvh = hh - nq;
    const size_t page = (size_t)(s / ps), off = (size_t)(s % ps);
    dst = kc + ((page * nkv + kvh) * ps + off) * hd;
  }
  for (int f = threadIdx.x; f < rot_half; f += blockDim.x) {
    float x1 = ldf<TI>(src + f) + (b ? b[f] : 0.f);
    float x2 = ldf<TI>(src + f + rot_half) + (b ? b[f + rot_half] : 0.f);
    float c = 1.f, s = 0.f;
    if (cs) {  // the step's table of cosines and sines: every head and layer reads the same values
      const float2 v = cs[(size_t)n * rot_half + f];
      c = v.x;
      s = v.y;
    } else {
      const int row = freq_row[f];
      if (row >= 0) {
        const float ang = (float)pos[(size_t)row * pos_stride + n] * inv_freq[f];
        sincosf(ang, &s, &c);
      }
    }
    stf<T>(dst + f, x1 * c - x2 * s);
    stf<T>(dst + f + rot_half, x2 * c + x1 * s);
  }
  for (int d = 2 * rot_half + threadIdx.x; d < hd; d += blockDim.x)
    stf<T>(dst + d, ldf<TI>(src + d) + (b ? b[d] : 0.f));
}

// The same for float32 sums, bfloat16 outputs and the table of cosines and sines in hand, with
// all widths multiples of 4 (the prompt portions of a bfloat16 run): a block per token, a thread
// per 4 neighbouring channels, 16-byte loads and 8-byte stores.
// x may come as nslabs slabs, slab_stride elements apart (partial sums of a product cut along its inner
// size): they are added in slab order, then the bias.
__global__ __launch_bounds__(256) void rope_kv_write_wide_kernel(
    const float* __restrict__ x, int x_stride, const float* __restrict__ bias, const float2* __restrict__ cs,
    const int* __restrict__ slot, bf16_t* __restrict__ q_out, bf16_t* __restrict__ kc, bf16_t* __restrict__ vc, int nq,
    int nkv, int hd, int rot_half, int ps, int nslabs, long long slab_stride) {
  const int n = blockIdx.x;
  const float* src = x + (size_t)n * x_stride;
  auto sums = [&](int at) {
    float4 v = *reinterpret_cast<const float4*>(src + at);
    for (int c = 1; c < nslabs; ++c) {
      const float4 e = *reinterpret_cast<const float4*>(src + (size_t)c * slab_stride + at);
      v.x += e.x; v.y += e.y; v.z += e.z; v.w += e.w;
    }
    return v;
  };
  const int s = nkv ? slot[n] : -1;
  const size_t page = s >= 0 ? (size_t)(s / ps) : 0, off = s >= 0 ? (size_t)(s % ps) : 0;
  auto add_bias = [&](float4 v, int at) {
    if (bias) {
      const float4 b = *reinterpret_cast<const float4*>(bias + at);
      v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
    }
    return v;
  };
  auto pack4 = [](float4 v) {
    uint2 o;
    o.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    o.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    return o;
  };
  // rotated heads: items (head, 4 frequencies)
  const int per_head = rot_half / 4, rotated = (nq + nkv) * per_head;
  for (int it = threadIdx.x; it < rotated; it += blockDim.x) {
    const int hh = it / per_head, f = (it - hh * per_head) * 4;
    bf16_t* dst;
    if (hh < nq) {
      dst = q_out + ((size_t)n * nq + hh) * hd;
    } else {
      if (s < 0) continue;
      dst = kc + ((page * nkv + (hh - nq)) * ps + off) * hd;
    }
    const float4 x1 = add_bias(sums(hh * hd + f), hh * hd + f);
    const float4 x2 = add_bias(sums(hh * hd + f + rot_half), hh * hd + f + rot_half);
    const float4 c01 = *reinterpret_cast<const float4*>(cs + (size_t)n * rot_half + f);      // (c0, s0, c1, s1)
    const float4 c23 = *reinterpret_cast<const float4*>(cs + (size_t)n * rot_half + f + 2);
    const float4 lo = {x1.x * c01.x - x2.x * c01.y, x1.y * c01.z - x2.y * c01.w, x1.z * c23.x - x2.z * c23.y,
                       x1.w * c23.z - x2.w * c23.w};
    const float4 hi = {x2.x * c01.x + x1.x * c01.y, x2.y * c01.z + x1.y * c01.w, x2.z * c23.x + x1.z * c23.y,
                       x2.w * c23.z + x1.w * c23.w};
    *reinterpret_cast<uint2*>(dst + f) = pack4(lo);
    *reinterpret_cast<uint2*>(dst + f + rot_half) = pack4(hi);
  }
  // channels past the rotation, unrotated
  const int tail = (hd - 2 * rot_half) / 4;
  for (int it = threadIdx.x; it < (nq + nkv) * tail; it += blockDim.x) {
    const int hh = it / tail, d = 2 * rot_half + (it - hh * tail) * 4;
    bf16_t* dst;
    if (hh < nq) {
      dst = q_out + ((size_t)n * nq + hh) * hd;
    } else {
      if (s < 0) continue;
      dst = kc + ((page * nkv + (hh - nq)) * ps + off) * hd;
    }
    *reinterpret_cast<uint2*>(dst + d) = pack4(add_bias(sums(hh * hd + d), hh * hd + d));
  }
  // values: [page][kv head][channel][slot]
  if (s >= 0) {
    for (int it = threadIdx.x; it < nkv * (hd / 4); it += blockDim.x) {
      const int kvh = it / (hd / 4), d = (it - kvh * (hd / 4)) * 4, at = (nq + nkv + kvh) * hd + d;
      const float4 v = add_bias(sums(at), at);
      bf16_t* dst = vc + ((page * nkv + kvh) * hd + d) * ps + off;
      dst[0] = f32_to_bf16(v.x);
      dst[(size_t)ps] = f32_to_bf16(v.y);
      dst[(size_t)2 * ps] = f32_to_bf16(v.z);
      dst[(size_t)3 * ps] = f32_to_bf16(v.w);
    }
  }
}

// cs: null, or float32 [N, rot_half, 2] from qvl_rope_table (then pos, inv_freq and freq_row are not read).
// nslabs > 1: x is float32 slabs of partial sums, slab_stride elements apart; taken with float32 in,
// bfloat16 out, cs given and all widths multiples of 4 only (else QVL_ERR_SHAPE).
extern "C" int qvl_rope_kv_write(const void* x, int x_stride, const void* bias, const void* pos, int pos_stride,
                                 const void* inv_freq, const void* freq_row, const void* cs, const void* slot,
                                 void* q_out, void* kc,
                                 void* vc, int N, int nq, int nkv, int hd, int rot_half, int ps, int in_dtype,
                                 int dtype, int nslabs, long long slab_stride, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (nslabs < 1 || (nslabs > 1 && (slab_stride < (long long)(nq + 2 * nkv) * hd || slab_stride % 4))) return QVL_ERR_SHAPE;
  if (nq < 0 || nkv < 0 || nq + nkv == 0 || hd <= 0 || rot_half < 0 || 2 * rot_half > hd || ps <= 0)
    return QVL_ERR_SHAPE;
  if (x_stride < (nq + 2 * nkv) * hd) return QVL_ERR_SHAPE;
  if (nq + 2 * nkv > 65535) return QVL_ERR_LIMIT;
  if (in_dtype == 0 && dtype == 1 && cs && hd % 4 == 0 && rot_half % 4 == 0 && x_stride % 4 == 0 &&
      (((uintptr_t)x | (uintptr_t)bias | (uintptr_t)cs) & 15) == 0 && (((uintptr_t)q_out | (uintptr_t)kc) & 7) == 0) {
    hipLaunchKernelGGL(rope_kv_write_wide_kernel, dim3(N), dim3(256), 0, stream, (const float*)x, x_stride,
                       (const float*)bias, (const float2*)cs, (const int*)slot, (bf16_t*)q_out, (bf16_t*)kc,
                       (bf16_t*)vc, nq, nkv, hd, rot_half, ps, nslabs, slab_stride);
    return qvl_launch_status();
  }
  if (nslabs > 1) return QVL_ERR_SHAPE;
  const dim3 grid(N, nq + 2 * nkv);
#define QVL_ROPE_CASE(ID, OD, TI, T)                                                                               \
  if (in_dtype == ID && dtype == OD) {                                                                             \
    hipLaunchKernelGGL((rope_kv_write_kernel<TI, T>), grid, dim3(64), 0, stream, (const TI*)x, x_stride,           \
                       (const float*)bias, (const int*)pos, pos_stride, (const float*)inv_freq,                    \
                       (const int*)freq_row, (const float2*)cs, (const int*)slot, (T*)q_out, (T*)kc, (T*)vc, nq,   \
                       nkv, hd, rot_half, ps);                                                                     \
    return qvl_launch_status();                                                                                    \
  }
  QVL_ROPE_CASE(0, 0, float, float)
  QVL_ROPE_CASE(0, 1, float, bf16_t)
  QVL_ROPE_CASE(1, 1, bf16_t, bf16_t)
#undef QVL_ROPE_CASE
  return QVL_ERR_DTYPE;
}

// ---------------------------------------------------------------------------------------
// The rotation's cosines and sines of a step, for kernels that rotate without computing angles:
// out[n, f] = (cos, sin) of pos[freq_row[f], n] * inv_freq[f], or (1, 0) where freq_row[f] < 0.
// ---------------------------------------------------------------------------------------
__global__ void rope_table_kernel(const int* __restrict__ pos, int pos_stride, const float* __restrict__ inv_freq,
                                  const int* __restrict__ freq_row, float2* __restrict__ out, int rot_half) {
  const int n = blockIdx.x;
  for (int f = threadIdx.x; f < rot_half; f += blockDim.x) {
    const int row = freq_row[f];
    float c = 1.f, s = 0.f;
    if (row >= 0) sincosf((float)pos[(size_t)row * pos_stride + n] * inv_freq[f], &s, &c);
    out[(size_t)n * rot_half + f] = float2{c, s};
  }
}

extern "C" int qvl_rope_table(const void* pos, int pos_stride, const void* inv_freq, const void* freq_row, void* out,
                              int N, int rot_half, hipStream_t stream) {
  if (N <= 0 || rot_half <= 0) return QVL_OK;
  if (pos_stride < N) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(rope_table_kernel, dim3(N), dim3(64), 0, stream, (const int*)pos, pos_stride,
                     (const float*)inv_freq, (const int*)freq_row, (float2*)out, rot_half);
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// SwiGLU: out[n, i] = silu(gate[n, i]) * up[n, i],  silu(z) = z / (1 + exp(-z))  (reference text.py:66)
// x[n] holds gate and up: plain, gate in columns 0..I-1 and up in I..2I-1; grouped, alternating
// groups of 8 gate columns and 8 up columns (feature i: gate at 16 (i/8) + i%8, up 8 further),
// the layout that lets the product before it apply the activation to a 16-row tile by itself.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ x, T* __restrict__ out, int I, int grouped) {
  const int n = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= I) return;
  const T* row = x + (size_t)n * 2 * I;
  const int gc = grouped ? 16 * (i >> 3) + (i & 7) : i;
  const int uc = grouped ? gc + 8 : I + i;
  const float g = ldf<T>(row + gc), u = ldf<T>(row + uc);
  stf<T>(out + (size_t)n * I + i, (g / (1.0f + expf(-g))) * u);
}

// bfloat16 rows whose width is a multiple of 8: eight values per thread, 16-byte loads and stores.
__global__ __launch_bounds__(256) void swiglu_bf16x8_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ out,
                                                            int I, long long total8, int grouped) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int per_row = I >> 3;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total8;
       idx += (long long)gridDim.x * blockDim.x) {
    const long long n = idx / per_row;
    const int c = (int)(idx - n * per_row) << 3;
    const bf16_t* row = x + (size_t)n * 2 * I;
    const u32x4 gv = *reinterpret_cast<const u32x4*>(row + (grouped ? 2 * c : c));
    const u32x4 uv = *reinterpret_cast<const u32x4*>(row + (grouped ? 2 * c + 8 : I + c));
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g0 = __uint_as_float(gv[k] << 16), g1 = __uint_as_float(gv[k] & 0xffff0000u);
      const float u0 = __uint_as_float(uv[k] << 16), u1 = __uint_as_float(uv[k] & 0xffff0000u);
      const float a0 = (g0 / (1.0f + expf(-g0))) * u0, a1 = (g1 / (1.0f + expf(-g1))) * u1;
      o[k] = (uint32_t)f32_to_bf16(a0) | ((uint32_t)f32_to_bf16(a1) << 16);
    }
    *reinterpret_cast<u32x4*>(out + (size_t)n * I + c) = o;
  }
}

extern "C" int qvl_swiglu(const void* x, void* out, int N, int I, int dtype, int grouped, hipStream_t stream) {
  if (N <= 0) return QVL_OK;
  if (I <= 0 || (grouped && I % 8)) return QVL_ERR_SHAPE;
  if (N > 65535) return QVL_ERR_LIMIT;
  const dim3 grid((I + 255) / 256, N);
  if (dtype == 0)
    hipLaunchKernelGGL(swiglu_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, (float*)out, I, grouped);
  else if (dtype == 1 && I % 8 == 0 && (((uintptr_t)x | (uintptr_t)out) & 15) == 0) {
    const long long total8 = (long long)N * (I >> 3);
    long long blocks = (total8 + 255) / 256;
    blocks = blocks > 8192 ? 8192 : blocks;
    hipLaunchKernelGGL(swiglu_bf16x8_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const bf16_t*)x,
                       (bf16_t*)out, I, total8, grouped);
  } else if (dtype == 1)
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)x, (bf16_t*)out, I,
                       grouped);
  else
    return QVL_ERR_DTYPE;
  return qvl_launch_status();
}

// ---------------------------------------------------------------------------------------
// Page copy (reference cache.py:537-545): page src[i] -> page dst[i] in every layer of a cache
// tensor [layers, pages, page_bytes].  Used when a request is forked: whole pages are shared,
// the page being filled is copied.
// ---------------------------------------------------------------------------------------
__global__ void copy_pages_kernel(char* __restrict__ cache, size_t layer_bytes, int page_bytes,
                                  const int* __restrict__ src, const int* __restrict__ dst) {
  const int i = blockIdx.x, layer = blockIdx.y;
  const uint4* from = reinterpret_cast<const uint4*>(cache + layer * layer_bytes + (size_t)src[i] * page_bytes);
  uint4* to = reinterpret_cast<uint4*>(cache + layer * layer_bytes + (size_t)dst[i] * page_bytes);
  for (int c = threadIdx.x; c < page_bytes / 16; c += blockDim.x) to[c] = from[c];
}

extern "C" int qvl_copy_pages(void* cache, long long layer_bytes, int page_bytes, const void* src, const void* dst,
                              int n, int layers, hipStream_t stream) {
  if (n <= 0 || layers <= 0) return QVL_OK;
  if (page_bytes <= 0 || page_bytes % 16 || layer_bytes < page_bytes || ((uintptr_t)cache & 15)) return QVL_ERR_SHAPE;
  if (layers > 65535) return QVL_ERR_LIMIT;
  hipLaunchKernelGGL(copy_pages_kernel, dim3(n, layers), dim3(256), 0, stream, (char*)cache, (size_t)layer_bytes,
                     page_bytes, (const int*)src, (const int*)dst);
  return qvl_launch_status();
}
