// Sampling one token per logits row on the device (reference src/qwen25vl_lite/sampling.py:44-106):
// penalties over the tokens generated so far, then greedy argmax (temperature <= 0) or
// temperature, top-k, min-p, top-p and a draw from what is left.  One block of 1024 threads per
// row; all reductions run in a fixed order, so a row's token depends on nothing else in the batch.
//
// The draw inverts the distribution function with a uniform number u that the host supplies for
// the row: the token is the first index whose running probability mass exceeds u.
#include "common.h"

#define SAMPLE_THREADS 1024

struct RowParams {
  float temperature, top_p, min_p, u;
  float repetition, presence, frequency;
  int top_k;
  int prev_begin, prev_end;  // this row's generated tokens in prev_ids
};

__device__ __forceinline__ uint32_t order_key(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float block_reduce_sum(float v, float* red) { return block_sum(v, red); }

__device__ __forceinline__ float block_reduce_max(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = red[0];
    for (int i = 1; i < nwaves; ++i) t = fmaxf(t, red[i]);
    red[16] = t;
  }
  __syncthreads();
  return red[16];
}

// Largest key t such that the mass of {i : key(sc[i]) >= t} reaches `target`; mass of an entry
// is 1 (count_mode) or exp(sc[i] - mx).  0 if even all entries together do not reach it.
__device__ uint32_t threshold_search(const float* sc, int V, float mx, float target, bool count_mode, float* red) {
  uint32_t t = 0;
  for (int b = 31; b >= 0; --b) {
    const uint32_t cand = t | (1u << b);
    float part = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float s = sc[i];
      if (order_key(s) >= cand) part += count_mode ? 1.f : expf(s - mx);
    }
    if (block_reduce_sum(part, red) >= target) t = cand;
  }
  return t;
}

// A row's largest logit, found by ARGMAX_SPLITS blocks side by side (one block for a row of a
// hundred and fifty thousand logits is slower than the step's other kernels together): block s
// scans the logits s * per .. (s + 1) * per - 1 and leaves (value, index), the lowest index among
// equals; the row's block below picks among the splits, again the lowest index among equals.
#define ARGMAX_SPLITS 32
struct ArgmaxPart {
  float value;
  int index;
};

__global__ __launch_bounds__(256) void argmax_parts_kernel(const float* __restrict__ logits,
                                                            ArgmaxPart* __restrict__ parts, int V) {
  __shared__ float vals[4];
  __shared__ int idxs[4];
  const int m = blockIdx.y, s = blockIdx.x;
  const int per = (V + ARGMAX_SPLITS - 1) / ARGMAX_SPLITS;
  const int lo = s * per, hi = min(V, lo + per);
  const float* lg = logits + (size_t)m * V;
  float bv = -INFINITY;
  int bi = V;
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const float x = lg[i];
    if (x > bv) { bv = x; bi = i; }   // indices rise within a thread: the first of equals stays
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, QVL_WAVE);
    const int oi = __shfl_xor(bi, o, QVL_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if ((threadIdx.x & 63) == 0) { vals[threadIdx.x >> 6] = bv; idxs[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (vals[w] > bv || (vals[w] == bv && idxs[w] < bi)) { bv = vals[w]; bi = idxs[w]; }
    parts[(size_t)m * ARGMAX_SPLITS + s] = ArgmaxPart{bv, bi};
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits,
                                                                     float* __restrict__ scores,
                                                                     const RowParams* __restrict__ params,
                                                                     const int* __restrict__ prev_ids,
                                                                     const ArgmaxPart* __restrict__ parts,
                                                                     int* __restrict__ out, int V) {
  __shared__ float red[17];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ int pick_thread;
  __shared__ float pick_target;
  __shared__ int best_idx[17];

  const int m = blockIdx.x, tid = threadIdx.x;
  const RowParams p = params[m];
  const float* lg = logits + (size_t)m * V;
  float* sc = scores + (size_t)m * V;
  const int L = p.prev_end - p.prev_begin;
  const bool penal = L > 0 && (p.repetition != 1.f || p.presence != 0.f || p.frequency != 0.f);
  const bool greedy = p.temperature <= 0.f;

  const float* src = lg;
  if (penal || !greedy) {
    for (int i = tid; i < V; i += blockDim.x) sc[i] = lg[i];
    __syncthreads();
    src = sc;
  }
  if (penal) {
    const int* prev = prev_ids + p.prev_begin;
    for (int i = tid; i < L; i += blockDim.x) {
      const int t = prev[i];
      if (t < 0 || t >= V) continue;
      int count = 0;
      bool first = true;
      for (int j = 0; j < L; ++j)
        if (prev[j] == t) {
          ++count;
          if (j < i) first = false;
        }
      if (!first) continue;
      float s = sc[t];
      if (p.repetition != 1.f) s = s > 0.f ? s / p.repetition : s * p.repetition;
      s = s - p.presence - p.frequency * (float)count;
      sc[t] = s;
    }
    __syncthreads();
  }

  if (greedy && !penal && parts) {
    // the splits have scanned the row already
    if (tid < 64) {
      float bv = -INFINITY;
      int bi = V;
      if (tid < ARGMAX_SPLITS) { bv = parts[(size_t)m * ARGMAX_SPLITS + tid].value; bi = parts[(size_t)m * ARGMAX_SPLITS + tid].index; }
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, QVL_WAVE);
        const int oi = __shfl_xor(bi, o, QVL_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      if (tid == 0) out[m] = bi < V ? bi : 0;
    }
    return;
  }
  if (greedy) {
    // argmax, the lowest index among equals
    float bv = -INFINITY;
    int bi = V;
    for (int i = tid; i < V; i += blockDim.x) {
      const float s = src[i];
      if (s > bv || (s == bv && i < bi)) { bv = s; bi = i; }
    }
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, QVL_WAVE);
      const int oi = __shfl_xor(bi, o, QVL_WAVE);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const int lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    if (lane == 0) { red[wave] = bv; best_idx[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
      float v = red[0];
      int idx = best_idx[0];
      for (int w = 1; w < nwaves; ++w)
        if (red[w] > v || (red[w] == v && best_idx[w] < idx)) { v = red[w]; idx = best_idx[w]; }
      out[m] = idx < V ? idx : 0;
    }
    return;
  }

  for (int i = tid; i < V; i += blockDim.x) sc[i] = sc[i] / p.temperature;
  __syncthreads();

  if (p.top_k > 0 && p.top_k < V) {
    const uint32_t kth = threshold_search(sc, V, 0.f, (float)p.top_k, true, red);
    for (int i = tid; i < V; i += blockDim.x)
      if (order_key(sc[i]) < kth) sc[i] = -INFINITY;
    __syncthreads();
  }

  float part = -INFINITY;
  for (int i = tid; i < V; i += blockDim.x) part = fmaxf(part, sc[i]);
  const float mx = block_reduce_max(part, red);

  if (p.min_p > 0.f) {
    for (int i = tid; i < V; i += blockDim.x)
      if (expf(sc[i] - mx) < p.min_p) sc[i] = -INFINITY;
    __syncthreads();
  }

  if (p.top_p < 1.f) {
    float e = 0.f;
    for (int i = tid; i < V; i += blockDim.x) e += expf(sc[i] - mx);
    const float total = block_reduce_sum(e, red);
    const uint32_t cut = threshold_search(sc, V, mx, p.top_p * total, false, red);
    for (int i = tid; i < V; i += blockDim.x)
      if (order_key(sc[i]) < cut) sc[i] = -INFINITY;
    __syncthreads();
  }

  // draw: thread t owns the contiguous indices [t*C, (t+1)*C)
  const int C = (V + blockDim.x - 1) / blockDim.x;
  const int lo = tid * C, hi = min(V, lo + C);
  float mine = 0.f;
  for (int i = lo; i < hi; ++i) mine += expf(sc[i] - mx);
  sums[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float z = 0.f;
    for (int t = 0; t < (int)blockDim.x; ++t) z += sums[t];
    const float target = p.u * z;
    float acc = 0.f;
    int chosen = -1, last = 0;
    for (int t = 0; t < (int)blockDim.x; ++t) {
      if (sums[t] > 0.f) last = t;
      if (chosen < 0 && sums[t] > 0.f && acc + sums[t] > target) { chosen = t; pick_target = target - acc; }
      acc += sums[t];
    }
    if (chosen < 0) { chosen = last; pick_target = INFINITY; }
    pick_thread = chosen;
  }
  __syncthreads();
  if (tid == pick_thread) {
    float acc = 0.f;
    int token = -1, last = lo;
    for (int i = lo; i < hi; ++i) {
      const float e = expf(sc[i] - mx);
      if (e > 0.f) {
        last = i;
        acc += e;
        if (acc > pick_target) { token = i; break; }
      }
    }
    out[m] = token >= 0 ? token : last;
  }
}

// parts: null, or room for M * qvl_sample_argmax_part_bytes() bytes: then the rows' largest logits
// are found by several blocks each first (worth it when some row is greedy without penalties).
extern "C" int qvl_sample_rows(const void* logits, void* scores, const void* params, const void* prev_ids,
                               void* parts, void* out, int M, int V, hipStream_t stream) {
  if (M <= 0) return QVL_OK;
  if (V <= 0) return QVL_ERR_SHAPE;
  if (M > 65535) return QVL_ERR_LIMIT;
  if (parts) {
    hipLaunchKernelGGL(argmax_parts_kernel, dim3(ARGMAX_SPLITS, M), dim3(256), 0, stream, (const float*)logits,
                       (ArgmaxPart*)parts, V);
    if (hipGetLastError() != hipSuccess) return QVL_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(sample_rows_kernel, dim3(M), dim3(SAMPLE_THREADS), 0, stream, (const float*)logits,
                     (float*)scores, (const RowParams*)params, (const int*)prev_ids, (const ArgmaxPart*)parts,
                     (int*)out, V);
  return qvl_launch_status();
}

extern "C" int qvl_sample_argmax_part_bytes() { return (int)(ARGMAX_SPLITS * sizeof(ArgmaxPart)); }

extern "C" int qvl_sample_params_size() { return (int)sizeof(RowParams); }
