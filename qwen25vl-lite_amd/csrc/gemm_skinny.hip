// Products with few rows (decode): out[M, N] = X[M, K] . W[N, K]^T (+ bias), bfloat16 operands,
// float32 accumulation, float32 or bfloat16 output, M <= 64.
//
// The step is bound by reading W once from HBM, so W is the streamed operand: a block owns 16
// rows of W (16 outputs) and its waves split K into contiguous ranges; every lane keeps several
// 16-byte loads of W in flight.  W rows are the A operand of v_mfma_f32_16x16x32_bf16 and the
// rows of X (up to 16 per column tile) its B operand, read straight from L2, where the few rows of
// X stay.  The waves' partial sums meet in LDS and are added in wave order, so the result does
// not depend on timing.  Rows of X beyond M and rows of W beyond N are fed as zeros.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define NW 8      // waves per block
#define UNROLL 4  // 32-wide K steps in flight per wave

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(p));
}
__device__ __forceinline__ bf16x8_t zero8() {
  u32x4_t z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8_t, z);
}

template <int MT, typename TO>
__global__ __launch_bounds__(64 * NW) void gemm_skinny_kernel(const bf16_t* __restrict__ X, int ldx,
                                                              const bf16_t* __restrict__ W, int ldw,
                                                              const float* __restrict__ bias, TO* __restrict__ out,
                                                              int ldo, int M, int N, int K) {
  __shared__ float red[NW][MT][256];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int n0 = blockIdx.x * 16;
  const bool row_ok = n0 + r < N;
  const bf16_t* wrow = W + (size_t)(row_ok ? n0 + r : 0) * ldw;
  const bf16_t* xrow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    m_ok[mt] = mt * 16 + r < M;
    xrow[mt] = X + (size_t)(m_ok[mt] ? mt * 16 + r : 0) * ldx;
  }
  const int ksteps = (K + 31) / 32;
  const int per = (ksteps + NW - 1) / NW;
  const int ks0 = wave * per;
  const int ks1 = ks0 + per < ksteps ? ks0 + per : ksteps;
  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  for (int ks = ks0; ks < ks1; ks += UNROLL) {
    bf16x8_t a[UNROLL], b[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = (ks + u) * 32 + 8 * lg;
      const bool ok = ks + u < ks1 && k < K;
      a[u] = (ok && row_ok) ? load8(wrow + k) : zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = (ok && m_ok[mt]) ? load8(xrow[mt] + k) : zero8();
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mt], acc[mt], 0, 0, 0);
  }
  // lane holds out^T[n = 4*lg + i][m = r] of each column tile
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][mt][(4 * lg + i) * 16 + r] = acc[mt][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
    const int mt = idx >> 8, e = idx & 255;
    const int m = mt * 16 + (e >> 4), n = n0 + (e & 15);
    if (m >= M || n >= N) continue;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += red[w][mt][(e & 15) * 16 + (e >> 4)];
    if (bias) sum += bias[n];
    stf<TO>(out + (size_t)m * ldo + n, sum);
  }
}

template <typename TO>
static int launch(const void* X, int ldx, const void* W, int ldw, const void* bias, void* out, int ldo, int M, int N,
                  int K, hipStream_t stream) {
  const dim3 grid((N + 15) / 16), block(64 * NW);
#define QVL_SKINNY(MT)                                                                                            \
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, TO>), grid, block, 0, stream, (const bf16_t*)X, ldx, (const bf16_t*)W, \
                     ldw, (const float*)bias, (TO*)out, ldo, M, N, K)
  if (M <= 16) QVL_SKINNY(1);
  else if (M <= 32) QVL_SKINNY(2);
  else QVL_SKINNY(4);
#undef QVL_SKINNY
  return qvl_launch_status();
}

extern "C" int qvl_gemm_skinny(const void* X, int ldx, const void* W, int ldw, const void* bias, void* out, int ldo,
                               int M, int N, int K, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 64) return QVL_ERR_LIMIT;
  if (K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo < N) return QVL_ERR_SHAPE;
  if (out_dtype == 0) return launch<float>(X, ldx, W, ldw, bias, out, ldo, M, N, K, stream);
  if (out_dtype == 1) return launch<bf16_t>(X, ldx, W, ldw, bias, out, ldo, M, N, K, stream);
  return QVL_ERR_DTYPE;
}
