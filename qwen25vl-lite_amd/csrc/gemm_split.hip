// Products with 17 to 64 rows whose rows one compute unit cannot hold for all of K:
// out[c][M, N] = partial sums of X[M, K] . W[N, K]^T over chunk c of K, bfloat16 operands, float32
// sums.  The slabs out[c] are added by whoever reads them (the norm that follows), in chunk order.
//
// The resident kernel (gemm_resident.hip) keeps the rows of X in the registers of a block's 16
// waves, each wave its own 256 columns of K, and streams row tiles of W past them: that is the
// form that reads W at the device's rate.  Registers hold 16 rows that way, not 64.  Here a wave
// keeps 128 columns instead, of up to 64 rows (four column tiles of the matrix instruction: 64
// registers), so a block covers a chunk of 2,048 columns of K and the grid is chunks of K times
// ranges of W's tiles.  Everything else is the resident kernel's way: a tile's 16 rows of W are
// split among the waves along K, every W fragment that is loaded is multiplied with all column
// tiles, two half-tile buffers of W go round, the waves' sums meet in LDS and are added in wave
// order, every load goes through a buffer descriptor (a lane with nothing to load asks past the
// end and gets zeros: no load inside a branch, exact wait counts).
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

#define PAST_END 0xffffff00u
#define BUFFER_LIMIT 0xffffff00ull
#define HOLD_ORDER() __builtin_amdgcn_sched_barrier(0)   // nothing is scheduled across this point

#define SW 16                   // waves per block
#define SK 4                    // 32-wide K steps per wave (8 was measured too: 31 us against 27 for the 7B down projection at 8 rows;
                                // a block's first tile is twice as long on its way, and a block has half as many tiles to hide that behind)
#define CHUNK_K (SW * SK * 32)  // the most columns of K a block covers

struct SplitArgs {
  const bf16_t* X;   // [M, K]
  int ldx;
  const bf16_t* W;   // [N, K]
  int ldw;
  float* out;        // [chunks][M][N]
  int M, N, K;
  int chunks, chunk_k;      // chunk c covers columns c * chunk_k ... of K (chunk_k a multiple of 32, at most CHUNK_K)
  int per_chunk;            // blocks per chunk: the grid is chunks * per_chunk
  int rows, ntiles;         // rows of W per tile (at most 16) and tiles of all of W
};

__device__ __forceinline__ rsrc_t buffer_of(const void* p, unsigned long long bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(uint32_t)bytes, 0x00020000);
}
__device__ __forceinline__ bf16x8_t load16(rsrc_t r, uint32_t byte_offset, int fixed) {
  return __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, fixed, 0));
}

template <int MT>
__global__ __launch_bounds__(64 * SW) void gemm_split_kernel(SplitArgs p) {
  constexpr int COLS = 16 * MT;
  // a tile's sums of every wave: two buffers, so that a tile's sums are read while the next tile's are written
  __shared__ __attribute__((aligned(16))) float red[2][SW][16 * COLS];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int chunk = blockIdx.x / p.per_chunk, first = blockIdx.x - chunk * p.per_chunk;
  const int k_base = chunk * p.chunk_k;
  const int k_len = p.K - k_base < p.chunk_k ? p.K - k_base : p.chunk_k;   // columns of this chunk
  const int k_lane = wave * SK * 32 + 8 * lg;                              // this lane's first column within the chunk
  const int inside = (k_len - k_lane + 31) >> 5;                           // how many of its steps begin inside the chunk
  const rsrc_t w_buf = buffer_of(p.W, ((unsigned long long)(p.N - 1) * p.ldw + p.K) * 2);
  const rsrc_t x_buf = buffer_of(p.X, ((unsigned long long)(p.M - 1) * p.ldx + p.K) * 2);

  // half h (steps 2h, 2h + 1) of a tile's W operand; a tile beyond the last asks past the end
  auto load_w_half = [&](int tile, int h, bf16x8_t* a) {
    const int row = tile * p.rows + r;
    const bool row_ok = tile < p.ntiles && r < p.rows && row < p.N;
    const uint32_t at = row_ok ? ((uint32_t)row * p.ldw + k_base + k_lane) * 2 : PAST_END;
#pragma unroll
    for (int i = 0; i < SK / 2; ++i) {
      const int u = h * (SK / 2) + i;
      a[i] = load16(w_buf, u < inside ? at : PAST_END, u * 64);
    }
  };
  bf16x8_t w[2][SK / 2];
  int tile = first;
  load_w_half(tile, 0, w[0]);   // W first: it is the long wait
  load_w_half(tile, 1, w[1]);
  // the block's chunk of every row of X: column tile t holds rows 16 t .. 16 t + 15
  bf16x8_t xb[MT][SK];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = 16 * t + r;
    const uint32_t at = row < p.M ? ((uint32_t)row * p.ldx + k_base + k_lane) * 2 : PAST_END;
#pragma unroll
    for (int u = 0; u < SK; ++u) xb[t][u] = load16(x_buf, u < inside ? at : PAST_END, u * 64);
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float* slab = p.out + (size_t)chunk * p.M * p.N;
  int parity = 0;
  while (tile < p.ntiles) {
    const int next = tile + p.per_chunk;
    HOLD_ORDER();
#pragma unroll
    for (int i = 0; i < SK / 2; ++i)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[0][i], xb[t][i], acc[t], 0, 0, 0);
    HOLD_ORDER();
    load_w_half(next, 0, w[0]);   // each half is asked for again the moment it is multiplied
    HOLD_ORDER();
#pragma unroll
    for (int i = 0; i < SK / 2; ++i)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[1][i], xb[t][SK / 2 + i], acc[t], 0, 0, 0);
    HOLD_ORDER();
    load_w_half(next, 1, w[1]);
    HOLD_ORDER();
    // merge the waves' sums: a wave's lie as [row of X][row of the tile], a lane writes its four at
    // once, and the thread that finishes element e = 16 m + nl reads word e of every wave, in wave order
    float (*buf)[16 * COLS] = red[parity];
    parity ^= 1;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      *reinterpret_cast<f32x4_t*>(&buf[wave][(16 * t + r) * 16 + 4 * lg]) = acc[t];
      acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();
    if (threadIdx.x < 16 * COLS) {
      const int e = threadIdx.x, m = e >> 4, nl = e & 15, n = tile * p.rows + nl;
      float sum = 0.f;
#pragma unroll
      for (int v = 0; v < SW; ++v) sum += buf[v][e];
      if (m < p.M && nl < p.rows && n < p.N) slab[(size_t)m * p.N + n] = sum;
    }
    tile = next;
  }
}

// How a product is cut on a device with `cus` compute units: chunks of K (as few as fit a block, all of
// one length in whole steps of 32), blocks per chunk, and rows per tile such that the tiles divide evenly.
struct Cut {
  int chunks, chunk_k, per_chunk, rows, ntiles;
};
static Cut cut_for(int N, int K, int cus) {
  Cut c;
  c.chunks = (K + CHUNK_K - 1) / CHUNK_K;
  if (c.chunks > cus) c.chunks = cus;
  c.chunk_k = ((K + c.chunks - 1) / c.chunks + 31) / 32 * 32;
  c.per_chunk = cus / c.chunks;
  if (c.per_chunk < 1) c.per_chunk = 1;
  const long long per_round = 16LL * c.per_chunk, rounds = (N + per_round - 1) / per_round;
  c.rows = (int)((N + rounds * c.per_chunk - 1) / (rounds * c.per_chunk));
  c.ntiles = (N + c.rows - 1) / c.rows;
  if (c.per_chunk > c.ntiles) c.per_chunk = c.ntiles;
  return c;
}

// Whether qvl_gemm_split takes these sizes, and how many slabs it then writes (0: it does not).
extern "C" int qvl_gemm_split_chunks(int M, int N, int K, int cus) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || K % 8 || cus <= 0) return 0;
  const Cut c = cut_for(N, K, cus);
  if ((long long)c.chunks * c.chunk_k < K || c.chunk_k > CHUNK_K) return 0;   // more chunks than compute units
  return c.chunks;
}

// x: bfloat16 [M, K] (ldx elements a row).  W: bfloat16 [N, K].  out: float32 [chunks][M][N], chunks =
// qvl_gemm_split_chunks(M, N, K, cus); the product is the sum of the slabs.  M at most 64, K a multiple of 8.
extern "C" int qvl_gemm_split(const void* x, int ldx, const void* W, int ldw, void* out, int M, int N, int K, int cus,
                              hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 64) return QVL_ERR_LIMIT;
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || ldx % 8 || ldx < K || cus <= 0 || !x || !W || !out) return QVL_ERR_SHAPE;
  if (((unsigned long long)(N - 1) * ldw + K) * 2 >= BUFFER_LIMIT || ((unsigned long long)(M - 1) * ldx + K) * 2 >= BUFFER_LIMIT)
    return QVL_ERR_LIMIT;
  if (qvl_gemm_split_chunks(M, N, K, cus) == 0) return QVL_ERR_LIMIT;
  const Cut c = cut_for(N, K, cus);
  SplitArgs p;
  p.X = (const bf16_t*)x; p.ldx = ldx; p.W = (const bf16_t*)W; p.ldw = ldw; p.out = (float*)out;
  p.M = M; p.N = N; p.K = K; p.chunks = c.chunks; p.chunk_k = c.chunk_k; p.per_chunk = c.per_chunk;
  p.rows = c.rows; p.ntiles = c.ntiles;
  const dim3 grid(c.chunks * c.per_chunk), block(64 * SW);
  if (M <= 16) hipLaunchKernelGGL(gemm_split_kernel<1>, grid, block, 0, stream, p);
  else if (M <= 32) hipLaunchKernelGGL(gemm_split_kernel<2>, grid, block, 0, stream, p);
  else if (M <= 48) hipLaunchKernelGGL(gemm_split_kernel<3>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(gemm_split_kernel<4>, grid, block, 0, stream, p);
  return qvl_launch_status();
}
