// Products with 17 to 64 rows whose rows do not fit a compute unit whole: out[c][M, N] = partial
// sums of X[M, K] . W[N, K]^T over chunk c of K, bfloat16 operands, float32 sums.
//
// With up to 32 rows the resident kernel keeps all of X in one compute unit (registers and LDS)
// while W streams by.  64 rows of a 3584-wide X are 459 KB: more than a compute unit holds.  Here
// K is cut into chunks that do fit: a block owns one chunk of K (at most 1248 wide) and a range of
// W's rows.  It puts its chunk of all rows of X into LDS once, and then each of its 16 waves
// streams the chunk's part of its own rows of W (tiles of at most 16 rows, one wave one tile,
// v_mfma_f32_16x16x32_bf16 with the X operand read from LDS), through a ring of 8 loads in
// flight per wave.  No wave waits for another after the fill: no sums are merged inside the
// block, and X costs L2 no more than W costs HBM.  What is left is the sum over the chunks: every
// block writes its partial sums as a slab of their own, out[chunk][M][N] in float32, and whoever
// reads the result adds the slabs in chunk order (the norm that follows), so
// the result does not depend on which block finished first.
//
// The fill can apply the feed-forward's activation on the way (X = silu(gate) * up from the
// grouped gate | up product), which saves that kernel's launch.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define CW 16            // waves per block
#define RING 8          // W loads in flight per wave
#define MAX_STEPS 39     // 32-wide steps of a chunk: 64 rows of (39 * 64 + 16) bytes are 160,768 bytes of LDS
#define ROW16 (MAX_STEPS * 4 + 1)   // 16-byte units of a row of X in LDS (one of padding: no bank conflicts)

struct ChunkedArgs {
  const bf16_t* X;   // [M, K], or with `swiglu` the grouped gate | up product [M, 2 K]
  int ldx;
  const bf16_t* W;   // [N, K]
  int ldw;
  float* out;        // [chunks][M][N]
  int M, N, K;
  int chunks, ranges;   // grid = chunks * ranges
  int tile_rows;        // rows of W per wave tile, 1..16
  int swiglu;
};

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(p));
}
__device__ __forceinline__ u32x4_t zero16() { return u32x4_t{0u, 0u, 0u, 0u}; }
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  bf16x2_t v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float lo16(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi16(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float silu_mul(float g, float u) {
  // the value the activation kernel stores: silu(g) * u rounded once (reference text.py:66)
  return (g / (1.0f + expf(-g))) * u;
}

template <int MT>
__global__ __launch_bounds__(64 * CW) void gemm_chunked_kernel(ChunkedArgs p) {
  __shared__ u32x4_t xs[16 * MT * ROW16];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int chunk = blockIdx.x / p.ranges, range = blockIdx.x - chunk * p.ranges;
  // chunk: steps [s0, s1) of the ceil(K / 32) steps, as even as they divide
  const int steps_all = (p.K + 31) >> 5;
  const int s0 = (int)((long long)chunk * steps_all / p.chunks), s1 = (int)((long long)(chunk + 1) * steps_all / p.chunks);
  const int steps = s1 - s0, k0 = s0 << 5;
  // range: rows [n_begin, n_end) of W, as even as they divide
  const int n_begin = (int)((long long)range * p.N / p.ranges), n_end = (int)((long long)(range + 1) * p.N / p.ranges);

  // ---- every wave its own tiles of W; the first tile's loads are asked for before X is ---------
  const int nr = p.tile_rows;
  const int tiles = (n_end - n_begin + nr - 1) / nr;
  int n0 = 0, rows_here = 0;
  bool row_ok = false;
  const bf16_t* wrow = p.W;
  auto set_tile = [&](int tile) {
    n0 = n_begin + tile * nr;
    rows_here = min(nr, n_end - n0);
    row_ok = r < rows_here;
    wrow = p.W + (size_t)(row_ok ? n0 + r : n0) * p.ldw + k0 + 8 * lg;
  };
  // Step s of the tile's W operand.  Every lane always loads from a valid address, with no branch
  // around the load and no use of the value before its step comes (the compiler then counts the
  // loads in flight exactly and each step waits for its own load only): a step past the chunk's
  // end reads the last step again, a lane past the tile's rows reads the tile's first row (its
  // sums are never stored), and in the last step of K a lane past K reads the last 8 values of
  // its row instead, which meet zeros of X.
  const int k_last = k0 + 32 * (steps - 1) + 8 * lg;
  const int last_back = k_last < p.K ? 0 : k_last - (p.K - 8);
  auto load_w = [&](int s) {
    s = s < steps ? s : steps - 1;
    return load8(wrow + 32 * s - (s == steps - 1 ? last_back : 0));
  };
  bf16x8_t ring[RING];
  auto prime = [&]() {
#pragma unroll
    for (int j = 0; j < RING; ++j) ring[j] = load_w(j);
  };
  if (wave < tiles) {
    set_tile(wave);
    prime();
  }

  // ---- this chunk of every row of X into LDS, four 16-byte units a thread in flight --------------
  const int units = steps * 4;   // 16-byte units of a row
  const int total = 16 * MT * units;
  auto fetch = [&](int idx) {
    const int row = idx / units, u = idx - row * units, k = k0 + 8 * u;
    u32x4_t v = zero16();
    if (idx < total && row < p.M && k < p.K) {
      if (!p.swiglu) {
        v = *reinterpret_cast<const u32x4_t*>(p.X + (size_t)row * p.ldx + k);
      } else {   // features k .. k + 7: gate at columns 2 k .. 2 k + 7, up at the 8 after them
        const u32x4_t g = *reinterpret_cast<const u32x4_t*>(p.X + (size_t)row * p.ldx + 2 * k);
        const u32x4_t up = *reinterpret_cast<const u32x4_t*>(p.X + (size_t)row * p.ldx + 2 * k + 8);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          v[j] = pack2(silu_mul(lo16(g[j]), lo16(up[j])), silu_mul(hi16(g[j]), hi16(up[j])));
      }
    }
    return v;
  };
  for (int base = threadIdx.x; base < total; base += 4 * blockDim.x) {
    u32x4_t v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = fetch(base + j * blockDim.x);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int idx = base + j * blockDim.x;
      if (idx < total) {
        const int row = idx / units;
        xs[row * ROW16 + (idx - row * units)] = v[j];
      }
    }
  }
  __syncthreads();

  for (int tile = wave; tile < tiles; tile += CW) {
    if (tile != wave) {
      set_tile(tile);
      prime();
    }
    f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int whole = steps / RING;   // rounds of RING steps, each of which asks for the round after it
    for (int round = 0; round < whole; ++round) {
#pragma unroll
      for (int j = 0; j < RING; ++j) {
        const int s = round * RING + j;
        const bf16x8_t a = ring[j];
        ring[j] = load_w(s + RING);
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              a, __builtin_bit_cast(bf16x8_t, xs[(16 * t + r) * ROW16 + 4 * s + lg]), acc[t], 0, 0, 0);
      }
    }
    const int left = steps - whole * RING;   // the same for the whole wave; their loads are in the ring
#pragma unroll
    for (int j = 0; j < RING; ++j) {
      if (j < left) {
        const int s = whole * RING + j;
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              ring[j], __builtin_bit_cast(bf16x8_t, xs[(16 * t + r) * ROW16 + 4 * s + lg]), acc[t], 0, 0, 0);
      }
    }
    // lane (r, lg) holds the sums of row 16 t + r of X with rows n0 + 4 lg .. + 3 of W
    float* slab = p.out + (size_t)chunk * p.M * p.N;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = 16 * t + r;
      if (m < p.M) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (4 * lg + v < rows_here) slab[(size_t)m * p.N + n0 + 4 * lg + v] = acc[t][v];
      }
    }
  }
}

// How a product of these sizes is cut on a device with `cus` compute units: chunks of K (each at
// most MAX_STEPS steps), ranges of W's rows per chunk, rows per wave tile.  More chunks than K
// needs give a small W more blocks to stream it; the cut whose busiest wave has the least to do
// wins, fewer chunks on a tie (every chunk is another slab to write and to add).
struct Cut {
  int chunks, ranges, tile_rows;
};
static Cut cut_for(int N, int K, int cus) {
  const int steps_all = (K + 31) / 32;
  const int least = (steps_all + MAX_STEPS - 1) / MAX_STEPS;
  Cut best{least, 1, 16};
  double best_cost = 1e300;
  for (int chunks = least; chunks <= steps_all && chunks <= cus && chunks <= 4 * least + 16; ++chunks) {
    const int ranges = cus / chunks > N ? N : cus / chunks;
    if (ranges <= 0) break;
    const int rows = (N + ranges - 1) / ranges;                    // rows of the largest range
    const int per_wave = (rows + CW - 1) / CW;                     // rows of the busiest wave
    const int tiles = (per_wave + 15) / 16;                        // its tiles
    const int tile_rows = (per_wave + tiles - 1) / tiles;
    const int steps = (steps_all + chunks - 1) / chunks;
    // a wave's time: its loads (a load instruction moves at most 16 rows; fewer rows, the same instruction)
    // plus the fill of X, plus the slab it writes and somebody reads again
    const double cost = (double)tiles * steps * (tile_rows < 4 ? 4 : tile_rows) / 16.0 + 0.02 * steps + 0.15 * chunks;
    if (cost < best_cost - 1e-9) {
      best_cost = cost;
      best = Cut{chunks, ranges, tile_rows};
    }
  }
  return best;
}

// The number of slabs qvl_gemm_chunked writes for these sizes: out must hold chunks * M * N floats.
extern "C" int qvl_gemm_chunked_chunks(int N, int K, int cus) {
  if (N <= 0 || K <= 0 || cus <= 0) return 0;
  return cut_for(N, K, cus).chunks;
}

// x: bfloat16 [M, K] (ldx elements a row), or with swiglu != 0 the grouped gate | up product
// [M, 2 K] (groups of 8 gate, 8 up columns), from which X = silu(gate) * up is formed on the way.
// W: bfloat16 [N, K].  out: float32 [chunks][M][N], chunks = qvl_gemm_chunked_chunks(N, K, cus);
// the product is the sum of the slabs.  M at most 64, K a multiple of 8.
extern "C" int qvl_gemm_chunked(const void* x, int ldx, const void* W, int ldw, void* out, int M, int N, int K,
                                int swiglu, int cus, hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 64) return QVL_ERR_LIMIT;
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || ldx % 8 || ldx < (swiglu ? 2 * K : K) || cus <= 0 || !x || !W || !out)
    return QVL_ERR_SHAPE;
  const Cut cut = cut_for(N, K, cus);
  ChunkedArgs p;
  p.X = (const bf16_t*)x; p.ldx = ldx; p.W = (const bf16_t*)W; p.ldw = ldw; p.out = (float*)out;
  p.M = M; p.N = N; p.K = K; p.chunks = cut.chunks; p.ranges = cut.ranges; p.tile_rows = cut.tile_rows;
  p.swiglu = swiglu ? 1 : 0;
  const dim3 grid(cut.chunks * cut.ranges), block(64 * CW);
  if (M <= 16) hipLaunchKernelGGL(gemm_chunked_kernel<1>, grid, block, 0, stream, p);
  else if (M <= 32) hipLaunchKernelGGL(gemm_chunked_kernel<2>, grid, block, 0, stream, p);
  else if (M <= 48) hipLaunchKernelGGL(gemm_chunked_kernel<3>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(gemm_chunked_kernel<4>, grid, block, 0, stream, p);
  return qvl_launch_status();
}
