// Products with 17 to 64 rows whose rows do not fit a compute unit whole: out[c][M, N] = partial
// sums of X[M, K] . W[N, K]^T over chunk c of K, bfloat16 operands, float32 sums.
//
// With up to 32 rows the resident kernel keeps all of X in one compute unit (registers and LDS)
// while W streams by.  64 rows of a 3584-wide X are 459 KB: more than a compute unit holds.  Here
// K is cut into chunks that do fit: a block owns one chunk of K (at most 1248 wide) and a range of
// W's rows.  It puts its chunk of all rows of X into LDS once, and then each of its 8 waves
// streams the chunk's part of its own rows of W: two tiles of at most 16 rows at a time,
// v_mfma_f32_16x16x32_bf16 with the X operand read from LDS and used for both tiles, through a ring
// of 16 steps (32 loads) in flight per wave.  The block has few waves so that each has the
// registers for that many loads: at the latency HBM shows under this load (about 9 us) the chip
// needs some 45 MB on their way to stream at 5 TB/s, 180 KB a compute unit.  No wave waits for
// another after the fill: no sums are merged inside the block, and X costs L2 no more than W
// costs HBM.  What is left is the sum over the chunks: every block writes its partial sums as a
// slab of their own, out[chunk][M][N] in float32, and whoever reads the result adds the slabs in
// chunk order (the norm that follows), so the result does not depend on which block finished first.
//
// Every wave streams rows of its own, 64 bytes of each at a time, so HBM sees many short streams
// side by side where the resident kernel gives it a few long ones: this kernel reaches 3 to 4 TB/s
// where that one reaches 5.  It is the better one where the resident kernel has to read its rows
// again and again (17 to 32 rows with a long inner size) and where the library has too few tiles
// to fill the device (33 to 64 rows against a small matrix).
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define CW 8             // waves per block: few, so that each has registers for many loads in flight
#define RING 10          // steps of W in flight per wave (two loads each: the wave has two tiles in hand)
#define MAX_STEPS 39     // 32-wide steps of a chunk: 64 rows of (39 * 64 + 16) bytes are 160,768 bytes of LDS
#define ROW16 (MAX_STEPS * 4 + 1)   // 16-byte units of a row of X in LDS (one of padding: no bank conflicts)

struct ChunkedArgs {
  const bf16_t* X;   // [M, K]
  int ldx;
  const bf16_t* W;   // [N, K]
  int ldw;
  float* out;        // [chunks][M][N]
  int M, N, K;
  int chunks, ranges;   // grid = chunks * ranges
  int tile_rows;        // rows of W per wave tile, 1..16
};

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(p));
}
__device__ __forceinline__ u32x4_t zero16() { return u32x4_t{0u, 0u, 0u, 0u}; }

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

  // ---- every wave its own tiles of W, two at a time; the first pair's loads are asked for before X is
  const int nr = p.tile_rows;
  const int tiles = (n_end - n_begin + nr - 1) / nr, pairs = (tiles + 1) / 2;
  int n0[2], rows_here[2];
  const bf16_t* wrow[2];
  auto set_pair = [&](int pair) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int tile = 2 * pair + i;
      n0[i] = n_begin + tile * nr;
      rows_here[i] = tile < tiles ? min(nr, n_end - n0[i]) : 0;
      // a lane past the tile's rows (or a tile past the range) reads the range's first row: never stored
      wrow[i] = p.W + (size_t)(r < rows_here[i] ? n0[i] + r : n_begin) * p.ldw + k0 + 8 * lg;
    }
  };
  // Step s of a tile's W operand.  Every lane always loads from a valid address, with no branch
  // around the load and no use of the value before its step comes (the compiler then counts the
  // loads in flight exactly and each step waits for its own loads only): a step past the chunk's
  // end reads the last step again, and in the last step of K a lane past K reads the last 8 values
  // of its row instead, which meet zeros of X.
  const int k_last = k0 + 32 * (steps - 1) + 8 * lg;
  const int last_back = k_last < p.K ? 0 : k_last - (p.K - 8);
  auto load_w = [&](int i, int s) {
    s = s < steps ? s : steps - 1;
    return load8(wrow[i] + 32 * s - (s == steps - 1 ? last_back : 0));
  };
  bf16x8_t ring[RING][2];
  auto prime = [&]() {
#pragma unroll
    for (int j = 0; j < RING; ++j) {
      ring[j][0] = load_w(0, j);
      ring[j][1] = load_w(1, j);
    }
  };
  if (wave < pairs) {
    set_pair(wave);
    prime();
  }

  // ---- this chunk of every row of X into LDS ---------------------------------------------------
  const int units = steps * 4;   // 16-byte units of a row
  const int total = 16 * MT * units;
  auto fetch = [&](int idx) {
    const int row = idx / units, u = idx - row * units, k = k0 + 8 * u;
    u32x4_t v = zero16();
    if (idx < total && row < p.M && k < p.K) v = *reinterpret_cast<const u32x4_t*>(p.X + (size_t)row * p.ldx + k);
    return v;
  };
  constexpr int FILL = 12;   // 16-byte units a thread has in flight: the whole fill is two or three round trips
  for (int base = threadIdx.x; base < total; base += FILL * blockDim.x) {
    u32x4_t v[FILL];
#pragma unroll
    for (int j = 0; j < FILL; ++j) v[j] = fetch(base + j * blockDim.x);
#pragma unroll
    for (int j = 0; j < FILL; ++j) {
      const int idx = base + j * blockDim.x;
      if (idx < total) {
        const int row = idx / units;
        xs[row * ROW16 + (idx - row * units)] = v[j];
      }
    }
  }
  __syncthreads();

  for (int pair = wave; pair < pairs; pair += CW) {
    if (pair != wave) {
      set_pair(pair);
      prime();
    }
    f32x4_t acc[2][MT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[i][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // one step of both tiles: every X operand that is read from LDS is multiplied with both
    auto step = [&](int s, bf16x8_t a0, bf16x8_t a1) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8_t x = __builtin_bit_cast(bf16x8_t, xs[(16 * t + r) * ROW16 + 4 * s + lg]);
        acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, x, acc[0][t], 0, 0, 0);
        acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, x, acc[1][t], 0, 0, 0);
      }
    };
    const int whole = steps / RING;   // rounds of RING steps, each of which asks for the round after it
    for (int round = 0; round < whole; ++round) {
#pragma unroll
      for (int j = 0; j < RING; ++j) {
        const int s = round * RING + j;
        const bf16x8_t a0 = ring[j][0], a1 = ring[j][1];
        ring[j][0] = load_w(0, s + RING);
        ring[j][1] = load_w(1, s + RING);
        step(s, a0, a1);
      }
    }
    const int left = steps - whole * RING;   // the same for the whole wave; their loads are in the ring
#pragma unroll
    for (int j = 0; j < RING; ++j)
      if (j < left) step(whole * RING + j, ring[j][0], ring[j][1]);
    // lane (r, lg) holds the sums of row 16 t + r of X with rows n0 + 4 lg .. + 3 of W
    float* slab = p.out + (size_t)chunk * p.M * p.N;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + r;
        if (m < p.M) {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (4 * lg + v < rows_here[i]) slab[(size_t)m * p.N + n0[i] + 4 * lg + v] = acc[i][t][v];
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
    int tiles = (per_wave + 15) / 16;                              // its tiles: it has two in hand at a time
    if (per_wave > 8 && tiles % 2) ++tiles;
    const int tile_rows = (per_wave + tiles - 1) / tiles;
    const int steps = (steps_all + chunks - 1) / chunks;
    // a wave's time: its loads (a load instruction moves at most 16 rows; fewer rows, the same instruction)
    // plus the fill of X, plus the slab it writes and somebody reads again
    const double cost = (double)tiles * steps * (tile_rows < 4 ? 4 : tile_rows) / 32.0 + 0.02 * steps + 0.15 * chunks;
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

// x: bfloat16 [M, K] (ldx elements a row).  W: bfloat16 [N, K].  out: float32 [chunks][M][N], chunks = qvl_gemm_chunked_chunks(N, K, cus);
// the product is the sum of the slabs.  M at most 64, K a multiple of 8.
extern "C" int qvl_gemm_chunked(const void* x, int ldx, const void* W, int ldw, void* out, int M, int N, int K,
                                int cus, hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 64) return QVL_ERR_LIMIT;
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || ldx % 8 || ldx < K || cus <= 0 || !x || !W || !out)
    return QVL_ERR_SHAPE;
  const Cut cut = cut_for(N, K, cus);
  ChunkedArgs p;
  p.X = (const bf16_t*)x; p.ldx = ldx; p.W = (const bf16_t*)W; p.ldw = ldw; p.out = (float*)out;
  p.M = M; p.N = N; p.K = K; p.chunks = cut.chunks; p.ranges = cut.ranges; p.tile_rows = cut.tile_rows;
  const dim3 grid(cut.chunks * cut.ranges), block(64 * CW);
  if (M <= 16) hipLaunchKernelGGL(gemm_chunked_kernel<1>, grid, block, 0, stream, p);
  else if (M <= 32) hipLaunchKernelGGL(gemm_chunked_kernel<2>, grid, block, 0, stream, p);
  else if (M <= 48) hipLaunchKernelGGL(gemm_chunked_kernel<3>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(gemm_chunked_kernel<4>, grid, block, 0, stream, p);
  return qvl_launch_status();
}
