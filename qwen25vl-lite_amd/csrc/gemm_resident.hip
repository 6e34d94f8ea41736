// Products with at most 16 rows (a decode step's projections): out[M, N] = X[M, K] . W[N, K]^T,
// bfloat16 operands, float32 accumulation.  The step is bound by reading W once from HBM, so W
// is the streamed operand and everything around the product is folded into this kernel, because
// between two products a short kernel of its own costs more than its arithmetic (its code and
// data have just been flushed from the caches by the weights).
//
// A block of 16 waves owns row tiles of W (tile, tile + gridDim.x, ...).  A tile has `rows` <= 16
// rows of W (= outputs); the host picks `rows` so that the tiles divide evenly among the compute
// units (3584 outputs on 256 units: 256 tiles of 14 rather than 224 of 16), the matrix-core tile's
// other rows stay zero.
// Wave w covers the 256 values of K from 256 w on, as the A operand (W rows) and B operand (X
// rows) of v_mfma_f32_16x16x32_bf16; the 16 waves' sums meet in LDS and are added in wave order.
// If K fits one pass (K <= 4096) the X operand stays in registers for all of the block's tiles and
// the W loads of the next tile are issued before the current tile's sums are merged; a longer K is
// walked in passes of 4096.
//
// What is folded in:
//   prologue  PRO_NORM      X = rmsnorm(H) * w, from the float32 residual H (statistics in float32,
//                           each wave sums its own 256 columns, the block adds the waves in order)
//   epilogue  EPI_RESIDUAL  out += product, out being the float32 residual
//             EPI_SWIGLU    W's rows come in groups of 8 gate rows, 8 up rows; out[M, N/2] =
//                           silu(gate) * up, in bfloat16
//             EPI_ROPE      W is the stacked query | key | value projection.  A tile of a query or
//                           key head takes 8 channels and the 8 channels they are rotated with
//                           (half a head further), so the rotation happens here; queries are
//                           written out, keys and values go straight into their page slots
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define RW 16   // waves per block
#define RK 8    // 32-wide K steps per wave and pass
#define PASS_K (RW * RK * 32)

enum { PRO_PLAIN = 0, PRO_NORM = 1 };
enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_ROPE = 3 };

struct ResidentArgs {
  const bf16_t* X;       // PRO_PLAIN: [M, K]
  int ldx;
  const float* H;        // PRO_NORM: float32 [M, K]
  int ldh;
  const float* norm_w;   // PRO_NORM: [K]
  float eps;
  const bf16_t* W;       // [N, K]
  int ldw;
  const float* bias;     // [N] or null (EPI_STORE and EPI_RESIDUAL)
  void* out;
  int ldo;
  int M, N, K, ntiles;
  int rows;              // rows of W per tile, 1..16 (16 with EPI_SWIGLU and EPI_ROPE)
  // EPI_ROPE: W rows are nq query heads, nkv key heads, nkv value heads of hd channels each
  // (hd a multiple of 16, rotation over the whole head in pairs (f, f + hd/2))
  const float* cs;       // [M, hd/2, 2] cosine and sine of each token's angle at each frequency
  const int* slot;       // [M] flat slot of each token in the cache (page * ps + offset), -1: none
  bf16_t* q_out;         // [M, nq hd]
  bf16_t* kc;            // [pages, nkv, ps, hd]
  bf16_t* vc;            // [pages, nkv, hd, ps]
  int nq, nkv, hd, ps;
  int pair_tiles;        // tiles of query and key heads (16 rows each); value tiles of `rows` rows follow
  // EPI_SWIGLU: the first whole_tiles tiles are whole groups of 8 + 8 rows; each group after them
  // is cut into `parts` tiles of `pairs` gate rows and their up rows, so that the last round of
  // tiles is as even as the rounds before it
  int whole_tiles, parts, pairs;
};

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(p));
}
__device__ __forceinline__ bf16x8_t zero8() {
  u32x4_t z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8_t, z);
}
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  bf16x2_t v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}

template <typename TO, int PRO, int EPI, bool ONE_PASS>
__global__ __launch_bounds__(64 * RW) void gemm_resident_kernel(ResidentArgs p) {
  __shared__ float red[2][RW][256];   // two buffers: a tile's sums are read while the next tile's are written
  __shared__ float rowsq[RW][16];
  __shared__ __attribute__((aligned(16))) float gains[PRO == PRO_NORM ? RW : 1][RK * 32];   // norm weights of each wave's columns
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int k_lane = wave * RK * 32 + 8 * lg;  // first K index of this lane within a pass
  const bool m_ok = r < p.M;

  // ---- the X operand of one pass ------------------------------------------------------------
  // first_w issues the block's first W loads at the point of the prologue where they fit best
  auto load_x = [&](int k0, bf16x8_t* xb, auto first_w) {
    if (PRO == PRO_PLAIN) {
      first_w();   // W first: it is the long wait
      const bf16_t* xrow = p.X + (size_t)(m_ok ? r : 0) * p.ldx;
#pragma unroll
      for (int u = 0; u < RK; ++u) {
        const int k = k0 + k_lane + u * 32;
        xb[u] = (m_ok && k < p.K) ? load8(xrow + k) : zero8();
      }
    } else {
      // rmsnorm of the float32 rows: this pass covers all of K (ONE_PASS), so the block's waves
      // hold whole rows between them.  Loads return in the order they are issued: the rows and
      // the norm weights are asked for first and W (by first_w) right behind them, so the
      // statistics and the scaling run while W is still on its way.  A lane fetches 4 of its
      // wave's 256 norm weights; they reach the lanes that need them through LDS.
      const float* hrow = p.H + (size_t)(m_ok ? r : 0) * p.ldh;
      float4 v[RK][2];
#pragma unroll
      for (int u = 0; u < RK; ++u) {
        const int k = k_lane + u * 32;
        if (m_ok && k < p.K) {
          v[u][0] = *reinterpret_cast<const float4*>(hrow + k);
          v[u][1] = *reinterpret_cast<const float4*>(hrow + k + 4);
        } else {
          v[u][0] = v[u][1] = float4{0.f, 0.f, 0.f, 0.f};
        }
      }
      const int kg = wave * RK * 32 + 4 * lane;
      const float4 g4 = kg < p.K ? *reinterpret_cast<const float4*>(p.norm_w + kg) : float4{0.f, 0.f, 0.f, 0.f};
      first_w();
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < RK; ++u)
        ss += v[u][0].x * v[u][0].x + v[u][0].y * v[u][0].y + v[u][0].z * v[u][0].z + v[u][0].w * v[u][0].w +
              v[u][1].x * v[u][1].x + v[u][1].y * v[u][1].y + v[u][1].z * v[u][1].z + v[u][1].w * v[u][1].w;
      ss += __shfl_xor(ss, 16, QVL_WAVE);
      ss += __shfl_xor(ss, 32, QVL_WAVE);
      if (lg == 0) rowsq[wave][r] = ss;
      *reinterpret_cast<float4*>(&gains[wave][4 * lane]) = g4;
      __syncthreads();
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < RW; ++w) total += rowsq[w][r];
      const float rs = 1.0f / sqrtf(total / (float)p.K + p.eps);
#pragma unroll
      for (int u = 0; u < RK; ++u) {
        const int k = k_lane + u * 32;
        if (k < p.K) {
          const float4 g0 = *reinterpret_cast<const float4*>(&gains[wave][8 * lg + u * 32]);
          const float4 g1 = *reinterpret_cast<const float4*>(&gains[wave][8 * lg + u * 32 + 4]);
          u32x4_t o = {pack2((v[u][0].x * rs) * g0.x, (v[u][0].y * rs) * g0.y),
                       pack2((v[u][0].z * rs) * g0.z, (v[u][0].w * rs) * g0.w),
                       pack2((v[u][1].x * rs) * g1.x, (v[u][1].y * rs) * g1.y),
                       pack2((v[u][1].z * rs) * g1.z, (v[u][1].w * rs) * g1.w)};
          xb[u] = __builtin_bit_cast(bf16x8_t, o);
        } else {
          xb[u] = zero8();
        }
      }
    }
  };
  // the rows of a tile, and the row of W behind row i of a tile
  auto tile_rows = [&](int tile) { return (EPI == EPI_ROPE && tile < p.pair_tiles) ? 16 : p.rows; };
  auto w_row = [&](int tile, int i) {
    if (EPI == EPI_ROPE) {
      if (tile < p.pair_tiles) {  // 8 channels of a query or key head and the 8 they are rotated with
        const int tph = p.hd >> 4, head = tile / tph, sub = tile - head * tph;
        return head * p.hd + 8 * sub + (i & 7) + (i >> 3) * (p.hd >> 1);
      }
      return (p.nq + p.nkv) * p.hd + (tile - p.pair_tiles) * p.rows + i;   // value rows
    }
    if (EPI == EPI_SWIGLU && tile >= p.whole_tiles) {
      // a part of one of the last groups: `pairs` gate rows and the up rows that belong to them
      const int part = tile - p.whole_tiles, group = p.whole_tiles + part / p.parts, s = part % p.parts;
      return (i & 7) < p.pairs ? group * 16 + (i >> 3) * 8 + s * p.pairs + (i & 7) : -1;
    }
    return tile * p.rows + i;
  };
  auto load_w = [&](int tile, int k0, bf16x8_t* a) {
    const int row = w_row(tile, r);
    const bool row_ok = r < tile_rows(tile) && row >= 0 && row < p.N;
    const bf16_t* wrow = p.W + (size_t)(row_ok ? row : 0) * p.ldw;
#pragma unroll
    for (int u = 0; u < RK; ++u) {
      const int k = k0 + k_lane + u * 32;
      a[u] = (row_ok && k < p.K) ? load8(wrow + k) : zero8();
    }
  };
  // What the epilogue of a tile reads from memory, for the element (m, nl) this thread finishes.
  // Loads return in the order they are issued, so these are asked for before the W loads of the
  // next tile: waiting for them must not wait for those.
  struct Epi {
    float bias, old;
    float2 cs;
    int slot;
  };
  auto epi_load = [&](int tile) {
    Epi e;
    e.bias = e.old = 0.f;
    e.cs = float2{1.f, 0.f};
    e.slot = -1;
    if (threadIdx.x >= 256 || EPI == EPI_SWIGLU) return e;
    const int m = threadIdx.x >> 4, nl = threadIdx.x & 15, n = w_row(tile, nl);
    if (m >= p.M || nl >= tile_rows(tile) || n >= p.N) return e;
    if (p.bias) e.bias = p.bias[n];
    if (EPI == EPI_RESIDUAL) e.old = reinterpret_cast<const float*>(p.out)[(size_t)m * p.ldo + n];
    if (EPI == EPI_ROPE) {
      const int head = n / p.hd, d = n - head * p.hd, half = p.hd >> 1;
      if (head < p.nq + p.nkv)
        e.cs = *reinterpret_cast<const float2*>(p.cs + ((size_t)m * half + (d < half ? d : d - half)) * 2);
      if (head >= p.nq) e.slot = p.slot[m];
    }
    return e;
  };
  // ---- merge the waves' sums of one tile and write the result -----------------------------------
  // One barrier per tile: the sums go into the buffer that was read two tiles ago; whoever reads
  // it (the first four waves) has passed the barrier of the tile in between since.
  int parity = 0;
  auto finish = [&](int tile, const f32x4_t& acc, const Epi& epi) {
    float (*buf)[256] = red[parity];
    parity ^= 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) buf[wave][(4 * lg + i) * 16 + r] = acc[i];
    __syncthreads();
    if (threadIdx.x < 256) {
      const int e = threadIdx.x;
      const int m = e >> 4, nl = e & 15, n = w_row(tile, nl);
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < RW; ++w) sum += buf[w][nl * 16 + m];
      if (EPI == EPI_SWIGLU) {
        const float up = __shfl_down(sum, 8, QVL_WAVE);  // rows 8..15 of the tile are the up rows
        if (nl < 8 && m < p.M && n >= 0 && n < p.N) {
          bf16_t* o = reinterpret_cast<bf16_t*>(p.out);
          o[(size_t)m * p.ldo + (n >> 4) * 8 + (n & 7)] = f32_to_bf16((sum / (1.0f + expf(-sum))) * up);
        }
      } else if (EPI == EPI_ROPE) {
        sum += epi.bias;
        const float other = __shfl_xor(sum, 8, QVL_WAVE);   // the channel this one is rotated with
        const int head = n / p.hd, d = n - head * p.hd;
        if (m < p.M && nl < tile_rows(tile) && n < p.N) {
          // (cos, sin) is (1, 0) for value heads; rows 0..7 of a rotated tile are the first halves
          const float val = (nl < 8 || head >= p.nq + p.nkv) ? sum * epi.cs.x - other * epi.cs.y
                                                              : sum * epi.cs.x + other * epi.cs.y;
          if (head < p.nq) {
            p.q_out[((size_t)m * p.nq + head) * p.hd + d] = f32_to_bf16(val);
          } else if (epi.slot >= 0) {
            const size_t page = (size_t)(epi.slot / p.ps), off = (size_t)(epi.slot % p.ps);
            if (head < p.nq + p.nkv)
              p.kc[((page * p.nkv + (head - p.nq)) * p.ps + off) * p.hd + d] = f32_to_bf16(val);
            else
              p.vc[((page * p.nkv + (head - p.nq - p.nkv)) * p.hd + d) * p.ps + off] = f32_to_bf16(val);
          }
        }
      } else if (m < p.M && nl < p.rows && n < p.N) {
        sum += epi.bias;
        if (EPI == EPI_RESIDUAL) {
          float* o = reinterpret_cast<float*>(p.out);
          o[(size_t)m * p.ldo + n] = epi.old + sum;
        } else {
          stf<TO>(reinterpret_cast<TO*>(p.out) + (size_t)m * p.ldo + n, sum);
        }
      }
    }
  };
  auto product = [&](const bf16x8_t* a, const bf16x8_t* xb, f32x4_t acc) {
#pragma unroll
    for (int u = 0; u < RK; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], xb[u], acc, 0, 0, 0);
    return acc;
  };
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};

  if (ONE_PASS) {
    bf16x8_t xb[RK];
    bf16x8_t a[2][RK];
    int tile = blockIdx.x;
    load_x(0, xb, [&] { if (tile < p.ntiles) load_w(tile, 0, a[0]); });
    for (; tile < p.ntiles; tile += 2 * gridDim.x) {
      const int t1 = tile + gridDim.x, t2 = tile + 2 * gridDim.x;
      const Epi e0 = epi_load(tile);
      if (t1 < p.ntiles) load_w(t1, 0, a[1]);
      finish(tile, product(a[0], xb, zero), e0);
      if (t1 >= p.ntiles) break;
      const Epi e1 = epi_load(t1);
      if (t2 < p.ntiles) load_w(t2, 0, a[0]);
      finish(t1, product(a[1], xb, zero), e1);
    }
  } else {
    for (int tile = blockIdx.x; tile < p.ntiles; tile += gridDim.x) {
      f32x4_t acc = zero;
      const Epi e = epi_load(tile);
      for (int k0 = 0; k0 < p.K; k0 += PASS_K) {
        bf16x8_t xb[RK], a[RK];
        load_x(k0, xb, [&] { load_w(tile, k0, a); });
        acc = product(a, xb, acc);
      }
      finish(tile, acc, e);
    }
  }
}

template <typename TO, int PRO, int EPI>
static void launch(const ResidentArgs& p, int blocks, hipStream_t stream) {
  const dim3 grid(blocks < p.ntiles ? blocks : p.ntiles), block(64 * RW);
  if (p.K <= PASS_K)
    hipLaunchKernelGGL((gemm_resident_kernel<TO, PRO, EPI, true>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_resident_kernel<TO, PRO, EPI, false>), grid, block, 0, stream, p);
}

extern "C" int qvl_gemm_resident_pass_k() { return PASS_K; }

// x: bfloat16 [M, K] (h null), or h: float32 [M, K] with norm_w [K] and eps (x null): X = rmsnorm(h) * norm_w.
// epilogue 0: out[M, N] in out_dtype (0 float32, 1 bfloat16); 1: out (float32 [M, N]) += product;
// 2: out[M, N/2] bfloat16 = silu(gate) * up for W rows in groups of 8 gate, 8 up.
// max_blocks: blocks to launch at most (the number of compute units).
extern "C" int qvl_gemm_resident(const void* x, int ldx, const void* h, int ldh, const void* norm_w, float eps,
                                 const void* W, int ldw, const void* bias, void* out, int ldo, int M, int N, int K,
                                 int out_dtype, int epilogue, int max_blocks, hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 16) return QVL_ERR_LIMIT;
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || max_blocks <= 0 || !W || !out) return QVL_ERR_SHAPE;
  const bool norm = h != nullptr;
  if (norm) {
    if (x || !norm_w || K > PASS_K || ldh % 4 || ldh < K) return QVL_ERR_SHAPE;
  } else if (!x || ldx % 8 || ldx < K) {
    return QVL_ERR_SHAPE;
  }
  if (epilogue == EPI_SWIGLU) {
    if (N % 16 || ldo < N / 2 || bias) return QVL_ERR_SHAPE;
  } else if (ldo < N) {
    return QVL_ERR_SHAPE;
  }
  ResidentArgs p;
  p.X = (const bf16_t*)x; p.ldx = ldx; p.H = (const float*)h; p.ldh = ldh; p.norm_w = (const float*)norm_w;
  p.eps = eps; p.W = (const bf16_t*)W; p.ldw = ldw; p.bias = (const float*)bias; p.out = out; p.ldo = ldo;
  p.M = M; p.N = N; p.K = K;
  p.cs = nullptr; p.slot = nullptr;
  p.q_out = nullptr; p.kc = nullptr; p.vc = nullptr; p.nq = p.nkv = p.hd = p.ps = 0; p.pair_tiles = 0;
  // as many rounds of tiles as 16-row tiles need, with rows per tile cut down to what fills them evenly
  p.rows = 16;
  if (epilogue != EPI_SWIGLU) {
    const long long per_round = 16LL * max_blocks;
    const long long rounds = (N + per_round - 1) / per_round;
    p.rows = (int)((N + rounds * max_blocks - 1) / (rounds * max_blocks));
  }
  p.ntiles = (N + p.rows - 1) / p.rows;
  p.whole_tiles = p.ntiles; p.parts = 1; p.pairs = 8;
  if (epilogue == EPI_SWIGLU) {
    const int groups = N / 16, left = groups % max_blocks;
    if (groups > max_blocks && left > 0) {
      while (p.parts < 8 && left * p.parts * 2 <= max_blocks) p.parts *= 2;
      p.pairs = 8 / p.parts;
      p.whole_tiles = groups - left;
      p.ntiles = p.whole_tiles + left * p.parts;
    }
  }
#define QVL_RES(TO, EPI)                                                    \
  do {                                                                      \
    if (norm) launch<TO, PRO_NORM, EPI>(p, max_blocks, stream);             \
    else launch<TO, PRO_PLAIN, EPI>(p, max_blocks, stream);                 \
  } while (0)
  if (epilogue == EPI_STORE && out_dtype == 0) QVL_RES(float, EPI_STORE);
  else if (epilogue == EPI_STORE && out_dtype == 1) QVL_RES(bf16_t, EPI_STORE);
  else if (epilogue == EPI_RESIDUAL) QVL_RES(float, EPI_RESIDUAL);
  else if (epilogue == EPI_SWIGLU) QVL_RES(bf16_t, EPI_SWIGLU);
  else return QVL_ERR_DTYPE;
#undef QVL_RES
  return qvl_launch_status();
}

// The stacked query | key | value projection of at most 16 tokens with rotation and cache write
// folded in (EPI_ROPE).  x / h / norm_w / eps as in qvl_gemm_resident.  W: [(nq + 2 nkv) hd, K];
// bias: float32 [(nq + 2 nkv) hd] or null.  cs: float32 [M, hd / 2, 2], cosine and sine of every
// token's angle at every frequency (1 and 0 where a frequency is not rotated);
// slot: int32 [M] flat cache slot of each token (null with nkv == 0: queries only);
// q_out: bfloat16 [M, nq hd]; kc: [pages, nkv, ps, hd]; vc: [pages, nkv, hd, ps].
// hd must be a multiple of 16 (the rotation covers the whole head, channel f with f + hd / 2).
extern "C" int qvl_gemm_resident_rope(const void* x, int ldx, const void* h, int ldh, const void* norm_w, float eps,
                                      const void* W, int ldw, const void* bias, int M, int K, const void* cs,
                                      const void* slot, void* q_out, void* kc, void* vc, int nq, int nkv, int hd, int ps,
                                      int max_blocks, hipStream_t stream) {
  if (M <= 0) return QVL_OK;
  if (M > 16) return QVL_ERR_LIMIT;
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || max_blocks <= 0 || !W || !q_out) return QVL_ERR_SHAPE;
  if (nq <= 0 || nkv < 0 || hd <= 0 || hd % 16 || ps <= 0 || !cs) return QVL_ERR_SHAPE;
  if (nkv > 0 && (!slot || !kc || !vc)) return QVL_ERR_SHAPE;
  const bool norm = h != nullptr;
  if (norm) {
    if (x || !norm_w || K > PASS_K || ldh % 4 || ldh < K) return QVL_ERR_SHAPE;
  } else if (!x || ldx % 8 || ldx < K) {
    return QVL_ERR_SHAPE;
  }
  ResidentArgs p;
  p.X = (const bf16_t*)x; p.ldx = ldx; p.H = (const float*)h; p.ldh = ldh; p.norm_w = (const float*)norm_w;
  p.eps = eps; p.W = (const bf16_t*)W; p.ldw = ldw; p.bias = (const float*)bias; p.out = nullptr; p.ldo = 0;
  p.M = M; p.N = (nq + 2 * nkv) * hd; p.K = K;
  // query and key heads in tiles of 8 + 8 rows, then the value rows in tiles as small as fills
  // the compute units evenly (36 heads of 128 on 256 units: 256 tiles of 16 and 256 of 2)
  p.pair_tiles = (nq + nkv) * (hd / 16);
  p.rows = 16;
  int value_tiles = 0;
  if (nkv > 0) {
    const long long vrows = (long long)nkv * hd, per_round = 16LL * max_blocks;
    const long long rounds = (vrows + per_round - 1) / per_round;
    p.rows = (int)((vrows + rounds * max_blocks - 1) / (rounds * max_blocks));
    value_tiles = (int)((vrows + p.rows - 1) / p.rows);
  }
  p.ntiles = p.pair_tiles + value_tiles;
  p.cs = (const float*)cs; p.slot = (const int*)slot; p.q_out = (bf16_t*)q_out; p.kc = (bf16_t*)kc;
  p.vc = (bf16_t*)vc; p.nq = nq; p.nkv = nkv; p.hd = hd; p.ps = ps;
  p.whole_tiles = 0; p.parts = 1; p.pairs = 8;
  if (norm) launch<bf16_t, PRO_NORM, EPI_ROPE>(p, max_blocks, stream);
  else launch<bf16_t, PRO_PLAIN, EPI_ROPE>(p, max_blocks, stream);
  return qvl_launch_status();
}
