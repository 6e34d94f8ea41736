// Products with at most 64 rows (a decode step's projections): out[M, N] = X[M, K] . W[N, K]^T,
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
// Up to 16 rows of X are one column tile of the matrix instruction; 17 to 32 rows are two (MT = 2):
// every W fragment that is loaded is multiplied with both.  33 to 64 rows are four (MT = 4): they
// fit neither the registers nor LDS, so X is not resident: for every tile of W each wave reads its
// columns of all rows of X again (from L2: four times the bytes of the tile's W), and a norm is
// not folded in (the host hands over normalised rows).
// If K fits one pass (K <= 4096) the X operand stays in registers (the second column tile, if
// there is one, in LDS, which takes K <= 32 * XHI_STEPS) for all of the block's tiles; W comes
// through three half-tile buffers that go round, so that the next tile and a half are on their way
// while a tile is multiplied and its sums are merged.  A longer K is walked in passes of 4096 that
// take their turns in the same rotation (X is then read again for every pass).
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
#define XHI_STEPS 120   // 32-wide K steps of the second column tile that fit LDS beside the sums: K <= 3840

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
  // More rows of X than a block carries: `groups` blocks form a team that walks the same tiles of W,
  // block g of the team with rows g * (16 MT) ... of X.  The blocks of a team run on the same XCD
  // at the same pace, so the tile that the first of them brings in from HBM the others find in
  // that XCD's L2 (or in the memory-side cache): W leaves HBM once.
  int groups;
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

template <typename TO, int PRO, int EPI, bool ONE_PASS, int MT>
__global__ __launch_bounds__(64 * RW) void gemm_resident_kernel(ResidentArgs p) {
  constexpr int COLS = 16 * MT;   // rows of X the block carries
  // MT = 1: two buffers, a tile's sums are read while the next tile's are written.  MT = 2: one
  // (LDS also holds the second column tile of X), and the norm weights borrow it before the first tile.
  static_assert(MT == 1 || MT == 2 || MT == 4, "one, two or four column tiles");
  static_assert(MT != 4 || PRO == PRO_PLAIN, "with four column tiles the rows arrive normalised");
  __shared__ __attribute__((aligned(16))) float red[MT == 1 ? 2 : 1][RW][16 * COLS];
  __shared__ float rowsq[RW][16];
  __shared__ __attribute__((aligned(16))) float gains_own[(PRO == PRO_NORM && MT == 1) ? RW : 1][RK * 32];
  __shared__ u32x4_t xhi[(MT == 2 && ONE_PASS) ? XHI_STEPS * 64 : 1];
  float (*gains)[RK * 32] = MT == 1 ? gains_own : reinterpret_cast<float (*)[RK * 32]>(&red[0][0][0]);  // norm weights of each wave's columns
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int k_lane = wave * RK * 32 + 8 * lg;  // first K index of this lane within a pass
  // Workgroups go to the XCDs in turn, so blocks b, b + 8, b + 16, ... share an XCD: consecutive
  // ones of them form a team.
  int team = blockIdx.x, teams = gridDim.x, m0 = 0;   // m0: this block's first row of X
  if (p.groups > 1) {   // the grid is a multiple of 8 groups
    const int xcd_turn = blockIdx.x >> 3;
    team = (xcd_turn / p.groups) * 8 + (blockIdx.x & 7);
    teams = (int)(gridDim.x >> 3) / p.groups * 8;
    m0 = (xcd_turn % p.groups) * COLS;
  }

  // ---- the X operand of one pass ------------------------------------------------------------
  // Column tile t holds rows 16 t .. 16 t + 15 of X.  first_w issues the block's first W loads at
  // the point of the prologue where they fit best.  again: another column tile's norm came before
  // (the norm weights are in LDS already, and the statistics' place may still be read).
  auto load_x = [&](int t, int k0, bf16x8_t* xb, auto first_w, bool again = false) {
    const int row = m0 + 16 * t + r;
    const bool m_ok = row < p.M;
    if (PRO == PRO_PLAIN) {
      first_w();   // W first: it is the long wait
      const bf16_t* xrow = p.X + (size_t)(m_ok ? row : 0) * p.ldx;
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
      const float* hrow = p.H + (size_t)(m_ok ? row : 0) * p.ldh;
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
      float4 g4 = {0.f, 0.f, 0.f, 0.f};
      if (!again && kg < p.K) g4 = *reinterpret_cast<const float4*>(p.norm_w + kg);
      first_w();
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < RK; ++u)
        ss += v[u][0].x * v[u][0].x + v[u][0].y * v[u][0].y + v[u][0].z * v[u][0].z + v[u][0].w * v[u][0].w +
              v[u][1].x * v[u][1].x + v[u][1].y * v[u][1].y + v[u][1].z * v[u][1].z + v[u][1].w * v[u][1].w;
      ss += __shfl_xor(ss, 16, QVL_WAVE);
      ss += __shfl_xor(ss, 32, QVL_WAVE);
      if (again) __syncthreads();   // the other column tile's statistics have been read
      if (lg == 0) rowsq[wave][r] = ss;
      if (!again) *reinterpret_cast<float4*>(&gains[wave][4 * lane]) = g4;
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
  // steps u0 .. u0 + n - 1 of a tile's W operand
  auto load_w_part = [&](int tile, int k0, int u0, int n, bf16x8_t* a) {
    const int row = w_row(tile, r);
    const bool row_ok = r < tile_rows(tile) && row >= 0 && row < p.N;
    const bf16_t* wrow = p.W + (size_t)(row_ok ? row : 0) * p.ldw;
#pragma unroll
    for (int u = 0; u < n; ++u) {
      const int k = k0 + k_lane + (u0 + u) * 32;
      a[u] = (row_ok && k < p.K) ? load8(wrow + k) : zero8();
    }
  };
  auto load_w = [&](int tile, int k0, bf16x8_t* a) { load_w_part(tile, k0, 0, RK, a); };
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
    if (threadIdx.x >= 16 * COLS || EPI == EPI_SWIGLU) return e;
    const int m = m0 + (threadIdx.x >> 4), nl = threadIdx.x & 15, n = w_row(tile, nl);
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
  // A wave's sums lie as [row of X][row of the tile]: a lane writes its four at once, and the
  // thread that finishes element e = 16 m + nl reads word e of every wave.
  // MT = 1, one barrier per tile: the sums go into the buffer that was read two tiles ago; whoever
  // reads it (the first four waves) has passed the barrier of the tile in between since.
  // MT = 2, one buffer: a second barrier keeps the next tile's sums out until these are read.
  struct Acc {
    f32x4_t t[MT];
  };
  int parity = 0;
  auto finish = [&](int tile, const Acc& acc, const Epi& epi) {
    float (*buf)[16 * COLS] = red[MT == 1 ? parity : 0];
    parity ^= 1;
#pragma unroll
    for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4_t*>(&buf[wave][(16 * t + r) * 16 + 4 * lg]) = acc.t[t];
    __syncthreads();
    if (threadIdx.x < 16 * COLS) {
      const int e = threadIdx.x;
      const int m = m0 + (e >> 4), nl = e & 15, n = w_row(tile, nl);
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < RW; ++w) sum += buf[w][e];
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
    if (MT >= 2) __syncthreads();
  };
  // The W operand's steps come as two halves (a_lo, a_hi).  x1: the second column tile's operand in
  // registers; null: it is in LDS (one pass), except for the waves whose steps lie beyond K then.
  const bool hi_live = wave * RK < XHI_STEPS;
  // steps u0 .. u0 + n - 1 of a tile, whose W operands are a[0 .. n - 1]
  auto product_part = [&](const bf16x8_t* a, int u0, int n, const bf16x8_t* x0, const bf16x8_t* x1, Acc acc) {
#pragma unroll
    for (int i = 0; i < n; ++i) {
      const int u = u0 + i;
      acc.t[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], x0[u], acc.t[0], 0, 0, 0);
      if (MT == 2) {
        if (!ONE_PASS)
          acc.t[MT - 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], x1[u], acc.t[MT - 1], 0, 0, 0);
        else if (hi_live)
          acc.t[MT - 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              a[i], __builtin_bit_cast(bf16x8_t, xhi[(wave * RK + u) * 64 + lane]), acc.t[MT - 1], 0, 0, 0);
      }
    }
    return acc;
  };
  auto product = [&](const bf16x8_t* a_lo, const bf16x8_t* a_hi, const bf16x8_t* x0, const bf16x8_t* x1, Acc acc) {
    acc = product_part(a_lo, 0, RK / 2, x0, x1, acc);
    return product_part(a_hi, RK / 2, RK / 2, x0, x1, acc);
  };
  // half of the plain X operand of the pass that starts at k0 (column tile 0): steps half * RK / 2 ...
  auto load_x_half = [&](int k0, int half, bf16x8_t* xb) {
    const int row = m0 + r;
    const bool m_ok = row < p.M;
    const bf16_t* xrow = p.X + (size_t)(m_ok ? row : 0) * p.ldx;
#pragma unroll
    for (int i = 0; i < RK / 2; ++i) {
      const int u = half * (RK / 2) + i, k = k0 + k_lane + u * 32;
      xb[u] = (m_ok && k < p.K) ? load8(xrow + k) : zero8();
    }
  };
  // MT = 4: the X operands of the pass that starts at k0 come from memory (L2) for every tile, two
  // steps of a column tile at a time through two small buffers that take turns, so that the next
  // loads are on their way while these are multiplied (and the other waves of the SIMD fill the rest
  // of the wait).
  auto product_streamed = [&](const bf16x8_t* a_lo, const bf16x8_t* a_hi, int k0, Acc acc) {
    constexpr int Q = 2, PARTS = RK / Q, CHUNKS = MT * PARTS;
    bf16x8_t xs[2][Q];
    auto load_chunk = [&](int c, bf16x8_t* dst) {
      const int t = c / PARTS, part = c % PARTS;
      const int row = m0 + 16 * t + r;
      const bool m_ok = row < p.M;
      const bf16_t* xrow = p.X + (size_t)(m_ok ? row : 0) * p.ldx;
#pragma unroll
      for (int u = 0; u < Q; ++u) {
        const int k = k0 + k_lane + (part * Q + u) * 32;
        dst[u] = (m_ok && k < p.K) ? load8(xrow + k) : zero8();
      }
    };
    load_chunk(0, xs[0]);
    load_chunk(1, xs[1]);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int t = c / PARTS, part = c % PARTS;
#pragma unroll
      for (int u = 0; u < Q; ++u) {
        const int step = part * Q + u;
        const bf16x8_t a = step < RK / 2 ? a_lo[step] : a_hi[step - RK / 2];
        acc.t[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, xs[c & 1][u], acc.t[t], 0, 0, 0);
      }
      if (c + 2 < CHUNKS) load_chunk(c + 2, xs[c & 1]);
    }
    return acc;
  };
  Acc zero;
#pragma unroll
  for (int t = 0; t < MT; ++t) zero.t[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  if (ONE_PASS || MT == 1 || MT == 4) {
    // The block's work is a sequence of steps: every tile of its own, and within a tile every pass
    // over K (one, if X stays resident).  Three half-step buffers of W go round: while a step is
    // multiplied, the first half of the next is on its way; its second half and the first half of
    // the step after it are asked for as soon as the product has freed their registers, and arrive
    // during the merge of the sums (or, between the passes of a tile, while the next rows of X come).
    const int passes = ONE_PASS ? 1 : (p.K + PASS_K - 1) / PASS_K;
    auto step_after = [&](int& t, int& ps) {
      if (++ps >= passes) {
        ps = 0;
        t += teams;
      }
    };
    bf16x8_t xb[RK];
    bf16x8_t w[3][RK / 2];
    int tile = team, pass = 0;
    if (MT == 4) {
      if (tile < p.ntiles) {
        load_w_part(tile, 0, 0, RK / 2, w[0]);
        load_w_part(tile, 0, RK / 2, RK / 2, w[1]);
      }
    } else if (MT == 1) {
      load_x(0, 0, xb, [&] {
        if (tile < p.ntiles) {
          load_w_part(tile, 0, 0, RK / 2, w[0]);
          load_w_part(tile, 0, RK / 2, RK / 2, w[1]);
        }
      });
    } else {
      // rows 16..31 first, while few registers are taken: each lane keeps its own operands of
      // them in LDS and reads them back itself
      bf16x8_t hi[RK];
      load_x(1, 0, hi, [&] { if (tile < p.ntiles) load_w_part(tile, 0, 0, RK / 2, w[0]); });
#pragma unroll
      for (int u = 0; u < RK; ++u)
        if (hi_live) xhi[(wave * RK + u) * 64 + lane] = __builtin_bit_cast(u32x4_t, hi[u]);
      load_x(0, 0, xb, [&] { if (tile < p.ntiles) load_w_part(tile, 0, RK / 2, RK / 2, w[1]); }, true);
      if (PRO == PRO_NORM) __syncthreads();   // the norm weights lie where the first tile's sums go
    }
    Epi e = epi_load(tile);
    {
      int t1 = tile, p1 = 0;
      step_after(t1, p1);
      if (t1 < p.ntiles) load_w_part(t1, p1 * PASS_K, 0, RK / 2, w[2]);
    }
    Acc acc = zero;
    // one step whose halves are in a_lo and a_hi; false: it was the block's last
    // A half buffer is asked for again the moment its steps are multiplied (not after the whole
    // step): every half then has a whole period, a step and a merge, to arrive in.  Between the
    // passes of a tile the next rows of X are asked for the same way, each half ahead of the W
    // half that is needed with it (loads come back in the order they were asked for).
    auto one = [&](bf16x8_t* a_lo, bf16x8_t* a_hi) {
      int tn = tile, pn = pass;
      step_after(tn, pn);
      int ta = tn, pa = pn;
      step_after(ta, pa);
      const bool tile_done = ONE_PASS || pn == 0;
      Epi e_next = e;
      if constexpr (MT == 4) {
        acc = product_streamed(a_lo, a_hi, pass * PASS_K, acc);
        if (tile_done) e_next = epi_load(tn);
        if (tn < p.ntiles) load_w_part(tn, pn * PASS_K, RK / 2, RK / 2, a_lo);
        if (ta < p.ntiles) load_w_part(ta, pa * PASS_K, 0, RK / 2, a_hi);
      } else {
        acc = product_part(a_lo, 0, RK / 2, xb, nullptr, acc);
        if (tn < p.ntiles) {
          if (!ONE_PASS && MT == 1) load_x_half(pn * PASS_K, 0, xb);
          load_w_part(tn, pn * PASS_K, RK / 2, RK / 2, a_lo);
        }
        acc = product_part(a_hi, RK / 2, RK / 2, xb, nullptr, acc);
        if (tile_done) e_next = epi_load(tn);
        if (tn < p.ntiles && !ONE_PASS && MT == 1) load_x_half(pn * PASS_K, 1, xb);
        if (ta < p.ntiles) load_w_part(ta, pa * PASS_K, 0, RK / 2, a_hi);
      }
      if (tile_done) {
        finish(tile, acc, e);
        acc = zero;
        e = e_next;
      }
      tile = tn;
      pass = pn;
      return tn < p.ntiles;
    };
    while (tile < p.ntiles) {
      if (!one(w[0], w[1])) break;
      if (!one(w[2], w[0])) break;
      if (!one(w[1], w[2])) break;
    }
  } else {
    for (int tile = team; tile < p.ntiles; tile += teams) {
      Acc acc = zero;
      const Epi e = epi_load(tile);
      for (int k0 = 0; k0 < p.K; k0 += PASS_K) {
        bf16x8_t xb[RK], x1[MT == 2 ? RK : 1], a[RK];
        load_x(0, k0, xb, [&] { load_w(tile, k0, a); });
        if (MT == 2) load_x(1, k0, x1, [] {}, true);
        acc = product(a, a + RK / 2, xb, x1, acc);
      }
      finish(tile, acc, e);
    }
  }
}

// How M rows are carried: column tiles per block (MT), blocks per team (groups), and whether X stays
// in the block for all its tiles (one pass over K).  Up to 32 rows one block carries them all.
// More rows, or 17 to 32 rows with a K too long for the second column tile's place in LDS, are
// spread over the blocks of a team; a device with too few compute units for teams (fewer than 8
// per group) falls back on one block that streams X (MT = 4).
struct Plan {
  int mt, groups;
  bool one_pass;
};
static Plan plan_for(int M, int K, bool norm, int blocks, bool prefer_teams) {
  if (M <= 16) return Plan{1, 1, K <= PASS_K};
  const bool two_fit = K <= 32 * XHI_STEPS;
  if (M <= 32 && two_fit) return Plan{2, 1, true};
  if (two_fit && blocks >= 8 * ((M + 31) / 32)) return Plan{2, (M + 31) / 32, true};
  const int singles = (M + 15) / 16;
  if ((M > 32 || prefer_teams || norm) && blocks >= 8 * singles) return Plan{1, singles, K <= PASS_K};
  if (M <= 32) return Plan{2, 1, false};
  return Plan{4, 1, K <= PASS_K};
}
// the number of teams the plan's grid has: what the tiles are divided among
static int plan_teams(const Plan& pl, int blocks) { return pl.groups == 1 ? blocks : blocks / (8 * pl.groups) * 8; }

template <typename TO, int PRO, int EPI>
static int launch(ResidentArgs p, const Plan& pl, int blocks, hipStream_t stream) {
  const int teams = plan_teams(pl, blocks);
  p.groups = pl.groups;
  const dim3 grid(pl.groups == 1 ? (teams < p.ntiles ? teams : p.ntiles) : teams * pl.groups), block(64 * RW);
#define QVL_GO(ONE, MT) hipLaunchKernelGGL((gemm_resident_kernel<TO, PRO, EPI, ONE, MT>), grid, block, 0, stream, p)
  if (PRO == PRO_NORM && !pl.one_pass) return QVL_ERR_LIMIT;   // a norm is only folded into a single pass
  if (pl.mt == 1) {
    if (pl.one_pass) QVL_GO(true, 1);
    else if constexpr (PRO == PRO_PLAIN) QVL_GO(false, 1);
  } else if (pl.mt == 2) {
    if (pl.one_pass) QVL_GO(true, 2);
    else if constexpr (PRO == PRO_PLAIN) QVL_GO(false, 2);
  } else if constexpr (PRO == PRO_PLAIN) {
    if (pl.one_pass) QVL_GO(true, 4);
    else QVL_GO(false, 4);
  } else {
    return QVL_ERR_LIMIT;
  }
#undef QVL_GO
  return qvl_launch_status();
}

// Whether qvl_gemm_resident(_rope) forms the norm of M rows of width K itself on a device with this
// many compute units.
extern "C" int qvl_gemm_resident_folds_norm(int M, int K, int blocks) {
  if (M <= 0 || M > 64 || K <= 0 || K > PASS_K || blocks <= 0) return 0;
  const Plan pl = plan_for(M, K, true, blocks, false);
  return pl.one_pass && pl.mt <= 2;
}

extern "C" int qvl_gemm_resident_pass_k() { return PASS_K; }
// the longest K with which 17 to 32 rows stay resident (and with which their norm is folded in)
extern "C" int qvl_gemm_resident_two_tile_k() { return 32 * XHI_STEPS; }

// x: bfloat16 [M, K] (h null), or h: float32 [M, K] with norm_w [K] and eps (x null): X = rmsnorm(h) * norm_w.
// epilogue 0: out[M, N] in out_dtype (0 float32, 1 bfloat16); 1: out (float32 [M, N]) += product;
// 2: out[M, N/2] bfloat16 = silu(gate) * up for W rows in groups of 8 gate, 8 up.
// max_blocks: blocks to launch at most (the number of compute units).
extern "C" int qvl_gemm_resident(const void* x, int ldx, const void* h, int ldh, const void* norm_w, float eps,
                                 const void* W, int ldw, const void* bias, void* out, int ldo, int M, int N, int K,
                                 int out_dtype, int epilogue, int max_blocks, int flags, hipStream_t stream) {
  // flags bit 0: 17 to 32 rows with a long K go to a team of two blocks rather than to one block
  // that reads its rows again for every pass
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 64) return QVL_ERR_LIMIT;
  if (M > 32 && K > PASS_K) return QVL_ERR_LIMIT;   // teams of more than two keep their rows for a single pass
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || max_blocks <= 0 || !W || !out) return QVL_ERR_SHAPE;
  const bool norm = h != nullptr;
  const Plan pl = plan_for(M, K, norm, max_blocks, flags & 1);
  const int teams = plan_teams(pl, max_blocks);
  if (norm) {
    if (x || !norm_w || K > PASS_K || ldh % 4 || ldh < K) return QVL_ERR_SHAPE;
    if (!qvl_gemm_resident_folds_norm(M, K, max_blocks)) return QVL_ERR_LIMIT;
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
    const long long per_round = 16LL * teams;
    const long long rounds = (N + per_round - 1) / per_round;
    p.rows = (int)((N + rounds * teams - 1) / (rounds * teams));
  }
  p.ntiles = (N + p.rows - 1) / p.rows;
  p.whole_tiles = p.ntiles; p.parts = 1; p.pairs = 8;
  if (epilogue == EPI_SWIGLU) {
    const int groups = N / 16, left = groups % teams;
    if (groups > teams && left > 0) {
      while (p.parts < 8 && left * p.parts * 2 <= teams) p.parts *= 2;
      p.pairs = 8 / p.parts;
      p.whole_tiles = groups - left;
      p.ntiles = p.whole_tiles + left * p.parts;
    }
  }
#define QVL_RES(TO, EPI) \
  return norm ? launch<TO, PRO_NORM, EPI>(p, pl, max_blocks, stream) : launch<TO, PRO_PLAIN, EPI>(p, pl, max_blocks, stream)
  if (epilogue == EPI_STORE && out_dtype == 0) QVL_RES(float, EPI_STORE);
  if (epilogue == EPI_STORE && out_dtype == 1) QVL_RES(bf16_t, EPI_STORE);
  if (epilogue == EPI_RESIDUAL) QVL_RES(float, EPI_RESIDUAL);
  if (epilogue == EPI_SWIGLU) QVL_RES(bf16_t, EPI_SWIGLU);
#undef QVL_RES
  return QVL_ERR_DTYPE;
}

// The stacked query | key | value projection of at most 32 tokens with rotation and cache write
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
  if (M > 64) return QVL_ERR_LIMIT;
  if (M > 32 && K > PASS_K) return QVL_ERR_LIMIT;   // as in qvl_gemm_resident
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || max_blocks <= 0 || !W || !q_out) return QVL_ERR_SHAPE;
  if (nq <= 0 || nkv < 0 || hd <= 0 || hd % 16 || ps <= 0 || !cs) return QVL_ERR_SHAPE;
  if (nkv > 0 && (!slot || !kc || !vc)) return QVL_ERR_SHAPE;
  const bool norm = h != nullptr;
  const Plan pl = plan_for(M, K, norm, max_blocks, false);
  const int teams = plan_teams(pl, max_blocks);
  if (norm) {
    if (x || !norm_w || K > PASS_K || ldh % 4 || ldh < K) return QVL_ERR_SHAPE;
    if (!qvl_gemm_resident_folds_norm(M, K, max_blocks)) return QVL_ERR_LIMIT;
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
    const long long vrows = (long long)nkv * hd, per_round = 16LL * teams;
    const long long rounds = (vrows + per_round - 1) / per_round;
    p.rows = (int)((vrows + rounds * teams - 1) / (rounds * teams));
    value_tiles = (int)((vrows + p.rows - 1) / p.rows);
  }
  p.ntiles = p.pair_tiles + value_tiles;
  p.cs = (const float*)cs; p.slot = (const int*)slot; p.q_out = (bf16_t*)q_out; p.kc = (bf16_t*)kc;
  p.vc = (bf16_t*)vc; p.nq = nq; p.nkv = nkv; p.hd = hd; p.ps = ps;
  p.whole_tiles = 0; p.parts = 1; p.pairs = 8;
  return norm ? launch<bf16_t, PRO_NORM, EPI_ROPE>(p, pl, max_blocks, stream)
              : launch<bf16_t, PRO_PLAIN, EPI_ROPE>(p, pl, max_blocks, stream);
}
