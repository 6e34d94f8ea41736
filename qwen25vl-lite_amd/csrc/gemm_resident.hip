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
// Wave w covers the 32 RK values of K from 32 RK w on (RK = 8: 256; a second build with RK = 4 serves
// inner sizes up to 2,048, where with 256 values a wave half the waves would have none and the
// other half would carry all loads), as the A operand (W rows) and B operand (X
// rows) of v_mfma_f32_16x16x32_bf16; the 16 waves' sums meet in LDS and are added in wave order.
// Up to 16 rows of X are one column tile of the matrix instruction; 17 to 32 rows are two (MT = 2):
// every W fragment that is loaded is multiplied with both.  More rows are spread over teams of
// blocks (below).
// If K fits one pass (K <= 4096) the X operand stays in registers (the second column tile, if
// there is one, in LDS, which takes K <= 32 * XHI_STEPS) for all of the block's tiles; W comes
// through two half-tile buffers, each asked for again the moment its half is multiplied, so that
// the next tile is on its way while a tile is multiplied and its sums are merged.  (A third buffer
// fits the registers only if the compiler keeps every load in the place it was written; it does
// not, and spills cost more than the deeper stream gains.)  A longer K is walked in passes of 4096
// that take their turns in the same rotation (X is then read again for every pass).
//
// Every load of the stream goes through a buffer descriptor (buffer_load with a byte offset that
// the hardware checks against the buffer's size): a lane that has nothing to load (a row beyond
// the tile, a column beyond K, a tile beyond the last) asks at an offset past the end and gets
// zeros without any traffic.  So no load sits inside a branch, every wave issues the same loads
// in the same order whatever its data, and the compiler can count exactly how many younger loads
// may stay in flight at each wait (a load inside a branch costs a wait for everything: the
// counter only says how many loads are outstanding, and the loads come back in order).
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

typedef __amdgpu_buffer_rsrc_t rsrc_t;
// An offset no buffer reaches: what is loaded there is zero.  Buffers stay below it (the host checks).
#define PAST_END 0xffffff00u
#define BUFFER_LIMIT 0xffffff00ull

__device__ __forceinline__ rsrc_t buffer_of(const void* p, unsigned long long bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, p ? (int)(uint32_t)bytes : 0, 0x00020000);
}
// `fixed` is a compile-time part of the offset: it rides in the instruction, the lanes' part in one register.
__device__ __forceinline__ u32x4_t buffer_load16(rsrc_t r, uint32_t byte_offset, int fixed = 0) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, fixed, 0);
}
__device__ __forceinline__ float buffer_load_f32(rsrc_t r, uint32_t byte_offset) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, 0, 0));
}

#define HOLD_ORDER() __builtin_amdgcn_sched_barrier(0)   // nothing is scheduled across this point

#ifdef QVL_TIMELINE
// Measurement aid (never compiled into the package's library): every block's first wave stamps the
// device's 100 MHz clock at a few places into a buffer set by qvl_gemm_resident_timeline().
static unsigned long long* timeline_buffer = nullptr;
extern "C" void qvl_gemm_resident_timeline(void* p) { timeline_buffer = (unsigned long long*)p; }
#define STAMP(i)                                                                                    \
  do {                                                                                              \
    if (p.timeline && threadIdx.x == 0) p.timeline[blockIdx.x * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); \
  } while (0)
#else
#define STAMP(i)
#endif

#define W_RING 2   // half-step buffers of W that go round
#define RW 16   // waves per block
#ifndef RK
#define RK 8    // 32-wide K steps per wave and pass (the host loads a build with 4 for inner sizes up to 2,048: all 16 waves then have columns)
#endif
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
#ifdef QVL_TIMELINE
  unsigned long long* timeline;
#endif
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
  static_assert(MT == 1 || MT == 2, "one or two column tiles");
  __shared__ __attribute__((aligned(16))) float red[MT == 1 ? 2 : 1][RW][16 * COLS];
  __shared__ float rowsq[RW][16];
  __shared__ __attribute__((aligned(16))) float gains_own[(PRO == PRO_NORM && MT == 1) ? RW : 1][RK * 32];
  __shared__ u32x4_t xhi[(MT == 2 && ONE_PASS) ? XHI_STEPS * 64 : 1];
  float (*gains)[RK * 32] = MT == 1 ? gains_own : reinterpret_cast<float (*)[RK * 32]>(&red[0][0][0]);  // norm weights of each wave's columns
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  const int k_lane = wave * RK * 32 + 8 * lg;  // first K index of this lane within a pass
  STAMP(0);
  // how many of this lane's 32-wide steps of the pass that starts at k0 begin inside K (K is a
  // multiple of 8, as is every lane's first index: a step lies inside K or outside)
  auto steps_inside = [&](int k0) { return (p.K - k0 - k_lane + 31) >> 5; };
  // what the kernel reads, each behind a descriptor that knows its size (a null pointer: size 0)
  const rsrc_t w_buf = buffer_of(p.W, ((unsigned long long)(p.N - 1) * p.ldw + p.K) * 2);
  const rsrc_t x_buf = buffer_of(p.X, ((unsigned long long)(p.M - 1) * p.ldx + p.K) * 2);
  const rsrc_t h_buf = buffer_of(p.H, ((unsigned long long)(p.M - 1) * p.ldh + p.K) * 4);
  const rsrc_t gain_buf = buffer_of(p.norm_w, (unsigned long long)p.K * 4);
  const rsrc_t bias_buf = buffer_of(p.bias, (unsigned long long)p.N * 4);
  const rsrc_t old_buf = buffer_of(EPI == EPI_RESIDUAL ? p.out : nullptr, ((unsigned long long)(p.M - 1) * p.ldo + p.N) * 4);
  const rsrc_t cs_buf = buffer_of(p.cs, (unsigned long long)p.M * p.hd * 4);
  const rsrc_t slot_buf = buffer_of(p.slot, (unsigned long long)p.M * 4);
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
      const uint32_t at = m_ok ? ((uint32_t)row * p.ldx + k0 + k_lane) * 2 : PAST_END;
      const int inside = steps_inside(k0);
#pragma unroll
      for (int u = 0; u < RK; ++u)
        xb[u] = __builtin_bit_cast(bf16x8_t, buffer_load16(x_buf, u < inside ? at : PAST_END, u * 64));
    } else {
      // rmsnorm of the float32 rows: this pass covers all of K (ONE_PASS), so the block's waves
      // hold whole rows between them.  Loads return in the order they are issued: the rows and
      // the norm weights are asked for first and W (by first_w) right behind them, so the
      // statistics and the scaling run while W is still on its way.  A lane fetches 4 of its
      // wave's 32 RK norm weights (the first 8 RK lanes do); they reach the lanes that need them
      // through LDS.
      const uint32_t at = m_ok ? ((uint32_t)row * p.ldh + k_lane) * 4 : PAST_END;
      const int inside = steps_inside(0);
      float4 v[RK][2];
#pragma unroll
      for (int u = 0; u < RK; ++u) {
        const uint32_t o = u < inside ? at : PAST_END;
        v[u][0] = __builtin_bit_cast(float4, buffer_load16(h_buf, o, u * 128));
        v[u][1] = __builtin_bit_cast(float4, buffer_load16(h_buf, o, u * 128 + 16));
      }
      const int kg = wave * RK * 32 + 4 * lane;
      const bool gain_lane = 4 * lane < RK * 32;
      // beyond K the descriptor's own size gives zeros (K is a multiple of 8, kg of 4)
      const float4 g4 =
          __builtin_bit_cast(float4, buffer_load16(gain_buf, (again || !gain_lane) ? PAST_END : (uint32_t)kg * 4));
      first_w();
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < RK; ++u)
        ss += v[u][0].x * v[u][0].x + v[u][0].y * v[u][0].y + v[u][0].z * v[u][0].z + v[u][0].w * v[u][0].w +
              v[u][1].x * v[u][1].x + v[u][1].y * v[u][1].y + v[u][1].z * v[u][1].z + v[u][1].w * v[u][1].w;
      ss += __shfl_xor(ss, 16, QVL_WAVE);
      ss += __shfl_xor(ss, 32, QVL_WAVE);
      asm volatile("s_nop 0" ::"v"(ss));
      STAMP(6);   // this wave's rows have arrived
      if (again) __syncthreads();   // the other column tile's statistics have been read
      if (lg == 0) rowsq[wave][r] = ss;
      if (!again && gain_lane) *reinterpret_cast<float4*>(&gains[wave][4 * lane]) = g4;
      __syncthreads();
      STAMP(7);   // every wave's have
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < RW; ++w) total += rowsq[w][r];
      const float rs = 1.0f / sqrtf(total / (float)p.K + p.eps);
#pragma unroll
      for (int u = 0; u < RK; ++u) {
        if (u < inside) {
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
    // a tile beyond the last has no rows: all of its loads are asked for past the end
    const int row = tile < p.ntiles ? w_row(tile, r) : -1;
    const bool row_ok = r < tile_rows(tile) && row >= 0 && row < p.N;
    const uint32_t at = row_ok ? ((uint32_t)row * p.ldw + k0 + k_lane) * 2 : PAST_END;
    const int inside = steps_inside(k0);
#pragma unroll
    for (int u = 0; u < n; ++u)
      a[u] = __builtin_bit_cast(bf16x8_t, buffer_load16(w_buf, u0 + u < inside ? at : PAST_END, (u0 + u) * 64));
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
    if (EPI == EPI_SWIGLU) return e;
    // Every thread asks, the ones without an element past the end (and gets zeros): the same loads
    // on every path.  The waves beyond the first 16 COLS threads have no element at all.
    const int m = m0 + (threadIdx.x >> 4), nl = threadIdx.x & 15;
    const int n = tile < p.ntiles ? w_row(tile, nl) : -1;
    const bool live = threadIdx.x < 16 * COLS && m < p.M && nl < tile_rows(tile) && n >= 0 && n < p.N;
    e.bias = buffer_load_f32(bias_buf, live ? (uint32_t)n * 4 : PAST_END);
    if (EPI == EPI_RESIDUAL) e.old = buffer_load_f32(old_buf, live ? ((uint32_t)m * p.ldo + n) * 4 : PAST_END);
    if (EPI == EPI_ROPE) {
      const int head = live ? n / p.hd : 0, d = n - head * p.hd, half = p.hd >> 1;
      const bool turns = live && head < p.nq + p.nkv;
      const uint32_t at = turns ? ((uint32_t)m * half + (d < half ? d : d - half)) * 8 : PAST_END;
      e.cs = float2{buffer_load_f32(cs_buf, at), buffer_load_f32(cs_buf, at + 4)};
      if (!turns) e.cs = float2{1.f, 0.f};
      const int slot = __builtin_bit_cast(int, buffer_load_f32(slot_buf, (live && head >= p.nq) ? (uint32_t)m * 4 : PAST_END));
      e.slot = (live && head >= p.nq) ? slot : -1;
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
    const uint32_t at = m_ok ? ((uint32_t)row * p.ldx + k0 + k_lane) * 2 : PAST_END;
    const int inside = steps_inside(k0);
#pragma unroll
    for (int i = 0; i < RK / 2; ++i) {
      const int u = half * (RK / 2) + i;
      xb[u] = __builtin_bit_cast(bf16x8_t, buffer_load16(x_buf, u < inside ? at : PAST_END, u * 64));
    }
  };
  Acc zero;
#pragma unroll
  for (int t = 0; t < MT; ++t) zero.t[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  if (ONE_PASS || MT == 1) {
    // The block's work is a sequence of steps: every tile of its own, and within a tile every pass
    // over K (one, if X stays resident).  Two half-step buffers of W go round: each is asked for
    // again, for the next step, as soon as the product has freed its registers, and arrives during
    // the merge of the sums (or, between the passes of a tile, while the next rows of X come).
    const int passes = ONE_PASS ? 1 : (p.K + PASS_K - 1) / PASS_K;
    auto step_after = [&](int& t, int& ps) {
      if (++ps >= passes) {
        ps = 0;
        t += teams;
      }
    };
    bf16x8_t xb[RK];
    bf16x8_t w[W_RING][RK / 2];
    int tile = team, pass = 0;
    if (MT == 1) {
      load_x(0, 0, xb, [&] {
        load_w_part(tile, 0, 0, RK / 2, w[0]);
        load_w_part(tile, 0, RK / 2, RK / 2, w[1]);
      });
    } else {
      // rows 16..31 first, while few registers are taken: each lane keeps its own operands of
      // them in LDS and reads them back itself
      bf16x8_t hi[RK];
      load_x(1, 0, hi, [&] { load_w_part(tile, 0, 0, RK / 2, w[0]); });
#pragma unroll
      for (int u = 0; u < RK; ++u)
        if (hi_live) xhi[(wave * RK + u) * 64 + lane] = __builtin_bit_cast(u32x4_t, hi[u]);
      load_x(0, 0, xb, [&] { load_w_part(tile, 0, RK / 2, RK / 2, w[1]); }, true);
      if (PRO == PRO_NORM) __syncthreads();   // the norm weights lie where the first tile's sums go
    }
    STAMP(1);   // the rows are in their registers, the first tile asked for
    Epi e = epi_load(tile);
    Acc acc = zero;
    // one step whose halves are in a_lo and a_hi; false: it was the block's last
    // A half buffer is asked for again the moment its steps are multiplied (not after the whole
    // step).  Between the passes of a tile the next rows of X are asked for the same way, each half
    // ahead of the W half that is needed with it (loads come back in the order they were asked
    // for).  Every step issues the same loads, a step beyond the block's last one past the end of
    // the buffers.  (A ring of three half buffers, the free one taking the first half of the step
    // after next, needs more registers than a lane has: the compiler spills, and a spill's scratch
    // store makes every wait a wait for everything.)
    auto one = [&](bf16x8_t* a_lo, bf16x8_t* a_hi) {
      int tn = tile, pn = pass;
      step_after(tn, pn);
      const bool tile_done = ONE_PASS || pn == 0;
      // the order below is the order of the instructions: the compiler's scheduler would pull the
      // loads of later steps ahead of the products and run out of registers for them
      HOLD_ORDER();
      acc = product_part(a_lo, 0, RK / 2, xb, nullptr, acc);
      if (tile == team) { asm volatile("s_nop 0" :: "v"(acc.t[0])); STAMP(2); }   // the first half tile was there
      HOLD_ORDER();
      if (!ONE_PASS && MT == 1) load_x_half(pn * PASS_K, 0, xb);
      load_w_part(tn, pn * PASS_K, 0, RK / 2, a_lo);
      HOLD_ORDER();
      acc = product_part(a_hi, RK / 2, RK / 2, xb, nullptr, acc);
      HOLD_ORDER();
      const Epi e_next = epi_load(tn);
      if (!ONE_PASS && MT == 1) load_x_half(pn * PASS_K, 1, xb);
      load_w_part(tn, pn * PASS_K, RK / 2, RK / 2, a_hi);
      HOLD_ORDER();
      if (tile_done) {
        if (tile == team) STAMP(3);   // all of the first tile multiplied
        finish(tile, acc, e);
        if (tile == team) STAMP(4);   // and merged and written
        acc = zero;
        e = e_next;
      }
      tile = tn;
      pass = pn;
      return tn < p.ntiles;
    };
    while (tile < p.ntiles) {
      if (!one(w[0], w[1])) break;
    }
    STAMP(5);
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
// per group) is refused (mt = 0).
struct Plan {
  int mt, groups;
  bool one_pass;
};
static Plan plan_for(int M, int K, bool norm, int blocks) {
  if (M <= 16) return Plan{1, 1, K <= PASS_K};
  const bool two_fit = K <= 32 * XHI_STEPS;
  if (M <= 32 && two_fit) return Plan{2, 1, true};
  if (two_fit && blocks >= 8 * ((M + 31) / 32)) return Plan{2, (M + 31) / 32, true};
  const int singles = (M + 15) / 16;
  if ((M > 32 || norm) && blocks >= 8 * singles) return Plan{1, singles, K <= PASS_K};
  if (M <= 32) return Plan{2, 1, false};
  return Plan{0, 1, false};
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
  const Plan pl = plan_for(M, K, true, blocks);
  return pl.one_pass && pl.mt <= 2;
}

// Whether every operand lies within what a buffer descriptor and a 32-bit byte offset reach.
static bool fits_descriptors(long long M, long long N, long long K, long long ldw, long long ldx, long long ldh,
                             long long ldo) {
  const unsigned long long w = ((N - 1) * ldw + K) * 2ull, x = ((M - 1) * ldx + K) * 2ull,
                           h = ((M - 1) * ldh + K) * 4ull, o = ((M - 1) * ldo + N) * 4ull;
  return w < BUFFER_LIMIT && x < BUFFER_LIMIT && h < BUFFER_LIMIT && o < BUFFER_LIMIT;
}
// The most bytes a weight matrix may span ((N - 1) ldw + K elements of two bytes).
extern "C" unsigned long long qvl_gemm_resident_max_weight_bytes() { return BUFFER_LIMIT - 1; }

extern "C" int qvl_gemm_resident_pass_k() { return PASS_K; }
// the longest K with which 17 to 32 rows stay resident (and with which their norm is folded in)
extern "C" int qvl_gemm_resident_two_tile_k() { return 32 * XHI_STEPS; }

// x: bfloat16 [M, K] (h null), or h: float32 [M, K] with norm_w [K] and eps (x null): X = rmsnorm(h) * norm_w.
// epilogue 0: out[M, N] in out_dtype (0 float32, 1 bfloat16); 1: out (float32 [M, N]) += product;
// 2: out[M, N/2] bfloat16 = silu(gate) * up for W rows in groups of 8 gate, 8 up.
// max_blocks: blocks to launch at most (the number of compute units).
extern "C" int qvl_gemm_resident(const void* x, int ldx, const void* h, int ldh, const void* norm_w, float eps,
                                 const void* W, int ldw, const void* bias, void* out, int ldo, int M, int N, int K,
                                 int out_dtype, int epilogue, int max_blocks, hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (M > 64) return QVL_ERR_LIMIT;
  if (M > 32 && K > PASS_K) return QVL_ERR_LIMIT;   // teams of more than two keep their rows for a single pass
  if (K <= 0 || K % 8 || ldw % 8 || ldw < K || max_blocks <= 0 || !W || !out) return QVL_ERR_SHAPE;
  if (!fits_descriptors(M, N, K, ldw, ldx, ldh, ldo)) return QVL_ERR_LIMIT;
  const bool norm = h != nullptr;
  const Plan pl = plan_for(M, K, norm, max_blocks);
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
#ifdef QVL_TIMELINE
  p.timeline = timeline_buffer;
#endif
  p.cs = nullptr; p.slot = nullptr;
  p.q_out = nullptr; p.kc = nullptr; p.vc = nullptr; p.nq = p.nkv = p.hd = p.ps = 0; p.pair_tiles = 0;
  // as many rounds of tiles as 16-row tiles need, with rows per tile cut down to what fills them evenly
  p.rows = 16;
  if (epilogue != EPI_SWIGLU) {
    const long long per_round = 16LL * teams;
    const long long rounds = (N + per_round - 1) / per_round;   // (more rounds of shorter tiles lose: a load instruction then carries fewer rows)
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
  if (nq <= 0 || nkv < 0 || hd <= 0) return QVL_ERR_SHAPE;
  if (!fits_descriptors(M, (nq + 2 * nkv) * hd, K, ldw, ldx, ldh, 0)) return QVL_ERR_LIMIT;
  if (nq <= 0 || nkv < 0 || hd <= 0 || hd % 16 || ps <= 0 || !cs) return QVL_ERR_SHAPE;
  if (nkv > 0 && (!slot || !kc || !vc)) return QVL_ERR_SHAPE;
  const bool norm = h != nullptr;
  const Plan pl = plan_for(M, K, norm, max_blocks);
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
#ifdef QVL_TIMELINE
  p.timeline = timeline_buffer;
#endif
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
