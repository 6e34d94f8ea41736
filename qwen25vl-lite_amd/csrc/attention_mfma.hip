// Paged attention on the matrix cores: bfloat16 storage, head size HD (a multiple of 16, set at
// compile time with -DHD=...), float32 softmax.  One kernel serves prompt portions and decoded
// tokens of a mixed batch.
//
// Work is cut into tiles of 16 "columns" of one request and one key/value head.  A column is a
// (token of this step, query head of the group) pair, token-major, so the group's heads share
// every key and value that is loaded.  One wave owns a tile and walks the request's keys in
// blocks of 32 by absolute index, with two kinds of v_mfma_f32_16x16x32_bf16 per block:
//
//   S^T[key, col]  = K[key, :] . Q[col, :]        A = keys x dims,   B = dims x columns
//   O^T[dim, col] += V^T[dim, key] . P^T[key, col] A = dims x keys,   B = keys x columns
//
// Computing the transposes keeps a column in one lane (lane % 16) through both products: the
// softmax statistics of a column live in that lane, and the probabilities come out of the first
// product in the register layout the second wants as its B operand, if the 16 rows of the two
// key blocks are permuted so that lane group g = lane / 16 ends up with the 8 consecutive keys
// 8g .. 8g+7.  Keys are stored [page][kv head][slot][HD] and values transposed,
// [page][kv head][HD][slot], so both A operands are plain 16-byte loads from the pages.
//
// Two kernels use this walk.  With many tiles (prompt portions) every wave owns a tile.  With
// few tiles (decode) the waves of a block share one tile and merge through LDS; for very long
// contexts the keys are further split among blocks, whose partial sums a second kernel merges.
#include "common.h"

#ifndef HD
#error "compile with -DHD=<head size>"
#endif
#if HD % 16 != 0 || HD < 16 || HD > 256
#error "HD must be a multiple of 16 between 16 and 256"
#endif

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define KS ((HD + 31) / 32)  // 32-wide steps over the head for Q.K
#define NT (HD / 16)         // 16-wide tiles of the head for P.V
#define LOG2E 1.4426950408889634f

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(p));
}
__device__ __forceinline__ bf16x8_t zero8() {
  u32x4_t z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8_t, z);
}
// Two floats to two bfloat16 (round to nearest even) in one word; the compiler uses the packed
// hardware conversion of gfx950.
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  bf16x2_t v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}

struct TileState {
  float m, l;
  f32x4_t acc[NT];
};

// The page of each key row this lane loads in one 32-key block (two K row blocks, one V group).
struct BlockPages {
  int k[2], v;
};
// One 32-key block in registers: K rows as A operands of S^T, V^T rows as A operands of O^T.
struct BlockRegs {
  bf16x8_t k[2][KS];
  bf16x8_t v[NT];
};

// CT: column tiles (of 16 columns) a wave carries through the walk; every key block it loads is
// used for all of them.
template <int CT>
struct Walk {
  const bf16_t* kc;
  const bf16_t* vc;
  const int* bt;  // this request's row of the block table
  int max_key, nkv, kvh, ps;
  int my_lo[CT], my_p[CT], key_begin, key_end;
  int all_lo, all_hi;  // keys all_lo .. all_hi are seen by every column of the wave
  float scale_log2;
  int lg, r;

  // Row r of K block b holds key 8*(r/4) + 4b + r%4, so that after the product lane group lg
  // holds the 8 consecutive keys 8*lg .. 8*lg+7 (see the top of the file).
  __device__ __forceinline__ int krow_key(int kb, int b) const { return (kb << 5) + 8 * (r >> 2) + 4 * b + (r & 3); }

  __device__ __forceinline__ void issue_pages(int kb, BlockPages& pg) const {
#pragma unroll
    for (int b = 0; b < 2; ++b) pg.k[b] = bt[min(krow_key(kb, b), max_key) / ps];
    pg.v = bt[min((kb << 5) + 8 * lg, max_key) / ps];
  }

  __device__ __forceinline__ void issue_loads(int kb, const BlockPages& pg, BlockRegs& rg) const {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int key = krow_key(kb, b);
      const int page = pg.k[b] < 0 ? 0 : pg.k[b];  // keys nobody sees may have no page: read page 0, masked later
      const bf16_t* krow = kc + (((size_t)page * nkv + kvh) * ps + (size_t)(key % ps)) * HD;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + 8 * lg;
        rg.k[b][ks] = (d < HD) ? load8(krow + d) : zero8();
      }
    }
    const int vkey = (kb << 5) + 8 * lg;
    const int vpage = (pg.v < 0 || vkey > max_key) ? 0 : pg.v;
    const bf16_t* vbase = vc + (((size_t)vpage * nkv + kvh) * HD) * ps + (size_t)(vkey % ps);
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) rg.v[dt] = load8(vbase + (size_t)(dt * 16 + r) * ps);
  }

  __device__ __forceinline__ void compute(int kb, const bf16x8_t (*qb)[KS], const BlockRegs& rg, TileState* sts) const {
    const int key0 = kb << 5;
    const bool interior = key0 >= all_lo && key0 + 31 <= all_hi;
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      TileState& st = sts[t];
      f32x4_t s[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        f32x4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rg.k[b][ks], qb[t][ks], a, 0, 0, 0);
        s[b] = a;
      }
      // mask and online softmax; this lane holds keys key0 + 8*lg + j of column r.  A block that
      // lies wholly inside what every column of the wave sees needs no mask.
      float sv[8];
      float mloc = -INFINITY;
      if (interior) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          sv[j] = ((j < 4) ? s[0][j] : s[1][j - 4]) * scale_log2;
          mloc = fmaxf(mloc, sv[j]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = key0 + 8 * lg + j;
          const float raw = (j < 4) ? s[0][j] : s[1][j - 4];
          const bool ok = key >= my_lo[t] && key <= my_p[t] && key >= key_begin && key <= key_end;
          sv[j] = ok ? raw * scale_log2 : -INFINITY;
          mloc = fmaxf(mloc, sv[j]);
        }
      }
      mloc = fmaxf(mloc, __shfl_xor(mloc, 16, QVL_WAVE));
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, QVL_WAVE));
      const float m_new = fmaxf(st.m, mloc);
      float alpha = 1.f, psum = 0.f;
      float pv[8];
      if (m_new == -INFINITY) {
#pragma unroll
        for (int j = 0; j < 8; ++j) pv[j] = 0.f;
      } else {
        alpha = __builtin_amdgcn_exp2f(st.m - m_new);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          pv[j] = __builtin_amdgcn_exp2f(sv[j] - m_new);
          psum += pv[j];
        }
      }
      psum += __shfl_xor(psum, 16, QVL_WAVE);
      psum += __shfl_xor(psum, 32, QVL_WAVE);
      st.l = st.l * alpha + psum;
      st.m = m_new;
      // the running maximum rarely moves after the first blocks: skip the rescaling when no
      // column of the wave needs it
      const bool rescale = __any(alpha != 1.f);
      u32x4_t packed = {pack2(pv[0], pv[1]), pack2(pv[2], pv[3]), pack2(pv[4], pv[5]), pack2(pv[6], pv[7])};
      const bf16x8_t pb = __builtin_bit_cast(bf16x8_t, packed);
      if (rescale) {
#pragma unroll
        for (int dt = 0; dt < NT; ++dt) {
          f32x4_t o = st.acc[dt];
          o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
          st.acc[dt] = o;
        }
      }
#pragma unroll
      for (int dt = 0; dt < NT; ++dt)
        st.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rg.v[dt], pb, st.acc[dt], 0, 0, 0);
    }
  }
};

// Walk the 32-key blocks first, first + stride, ... that overlap keys [key_begin, key_end]
// (inclusive, absolute) of one tile.  The loads of the next block and the page lookups of the one
// after are issued before the current block is computed, so a wave always has a block in flight.
template <int CT>
__device__ __forceinline__ void attend(const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
                                       const int* __restrict__ bt, int table_width, int nkv, int kvh, int ps,
                                       const bf16x8_t (*qb)[KS], const int* my_lo, const int* my_p, float scale_log2,
                                       int key_begin, int key_end, int kb_offset, int kb_stride, TileState* st) {
  const int lane = threadIdx.x & 63;
  Walk<CT> w;
  w.kc = kc; w.vc = vc; w.bt = bt;
  w.max_key = table_width * ps - 1; w.nkv = nkv; w.kvh = kvh; w.ps = ps;
#pragma unroll
  for (int t = 0; t < CT; ++t) { w.my_lo[t] = my_lo[t]; w.my_p[t] = my_p[t]; }
  w.key_begin = key_begin; w.key_end = key_end;
  w.scale_log2 = scale_log2; w.lg = lane >> 4; w.r = lane & 15;
  {  // the range every column sees: largest first key and smallest last key over all lanes and tiles
    int lo = key_begin, hi = key_end;
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      if (my_p[t] >= 0) {  // a lane without a column computes on zeros and stores nothing
        lo = max(lo, my_lo[t]);
        hi = min(hi, my_p[t]);
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      lo = max(lo, __shfl_xor(lo, o, QVL_WAVE));
      hi = min(hi, __shfl_xor(hi, o, QVL_WAVE));
    }
    w.all_lo = lo;
    w.all_hi = hi;
  }
  const int s = kb_stride;
  int kb = (key_begin >> 5) + kb_offset;
#define LIVE(x) (((x) << 5) <= key_end)
  if (!LIVE(kb)) return;
  BlockPages p0, p1;
  BlockRegs ra, rb;
  w.issue_pages(kb, p0);
  if (LIVE(kb + s)) w.issue_pages(kb + s, p1);
  w.issue_loads(kb, p0, ra);
  for (;; kb += 2 * s) {
    if (LIVE(kb + 2 * s)) w.issue_pages(kb + 2 * s, p0);
    if (LIVE(kb + s)) w.issue_loads(kb + s, p1, rb);
    w.compute(kb, qb, ra, st);
    if (!LIVE(kb + s)) break;
    if (LIVE(kb + 3 * s)) w.issue_pages(kb + 3 * s, p1);
    if (LIVE(kb + 2 * s)) w.issue_loads(kb + 2 * s, p0, ra);
    w.compute(kb + s, qb, rb, st);
    if (!LIVE(kb + 2 * s)) break;
  }
#undef LIVE
}

// Everything a wave needs to know about its tile.
struct TileInfo {
  bool valid;      // this lane's column exists
  int token;       // row of q / out
  int head;        // query head
  int my_lo, my_p; // first and last key this lane's column sees
  int lo_tile, hi_tile;
};

__device__ __forceinline__ TileInfo tile_info(const int* cu_q, const int* ctx_len, int r, int ct, int g, int kvh,
                                              int window) {
  const int lane = threadIdx.x & 63, c = lane & 15;
  const int q0 = cu_q[r], qlen = cu_q[r + 1] - q0, ctx = ctx_len[r];
  const int col = ct * 16 + c;
  const int i = col / g, gh = col - i * g;
  TileInfo t;
  t.valid = i < qlen;
  t.token = q0 + (t.valid ? i : 0);
  t.head = kvh * g + gh;
  const int p = ctx - qlen + (t.valid ? i : 0);
  t.my_p = t.valid ? p : -1;
  t.my_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int i_first = (ct * 16) / g;
  int i_last = (ct * 16 + 15) / g;
  i_last = i_last < qlen - 1 ? i_last : qlen - 1;
  const int p_first = ctx - qlen + i_first;
  t.lo_tile = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  t.hi_tile = ctx - qlen + i_last;
  return t;
}

__device__ __forceinline__ void load_q(const bf16_t* __restrict__ q, int nq, const TileInfo& t, bf16x8_t* qb) {
  const int lg = (threadIdx.x & 63) >> 4;
  const bf16_t* qrow = q + ((size_t)t.token * nq + t.head) * HD;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + 8 * lg;
    qb[ks] = (t.valid && d < HD) ? load8(qrow + d) : zero8();
  }
}

// Column tiles per wave in the kernel for many tiles: every key block a wave loads serves two tiles.
#define TILE_CT 2

__device__ __forceinline__ void init_state(TileState& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) st.acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
}

// tile_ct counts in units of TILE_CT column tiles here.
__global__ __launch_bounds__(256) void attn_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc,
                                                        const bf16_t* __restrict__ vc, const int* __restrict__ bt,
                                                        int table_width, const int* __restrict__ cu_q,
                                                        const int* __restrict__ ctx_len,
                                                        const int* __restrict__ tile_req,
                                                        const int* __restrict__ tile_ct, int num_tiles,
                                                        bf16_t* __restrict__ out, int nq, int nkv, int ps, int window,
                                                        float scale) {
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= num_tiles) return;
  const int kvh = blockIdx.y, g = nq / nkv;
  const int r = tile_req[item], ct0 = tile_ct[item] * TILE_CT;
  const int ncols = (cu_q[r + 1] - cu_q[r]) * g;
  TileInfo t[TILE_CT];
  bf16x8_t qb[TILE_CT][KS];
  TileState st[TILE_CT];
  int my_lo[TILE_CT], my_p[TILE_CT];
  int lo = 0x7fffffff, hi = -1;
#pragma unroll
  for (int i = 0; i < TILE_CT; ++i) {
    const bool exists = (ct0 + i) * 16 < ncols;   // the last pair of a request may have one tile only
    t[i] = tile_info(cu_q, ctx_len, r, exists ? ct0 + i : ct0, g, kvh, window);
    if (!exists) { t[i].valid = false; t[i].my_p = -1; }
    load_q(q, nq, t[i], qb[i]);
    init_state(st[i]);
    my_lo[i] = t[i].my_lo;
    my_p[i] = t[i].my_p;
    if (exists) {
      lo = t[i].lo_tile < lo ? t[i].lo_tile : lo;
      hi = t[i].hi_tile > hi ? t[i].hi_tile : hi;
    }
  }
  attend<TILE_CT>(kc, vc, bt + (size_t)r * table_width, table_width, nkv, kvh, ps, qb, my_lo, my_p, scale * LOG2E, lo,
                  hi, 0, 1, st);
  const int lg = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int i = 0; i < TILE_CT; ++i) {
    if (!t[i].valid) continue;
    const float inv = 1.0f / st[i].l;
    bf16_t* orow = out + ((size_t)t[i].token * nq + t[i].head) * HD;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) {
      const int d = dt * 16 + 4 * lg;
      uint2 w;
      w.x = pack2(st[i].acc[dt][0] * inv, st[i].acc[dt][1] * inv);
      w.y = pack2(st[i].acc[dt][2] * inv, st[i].acc[dt][3] * inv);
      *reinterpret_cast<uint2*>(orow + d) = w;
    }
  }
}

// ---- few tiles (decode): the waves of a block share one tile ---------------------------------
// The COOP_WAVES waves of a block take the tile's 32-key blocks in turn (wave w the blocks
// w, w + COOP_WAVES, ...), then merge their sums and statistics through LDS in wave order.  With
// nsplit > 1 the key range is further cut among blocks (grid.z); each block then writes its
// merged partial to scratch and a second kernel merges the splits.
// scratch layout per (tile, kv head, split): 16 columns x PART_COLS floats (HD sums, m, l, and
// padding that keeps every column 16-byte aligned).
#define PART_COLS (HD + 4)
#define PART_STRIDE (16 * PART_COLS)
#if HD <= 128
#define COOP_WAVES 4
#else
#define COOP_WAVES 2
#endif

__global__ __launch_bounds__(64 * COOP_WAVES) void attn_mfma_coop_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int* __restrict__ bt, int table_width, const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    const int* __restrict__ tile_req, const int* __restrict__ tile_ct, bf16_t* __restrict__ out,
    float* __restrict__ scratch, int nq, int nkv, int ps, int window, float scale, int nsplit, int keys_per_split) {
  __shared__ __attribute__((aligned(16))) float sm[COOP_WAVES][PART_STRIDE];
  const int tile = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, c = lane & 15;
  const int g = nq / nkv;
  const int r = tile_req[tile], ct = tile_ct[tile];
  const TileInfo t = tile_info(cu_q, ctx_len, r, ct, g, kvh, window);
  int first = t.lo_tile, last = t.hi_tile;
  if (nsplit > 1) {  // splits are cut by absolute key index, in multiples of 32
    first = (t.lo_tile >> 5 << 5) + split * keys_per_split;
    last = first + keys_per_split - 1;
    last = last < t.hi_tile ? last : t.hi_tile;
    first = first > t.lo_tile ? first : t.lo_tile;
  }
  TileState st;
  init_state(st);
  if (first <= last) {
    bf16x8_t qb[1][KS];
    load_q(q, nq, t, qb[0]);
    attend<1>(kc, vc, bt + (size_t)r * table_width, table_width, nkv, kvh, ps, qb, &t.my_lo, &t.my_p, scale * LOG2E,
              first, last, wave, COOP_WAVES, &st);
  }
  // every wave leaves its column sums in LDS: column c, channels dt*16 + 4*lg .. +3, then m and l
  float* mine = &sm[wave][c * PART_COLS];
#pragma unroll
  for (int dt = 0; dt < NT; ++dt)
    *reinterpret_cast<float4*>(mine + dt * 16 + 4 * lg) =
        float4{st.acc[dt][0], st.acc[dt][1], st.acc[dt][2], st.acc[dt][3]};
  if (lg == 0) {
    mine[HD] = st.m;
    mine[HD + 1] = st.l;
  }
  __syncthreads();
  // merge: thread -> (column, 4 channels); waves are summed in order 0, 1, ...
  for (int idx = threadIdx.x; idx < 16 * (HD / 4); idx += blockDim.x) {
    const int col = idx / (HD / 4), d = (idx - col * (HD / 4)) * 4;
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < COOP_WAVES; ++w) m = fmaxf(m, sm[w][col * PART_COLS + HD]);
    float4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
#pragma unroll
    for (int w = 0; w < COOP_WAVES; ++w) {
      const float* p = &sm[w][col * PART_COLS];
      const float wgt = (p[HD] == -INFINITY) ? 0.f : exp2f(p[HD] - m);
      const float4 a = *reinterpret_cast<const float4*>(p + d);
      num.x += wgt * a.x; num.y += wgt * a.y; num.z += wgt * a.z; num.w += wgt * a.w;
      den += wgt * p[HD + 1];
    }
    const int colg = ct * 16 + col;
    const int i = colg / g, gh = colg - i * g;
    const int q0 = cu_q[r], qlen = cu_q[r + 1] - q0;
    if (nsplit > 1) {
      float* part = scratch + (((size_t)tile * nkv + kvh) * nsplit + split) * PART_STRIDE + (size_t)col * PART_COLS;
      *reinterpret_cast<float4*>(part + d) = num;
      if (d == 0) {
        part[HD] = m;
        part[HD + 1] = den;
      }
    } else if (i < qlen) {
      const float inv = 1.0f / den;
      uint2 wv;
      wv.x = pack2(num.x * inv, num.y * inv);
      wv.y = pack2(num.z * inv, num.w * inv);
      *reinterpret_cast<uint2*>(out + ((size_t)(q0 + i) * nq + kvh * g + gh) * HD + d) = wv;
    }
  }
}

__global__ void attn_mfma_merge_kernel(const float* __restrict__ scratch, const int* __restrict__ cu_q,
                                       const int* __restrict__ tile_req, const int* __restrict__ tile_ct,
                                       bf16_t* __restrict__ out, int nq, int nkv, int nsplit) {
  // one block per (tile, kv head); thread -> (column, 4 channels); splits are summed in order
  const int tile = blockIdx.x, kvh = blockIdx.y, g = nq / nkv;
  const int r = tile_req[tile], ct = tile_ct[tile];
  const int q0 = cu_q[r], qlen = cu_q[r + 1] - q0;
  const float* base = scratch + ((size_t)tile * nkv + kvh) * nsplit * PART_STRIDE;
  for (int idx = threadIdx.x; idx < 16 * (HD / 4); idx += blockDim.x) {
    const int col = idx / (HD / 4), d = (idx - col * (HD / 4)) * 4;
    const int colg = ct * 16 + col;
    const int i = colg / g, gh = colg - i * g;
    if (i >= qlen) continue;
    float m = -INFINITY;
    for (int s = 0; s < nsplit; ++s) m = fmaxf(m, base[(size_t)s * PART_STRIDE + col * PART_COLS + HD]);
    float4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float* p = base + (size_t)s * PART_STRIDE + col * PART_COLS;
      const float wgt = (p[HD] == -INFINITY) ? 0.f : exp2f(p[HD] - m);
      const float4 a = *reinterpret_cast<const float4*>(p + d);
      num.x += wgt * a.x; num.y += wgt * a.y; num.z += wgt * a.z; num.w += wgt * a.w;
      den += wgt * p[HD + 1];
    }
    const float inv = 1.0f / den;
    uint2 wv;
    wv.x = pack2(num.x * inv, num.y * inv);
    wv.y = pack2(num.z * inv, num.w * inv);
    *reinterpret_cast<uint2*>(out + ((size_t)(q0 + i) * nq + kvh * g + gh) * HD + d) = wv;
  }
}

static int check_common(int num_tiles, int nq, int nkv, int ps, int table_width) {
  if (num_tiles <= 0) return QVL_OK;
  if (nq <= 0 || nkv <= 0 || nq % nkv || ps <= 0 || ps % 16 || table_width <= 0) return QVL_ERR_SHAPE;
  if (nkv > 65535) return QVL_ERR_LIMIT;
  return -1;
}

extern "C" int qvl_attn_mfma_head_dim() { return HD; }
// Column tiles per entry of the tile list that qvl_attn_mfma expects (qvl_attn_mfma_coop: 1).
extern "C" int qvl_attn_mfma_tile_ct() { return TILE_CT; }

extern "C" int qvl_attn_mfma(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                             const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                             int num_tiles, void* out, int nq, int nkv, int ps, int window, float scale,
                             hipStream_t stream) {
  const int c = check_common(num_tiles, nq, nkv, ps, table_width);
  if (c >= 0) return c;
  const dim3 grid((num_tiles + 3) / 4, nkv);
  hipLaunchKernelGGL(attn_mfma_kernel, grid, dim3(256), 0, stream, (const bf16_t*)q, (const bf16_t*)kc,
                     (const bf16_t*)vc, (const int*)bt, table_width, (const int*)cu_q, (const int*)ctx_len,
                     (const int*)tile_req, (const int*)tile_ct, num_tiles, (bf16_t*)out, nq, nkv, ps, window, scale);
  return qvl_launch_status();
}

// Floats the scratch buffer of a split call must hold.
extern "C" long long qvl_attn_mfma_scratch_floats(int num_tiles, int nkv, int nsplit) {
  return (long long)num_tiles * nkv * nsplit * PART_STRIDE;
}

extern "C" int qvl_attn_mfma_coop(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                                  const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                                  int num_tiles, void* out, void* scratch, int nq, int nkv, int ps, int window,
                                  float scale, int nsplit, int keys_per_split, hipStream_t stream) {
  const int c = check_common(num_tiles, nq, nkv, ps, table_width);
  if (c >= 0) return c;
  if (nsplit <= 0 || nsplit > 65535 || (nsplit > 1 && (keys_per_split <= 0 || keys_per_split % 32 || !scratch)))
    return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(attn_mfma_coop_kernel, dim3(num_tiles, nkv, nsplit), dim3(64 * COOP_WAVES), 0, stream,
                     (const bf16_t*)q, (const bf16_t*)kc, (const bf16_t*)vc, (const int*)bt, table_width,
                     (const int*)cu_q, (const int*)ctx_len, (const int*)tile_req, (const int*)tile_ct, (bf16_t*)out,
                     (float*)scratch, nq, nkv, ps, window, scale, nsplit, keys_per_split);
  if (hipGetLastError() != hipSuccess) return QVL_ERR_LAUNCH;
  if (nsplit > 1)
    hipLaunchKernelGGL(attn_mfma_merge_kernel, dim3(num_tiles, nkv), dim3(256), 0, stream, (const float*)scratch,
                       (const int*)cu_q, (const int*)tile_req, (const int*)tile_ct, (bf16_t*)out, nq, nkv, nsplit);
  return qvl_launch_status();
}
