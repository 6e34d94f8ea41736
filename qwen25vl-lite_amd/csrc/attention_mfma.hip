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
// Two kernels use this arithmetic.  With many tiles (prompt portions) a block owns several tiles
// per wave and fetches every key block once, through LDS, for all of them.  With few tiles
// (decode) the waves of a block share one tile, each loading its own key blocks straight into
// registers, and merge through LDS; for very long contexts the keys are further split among
// blocks, whose partial sums a second kernel merges.
#include "common.h"
#include <type_traits>
#include "attention_mfma.h"
#include <atomic>
#include <mutex>

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
// The layout of a stage of the kernel for many tiles in LDS (described where that kernel begins).
#define CH_PER_KEY (HD / 8)                                       // 16-byte chunks of a key
#define KROW (HD + 8)                                             // elements of a K row in LDS
#define K_SKEW ((4 * (CH_PER_KEY + 1)) % 16)                      // 16-byte slots by which the second half's rows are set off
#define KH_LOADS ((16 * (CH_PER_KEY + 1) + K_SKEW + 63) / 64)     // 1 KB wave loads that cover the K rows of one half
#define K_LOADS (2 * KH_LOADS)
#define V_HALF_SLOTS ((2 * HD + 63) / 64 * 64)                    // slots of one half of the V^T rows (whole loads)
#define VH_LOADS (V_HALF_SLOTS / 64)
#define V_LOADS (2 * VH_LOADS)
#define STAGE_LOADS (K_LOADS + V_LOADS)
#define WAVE_LOADS (KH_LOADS > VH_LOADS ? KH_LOADS : VH_LOADS)    // what a wave issues a block: one of the four parts of a stage
#define STAGE_ELEMS (STAGE_LOADS * 512)
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

// A column's four lanes are r, r + 16, r + 32, r + 48.  v_permlane16_swap exchanges the odd rows
// of 16 lanes of its first operand with the even rows of its second, v_permlane32_swap the upper
// half of the first with the lower half of the second: with both operands equal, the two results
// hold each pair's two values in both lanes of the pair.
__device__ __forceinline__ bf16x8_t ones8() {
  const u32x4_t one = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  return __builtin_bit_cast(bf16x8_t, one);
}
__device__ __forceinline__ float max2(float a, float b);
__device__ __forceinline__ float max_over_groups(float v) {
  const uint32_t b = __builtin_bit_cast(uint32_t, v);
  const auto x = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  v = max2(__builtin_bit_cast(float, (uint32_t)x[0]), __builtin_bit_cast(float, (uint32_t)x[1]));
  const uint32_t c = __builtin_bit_cast(uint32_t, v);
  const auto y = __builtin_amdgcn_permlane32_swap(c, c, false, false);
  return max2(__builtin_bit_cast(float, (uint32_t)y[0]), __builtin_bit_cast(float, (uint32_t)y[1]));
}
__device__ __forceinline__ float sum_over_groups(float v) {
  const uint32_t b = __builtin_bit_cast(uint32_t, v);
  const auto x = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  v = __builtin_bit_cast(float, (uint32_t)x[0]) + __builtin_bit_cast(float, (uint32_t)x[1]);
  const uint32_t c = __builtin_bit_cast(uint32_t, v);
  const auto y = __builtin_amdgcn_permlane32_swap(c, c, false, false);
  return __builtin_bit_cast(float, (uint32_t)y[0]) + __builtin_bit_cast(float, (uint32_t)y[1]);
}
// IEEE maximum (a NaN would come through; there is none): one v_maximum3_f32 for up to three values,
// where fmaxf first makes each input canonical.
__device__ __forceinline__ float max2(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// Softmax state of a column.  m is the reference the exponentials are taken against, in the
// log2 domain (score * scale * log2 e).  It follows the running maximum lazily: it moves only
// when a block's maximum exceeds it by more than LAZY_LOG2, so the sums are rarely rescaled and
// no exponential exceeds 2^LAZY_LOG2; softmax does not depend on the reference.
#define LAZY_LOG2 8.0f
struct TileState {
  float m, l;            // l: this lane's share of the column's sum of probabilities (its 8 keys of every block), if the lanes add
  f32x4_t acc[NT + 1];   // acc[NT]: the column's sum of probabilities in every row, if the matrix cores add (see Walk::compute)
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
__device__ __forceinline__ void load16_to_lds(const char* base, uint32_t lane_bytes, uint32_t stage, uint32_t offset);

// Keys through LDS (the kernel for few tiles, head size 128).  Read straight into operand
// registers, a wave's key load covers 16 rows of 64 bytes, 256 bytes apart: a compute unit fetches
// a third slower that way than with loads that cover 1 KB contiguous (36 against 54 GB/s by
// itself).  So a wave brings the 32 keys of a block into 8 KB of LDS of its own with eight loads of
// 1 KB each (straight into LDS, no registers on the way) and reads its operands from there.  Row
// kappa of the block keeps its 16-byte chunk c at place c ^ f(kappa), f = the row of the
// matrix-core tile that key has (bits 4, 3, 1, 0 of kappa: the 16 keys one operand read touches
// have 16 different f), so the 16 lanes of an operand read hit 16 different places of the 256-byte
// bank period.  The lane that fills place s of row kappa fetches chunk s ^ f(kappa).
#define K_VIA_LDS (HD == 128)
struct HalfPages {
  int page[2], off[2];   // of the two 16-key halves of a block: the same for every lane
};

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

  // the table entries of a block's two halves (a page holds a multiple of 16 keys: a half lies in one page)
  __device__ __forceinline__ void issue_half_pages(int kb, HalfPages& hp) const {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int key = (kb << 5) + 16 * h, idx = min(key, max_key) / ps;
      hp.page[h] = bt[idx];
      hp.off[h] = key % ps;
    }
  }
  // this lane's byte offset within a half's 4 KB for the load that fills its place (see above), less the constant part
  __device__ __forceinline__ uint32_t lds_lane_offset() const {
    const uint32_t l = threadIdx.x & 63, i = l >> 4;
    return i * 256u + (((l & 15u) ^ i) << 4);
  }
  __device__ __forceinline__ void issue_k_to_lds(const HalfPages& hp, uint32_t stage, uint32_t lane_off) const {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int page = __builtin_amdgcn_readfirstlane(hp.page[h] < 0 ? 0 : hp.page[h]);   // no page: nobody sees these keys
      const int off = __builtin_amdgcn_readfirstlane(hp.off[h]);
      const char* from = reinterpret_cast<const char*>(kc + (((size_t)page * nkv + kvh) * ps + (size_t)off) * HD);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t f_fixed = (uint32_t)((h << 3) | ((j >> 1) << 2));
        load16_to_lds(from + j * 1024, lane_off ^ (f_fixed << 4), stage, (uint32_t)(h * 4 + j) * 1024u);
      }
    }
  }
  __device__ __forceinline__ void k_from_lds(const char* staged, BlockRegs& rg) const {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int kappa = 8 * (r >> 2) + 4 * b + (r & 3);
      const int f = ((kappa >> 4) << 3) | (((kappa >> 3) & 1) << 2) | (kappa & 3);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        rg.k[b][ks] = *reinterpret_cast<const bf16x8_t*>(staged + kappa * 256 + (((ks * 4 + lg) ^ f) << 4));
    }
  }
  __device__ __forceinline__ void issue_v(int kb, const BlockPages& pg, BlockRegs& rg) const {
    const int vkey = (kb << 5) + 8 * lg;
    const int vpage = (pg.v < 0 || vkey > max_key) ? 0 : pg.v;
    const bf16_t* vbase = vc + (((size_t)vpage * nkv + kvh) * HD) * ps + (size_t)(vkey % ps);
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) rg.v[dt] = load8(vbase + (size_t)(dt * 16 + r) * ps);
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

  // BY_MATRIX: the way of the kernel for many tiles, whose waves are bound by the instructions they
  // issue (the sum of the probabilities from the matrix cores, nothing done for a reference that
  // stays); otherwise the way of the kernel for few tiles, which waits for memory and has no
  // registers to spare.
  template <bool BY_MATRIX>
  __device__ __forceinline__ void compute(int kb, const bf16x8_t (*qb)[KS], const BlockRegs& rg, TileState* sts) const {
    const int key0 = kb << 5;
    const bool interior = key0 >= all_lo && key0 + 31 <= all_hi;
    // the scores of all column tiles first: while the exponentials of one tile are taken, the
    // matrix cores still work on the scores of the next
    f32x4_t s[CT][2];
#pragma unroll
    for (int t = 0; t < CT; ++t)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        f32x4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rg.k[b][ks], qb[t][ks], a, 0, 0, 0);
        s[t][b] = a;
      }
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      TileState& st = sts[t];
      // mask and online softmax; this lane holds keys key0 + 8*lg + j of column r.  A block that
      // lies wholly inside what every column of the wave sees needs no mask.
      float raw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) raw[j] = (j < 4) ? s[t][0][j] : s[t][1][j - 4];
      if (!interior) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = key0 + 8 * lg + j;
          const bool ok = key >= my_lo[t] && key <= my_p[t] && key >= key_begin && key <= key_end;
          raw[j] = ok ? raw[j] : -INFINITY;
        }
      }
      // the largest of this lane's eight scores
      float mloc = max2(max2(max2(raw[0], raw[1]), max2(raw[2], raw[3])),
                        max2(max2(raw[4], raw[5]), max2(raw[6], raw[7]))) * scale_log2;   // scale_log2 > 0
      if constexpr (!BY_MATRIX) {
        mloc = max_over_groups(mloc);
        const bool move = mloc > st.m + LAZY_LOG2;   // always at a column's first visible key (m = -inf)
        const float m_new = move ? mloc : st.m;
        const float alpha = move ? __builtin_amdgcn_exp2f(st.m - m_new) : 1.f;
        // a column that has seen no key yet has m = -inf and only -inf scores: against 0 they give 0
        const float ref = m_new == -INFINITY ? 0.f : m_new;
        float psum = 0.f;
        float pv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          pv[j] = __builtin_amdgcn_exp2f(fmaf(raw[j], scale_log2, -ref));
          psum += pv[j];
        }
        st.l = st.l * alpha + psum;
        st.m = m_new;
        // the reference rarely moves after the first blocks: skip the rescaling when no column of
        // the wave needs it
        const bool rescale = __any(move);
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
      } else {
        // The column's four lanes hold the same m.  Only if one of them has a score far enough above
        // it does the reference move (always at a column's first visible key, where m = -inf; rarely
        // after a walk's first blocks), and only then do the lanes exchange their maxima and are
        // the sums brought to the new reference.
        if (__any(mloc > st.m + LAZY_LOG2)) {
          mloc = max_over_groups(mloc);
          const bool move = mloc > st.m + LAZY_LOG2;
          const float m_new = move ? mloc : st.m;
          const float alpha = move ? __builtin_amdgcn_exp2f(st.m - m_new) : 1.f;
          st.m = m_new;
#pragma unroll
          for (int dt = 0; dt <= NT; ++dt) {
            f32x4_t o = st.acc[dt];
            o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
            st.acc[dt] = o;
          }
        }
        // a column that has seen no key yet has m = -inf and only -inf scores: against 0 they give 0.
        // Inside the range that every column sees, every column has seen a key.
        float nref = -st.m;
        if (!interior) nref = st.m == -INFINITY ? 0.f : nref;
        float pv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) pv[j] = __builtin_amdgcn_exp2f(fmaf(raw[j], scale_log2, nref));
        u32x4_t packed = {pack2(pv[0], pv[1]), pack2(pv[2], pv[3]), pack2(pv[4], pv[5]), pack2(pv[6], pv[7])};
        const bf16x8_t pb = __builtin_bit_cast(bf16x8_t, packed);
#pragma unroll
        for (int dt = 0; dt < NT; ++dt)
          st.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rg.v[dt], pb, st.acc[dt], 0, 0, 0);
        // the sum of the probabilities comes from the matrix cores too: a row of ones beside the V^T
        // rows adds up, for every column, exactly the rounded probabilities that the products use
        st.acc[NT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones8(), pb, st.acc[NT], 0, 0, 0);
      }
    }
  }

  // The same arithmetic for a wave that carries more column tiles than its registers hold operands
  // for: the K rows and V^T rows of the stage (ks, vs) pass through a few registers, each fragment
  // multiplied with every tile before the next is read; scores of all tiles, then the probabilities
  // of all tiles, then the sums.  The way of the kernel for many tiles (see compute<true>).
  __device__ __forceinline__ void compute_streamed(int kb, const bf16x8_t (*qb)[KS], const bf16_t* ks, const bf16_t* vs,
                                                   TileState* sts) const {
    const int key0 = kb << 5;
    const bool interior = key0 >= all_lo && key0 + 31 <= all_hi;
    f32x4_t s[CT][2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const bf16_t* row = ks + (r >> 3) * (KH_LOADS * 512 + K_SKEW * 8) + (8 * ((r >> 2) & 1) + 4 * b + (r & 3)) * KROW;
#pragma unroll
      for (int t = 0; t < CT; ++t) s[t][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < KS; ++q) {
        const int d = q * 32 + 8 * lg;
        const bf16x8_t k = (d < HD) ? load8(row + d) : zero8();
#pragma unroll
        for (int t = 0; t < CT; ++t) s[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k, qb[t][q], s[t][b], 0, 0, 0);
      }
    }
    bf16x8_t pb[CT];
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      TileState& st = sts[t];
      float raw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) raw[j] = (j < 4) ? s[t][0][j] : s[t][1][j - 4];
      if (!interior) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = key0 + 8 * lg + j;
          const bool ok = key >= my_lo[t] && key <= my_p[t] && key >= key_begin && key <= key_end;
          raw[j] = ok ? raw[j] : -INFINITY;
        }
      }
      float mloc = max2(max2(max2(raw[0], raw[1]), max2(raw[2], raw[3])),
                        max2(max2(raw[4], raw[5]), max2(raw[6], raw[7]))) * scale_log2;
      if (__any(mloc > st.m + LAZY_LOG2)) {
        mloc = max_over_groups(mloc);
        const bool move = mloc > st.m + LAZY_LOG2;
        const float m_new = move ? mloc : st.m;
        const float alpha = move ? __builtin_amdgcn_exp2f(st.m - m_new) : 1.f;
        st.m = m_new;
#pragma unroll
        for (int dt = 0; dt <= NT; ++dt) {
          f32x4_t o = st.acc[dt];
          o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
          st.acc[dt] = o;
        }
      }
      float nref = -st.m;
      if (!interior) nref = st.m == -INFINITY ? 0.f : nref;
      float pv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) pv[j] = __builtin_amdgcn_exp2f(fmaf(raw[j], scale_log2, nref));
      u32x4_t packed = {pack2(pv[0], pv[1]), pack2(pv[2], pv[3]), pack2(pv[4], pv[5]), pack2(pv[6], pv[7])};
      pb[t] = __builtin_bit_cast(bf16x8_t, packed);
      st.acc[NT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones8(), pb[t], st.acc[NT], 0, 0, 0);
    }
    const int vslot = (lg >> 1) * V_HALF_SLOTS + 2 * r + ((lg & 1) ^ (r >> 3));
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) {
      const bf16x8_t v = load8(vs + (vslot + 32 * dt) * 8);
#pragma unroll
      for (int t = 0; t < CT; ++t) sts[t].acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pb[t], sts[t].acc[dt], 0, 0, 0);
    }
  }
};

// Walk the 32-key blocks first, first + stride, ... that overlap keys [key_begin, key_end]
// (inclusive, absolute) of one tile.  The loads of the next block and the page lookups of the one
// after are issued before the current block is computed, so a wave always has a block in flight.
// all but the N loads this wave asked for last have arrived (in LDS or in registers); nothing moves across
template <int N>
__device__ __forceinline__ void wait_for_all_but() {
  static_assert(N == 0 || N == 16, "the counts the walk uses");
  if (N == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
}
// every LDS read of this wave has its data: the place it read may be written again
__device__ __forceinline__ void lds_reads_done() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

template <int CT>
__device__ __forceinline__ void attend(const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
                                       const int* __restrict__ bt, int table_width, int nkv, int kvh, int ps,
                                       const bf16x8_t (*qb)[KS], const int* my_lo, const int* my_p, float scale_log2,
                                       int key_begin, int key_end, int kb_offset, int kb_stride, TileState* st,
                                       uint32_t k_stage = 0, const char* k_staged = nullptr, uint32_t k_stage2 = 0,
                                       const char* k_staged2 = nullptr) {
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
  if (K_VIA_LDS && k_staged) {
    // Keys through two places of 8 KB in LDS that belong to this wave (LDS byte addresses k_stage and
    // k_stage2); values straight into registers.  Two blocks are on their way at a time: while block kb
    // is computed, block kb + s is coming in, and block kb + 2 s is asked for as soon as block kb's place
    // and registers are free.  A block's 16 loads (8 for the values, then 8 for the keys) are the last
    // thing asked for before the wait for the block before it, so that wait allows exactly 16 loads to
    // be outstanding (loads finish in the order they were asked for); without a next block it allows none.
    static_assert(!K_VIA_LDS || NT == 8, "a block's value loads are counted");
    const uint32_t lane_off = w.lds_lane_offset();
    HalfPages h0, h1;
    w.issue_pages(kb, p0);
    w.issue_half_pages(kb, h0);
    if (LIVE(kb + s)) {
      w.issue_pages(kb + s, p1);
      w.issue_half_pages(kb + s, h1);
    }
    w.issue_v(kb, p0, ra);
    w.issue_k_to_lds(h0, k_stage, lane_off);
    if (LIVE(kb + s)) {
      w.issue_v(kb + s, p1, rb);
      w.issue_k_to_lds(h1, k_stage2, lane_off);
    }
    for (;; kb += 2 * s) {
      if (LIVE(kb + s)) wait_for_all_but<16>();
      else wait_for_all_but<0>();
      w.k_from_lds(k_staged, ra);
      if (LIVE(kb + 2 * s)) {
        w.issue_pages(kb + 2 * s, p0);
        w.issue_half_pages(kb + 2 * s, h0);
      }
      w.template compute<false>(kb, qb, ra, st);
      if (!LIVE(kb + s)) break;
      if (LIVE(kb + 2 * s)) {
        lds_reads_done();
        w.issue_v(kb + 2 * s, p0, ra);
        w.issue_k_to_lds(h0, k_stage, lane_off);
        wait_for_all_but<16>();
      } else {
        wait_for_all_but<0>();
      }
      w.k_from_lds(k_staged2, rb);
      if (LIVE(kb + 3 * s)) {
        w.issue_pages(kb + 3 * s, p1);
        w.issue_half_pages(kb + 3 * s, h1);
      }
      w.template compute<false>(kb + s, qb, rb, st);
      if (!LIVE(kb + 2 * s)) break;
      if (LIVE(kb + 3 * s)) {
        lds_reads_done();
        w.issue_v(kb + 3 * s, p1, rb);
        w.issue_k_to_lds(h1, k_stage2, lane_off);
      }
    }
    lds_reads_done();
    return;
  }
  w.issue_pages(kb, p0);
  if (LIVE(kb + s)) w.issue_pages(kb + s, p1);
  w.issue_loads(kb, p0, ra);
  for (;; kb += 2 * s) {
    if (LIVE(kb + 2 * s)) w.issue_pages(kb + 2 * s, p0);
    if (LIVE(kb + s)) w.issue_loads(kb + s, p1, rb);
    w.template compute<false>(kb, qb, ra, st);
    if (!LIVE(kb + s)) break;
    if (LIVE(kb + 3 * s)) w.issue_pages(kb + 3 * s, p1);
    if (LIVE(kb + 2 * s)) w.issue_loads(kb + 2 * s, p0, ra);
    w.template compute<false>(kb + s, qb, rb, st);
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

// A request's run of tokens in this step.  Without the array of run starts every request brings one
// token, request r the token r (a step of decoded tokens only): nothing is read then.
struct Run {
  int q0, qlen;
};
__device__ __forceinline__ Run run_of(const int* cu_q, int r) {
  if (!cu_q) return Run{r, 1};
  const int q0 = cu_q[r];
  return Run{q0, cu_q[r + 1] - q0};
}

__device__ __forceinline__ TileInfo tile_info(const int* cu_q, const int* ctx_len, int r, int ct, int g, int kvh,
                                              int window) {
  const int lane = threadIdx.x & 63, c = lane & 15;
  const Run run = run_of(cu_q, r);
  const int q0 = run.q0, qlen = run.qlen, ctx = ctx_len[r];
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

__device__ __forceinline__ void init_state(TileState& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int dt = 0; dt <= NT; ++dt) st.acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
}

// ---- many tiles, keys shared through LDS -------------------------------------------------------
// A block owns BLK_WAVES * BLK_CT consecutive column tiles of one request and one key/value head;
// wave w carries tiles (cb * BLK_WAVES + w) * BLK_CT .. + BLK_CT - 1.  The block walks the union
// of its waves' key ranges.  Every 32-key block is fetched from the pages once per block, by all
// waves together, and laid out in LDS the way the A operands want it, so the four waves share
// every byte that leaves L2:
//   K rows by key, each padded by 16 bytes, the two halves of the block's keys in regions of whole
//   1 KB loads, the second half's rows set off by K_SKEW slots: the 16 lanes of a row group (keys
//   4b .. 4b+3 and 4b+8 .. 4b+11 of either half, see the top of the file) then read 16 different
//   bank groups when the head size is a multiple of 128;
//   V^T as two arrays [channel][2 chunks of 8 keys], one for each half of the block's keys, the two
//   chunks of channels 8 .. 15 (mod 16) swapped: no padding, and again 16 different bank groups.
// The data goes from global memory straight into LDS (global_load_lds_dwordx4: lane l of a wave
// puts its 16 bytes at M0 + 16 l, so one instruction fills 1 KB of a stage and each lane works out
// once per walk which 16 bytes of a page belong there; lanes on padding fetch a neighbour's bytes
// again).  The two halves of a block's keys may lie in different pages, and a stage has four parts:
// the K rows and the V^T rows of either half.  Each of the four waves fills one part, so all that
// a wave does for a block's loads is one table lookup, one base address (scalar arithmetic) and a
// few load instructions with that base and the lanes' constant offsets.  (A wave issues an
// instruction every eight clocks or so and a SIMD holds two of these waves: every instruction of
// the loop counts, whatever unit runs it.)
// No register holds data in flight, so BLK_STAGES - 1 blocks are on their way while one is
// computed.  The loads are issued from inline assembly and waited for with explicit vmcnt values:
// every wave issues exactly WAVE_LOADS of them per block.
// With head sizes up to 128 the kernel also comes with GROUPS = 2 such groups of BLK_WAVES waves in
// a workgroup, on the same column tiles: group g walks the key blocks g, g + 2, ... through stages
// of its own, and the groups' sums are merged through LDS at the end.  One such workgroup fills a
// compute unit where two of the plain kind do, and a walk takes half as long.  That pays where a
// step has no more walks than the plain kind has places and they differ much in length (one
// prompt of 2,048 tokens: the first tiles see few keys, the last ones all); with more walks the
// plain kind's independent workgroups overlap their matrix and vector phases better.
#define BLK_WAVES 4
#if HD <= 128
#ifndef BLK_CT
#define BLK_CT 2
#endif
#if BLK_CT > 2
#define BLK_MAX_GROUPS 1
#else
#define BLK_MAX_GROUPS 2
#endif
#else
#define BLK_CT 1
#define BLK_MAX_GROUPS 1
#endif
#define BLK_STAGES 4
#if 2 * WAVE_LOADS > 63
#error "the in-flight loads of a wave do not fit the vmcnt counter"
#endif

// The LDS address is stage + offset: added straight into M0.
__device__ __forceinline__ void load16_to_lds(const char* base, uint32_t lane_bytes, uint32_t stage, uint32_t offset) {
  asm volatile("s_add_i32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_bytes), "s"(base), "s"(stage), "s"(offset) : "memory", "scc", "m0");
}
// Wait until at most n of this wave's loads are outstanding (they finish in order).
template <int N>
__device__ __forceinline__ void wait_loads() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}

// The page of the 16-key half of a block that a wave loads from, as the block table has it, and
// the slot in the page where the half begins (a page holds a multiple of 16 keys, so a half never
// straddles pages).  The same for every thread of the wave: scalar registers.
struct StagePages {
  int page, off;
};

// Wave w of a group fills part w of a stage: the K rows (w < 2) or V^T rows of half w % 2 of the
// block's keys, with WAVE_LOADS loads (a part with fewer issues its last again: same bytes to the
// same place, and every wave has the same number in flight).  Everything about a lane's address
// that does not change from block to block is worked out once (start); the half's page index and
// slot move along with the blocks (next_pages is called for the blocks kb, kb + GROUPS, ... of a
// group), so the page size is divided by once.
template <int GROUPS>
struct BlockLoader {
  const char* base;              // of the head's keys (or values) in page 0
  const int* bt;
  int table_width, ps, wave;
  uint32_t page_bytes;           // bytes of one page over all heads, K and V alike
  uint32_t slot_bytes;           // bytes from one slot of a page to the next: a key's HD values, or one value of a V^T row
  int idx, off;                  // page index and slot of the half in the next block
  int step_pages, step_slots;    // from one block of the group to its next: whole pages and slots
  uint32_t part_offset[WAVE_LOADS];   // of the load's 1 KB in a stage
  uint32_t fixed[WAVE_LOADS];    // byte offset of the lane's 16 bytes from where the half begins in its page

  __device__ __forceinline__ void start(const bf16_t* kc, const bf16_t* vc, int kb, int nkv, int kvh) {
    const int lane = threadIdx.x & 63;
    const bool keys = wave < 2;
    const int half = wave & 1;
    page_bytes = 2u * (uint32_t)nkv * (uint32_t)ps * (uint32_t)HD;
    slot_bytes = keys ? 2u * HD : 2u;
    base = keys ? reinterpret_cast<const char*>(kc + (size_t)kvh * ps * HD) : reinterpret_cast<const char*>(vc + (size_t)kvh * HD * ps);
    const int key = (kb << 5) + 16 * half;
    idx = key / ps;
    off = key - idx * ps;
    step_pages = 32 * GROUPS / ps;
    step_slots = 32 * GROUPS - step_pages * ps;
#pragma unroll
    for (int i = 0; i < WAVE_LOADS; ++i) {
      if (keys) {
        const int load = i < KH_LOADS ? i : KH_LOADS - 1;
        part_offset[i] = 1024u * (uint32_t)(half * KH_LOADS + load);
        int slot = 64 * load + lane - half * K_SKEW;   // of the half's rows
        slot = slot < 0 ? 0 : slot;
        int row = slot / (CH_PER_KEY + 1), part = slot - row * (CH_PER_KEY + 1);
        row = row < 16 ? row : 15;
        part = part < CH_PER_KEY ? part : CH_PER_KEY - 1;
        fixed[i] = 2u * (uint32_t)(row * HD + part * 8);
      } else {
        const int load = i < VH_LOADS ? i : VH_LOADS - 1;
        part_offset[i] = 1024u * (uint32_t)(K_LOADS + half * VH_LOADS + load);
        const int slot = 64 * load + lane;
        int row = slot >> 1;
        row = row < HD ? row : HD - 1;
        const int chunk = (slot & 1) ^ ((row >> 3) & 1);
        fixed[i] = 2u * (uint32_t)(row * ps + 8 * chunk);
      }
    }
#pragma unroll
    for (int i = 0; i < WAVE_LOADS; ++i) part_offset[i] = __builtin_amdgcn_readfirstlane(part_offset[i]);
  }
  // The half's page in the next block; keys past the table or without a page (nobody sees them) read
  // page 0.  The table entry is only asked for here: waiting for it is left to issue(), a block's work later.
  __device__ __forceinline__ void next_pages(StagePages& pg) {
    pg.page = idx < table_width ? bt[idx] : 0;   // as the table has it
    pg.off = off;
    idx += step_pages;
    off += step_slots;
    if (off >= ps) {
      off -= ps;
      ++idx;
    }
  }
  // Issue this wave's loads of the block with page pg into the stage at LDS byte address stage.
  __device__ __forceinline__ void issue(const StagePages& pg, uint32_t stage) const {
    const char* from = base + (uint64_t)(uint32_t)(pg.page < 0 ? 0 : pg.page) * page_bytes + (uint32_t)pg.off * slot_bytes;
#pragma unroll
    for (int i = 0; i < WAVE_LOADS; ++i) load16_to_lds(from, fixed[i], stage, part_offset[i]);
  }
};
static_assert(BLK_WAVES == 4, "a stage has four parts, one a wave");

__device__ __forceinline__ void operands_from_lds(const bf16_t* ks, const bf16_t* vs, BlockRegs& rg) {
  const int lane = threadIdx.x & 63, lg = lane >> 4, r = lane & 15;
  // row r of K block b holds key 8 (r / 4) + 4 b + r % 4 of the block's 32 (see the top of the file):
  // key 8 (r / 4 % 2) + 4 b + r % 4 of half r / 8
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const bf16_t* row = ks + (r >> 3) * (KH_LOADS * 512 + K_SKEW * 8) + (8 * ((r >> 2) & 1) + 4 * b + (r & 3)) * KROW;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int d = s * 32 + 8 * lg;
      rg.k[b][s] = (d < HD) ? load8(row + d) : zero8();
    }
  }
  // keys 8 lg .. 8 lg + 7 of channel dt * 16 + r: half lg / 2, chunk lg % 2, swapped for channels 8 .. 15
  const int vslot = (lg >> 1) * V_HALF_SLOTS + 2 * r + ((lg & 1) ^ (r >> 3));
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) rg.v[dt] = load8(vs + (vslot + 32 * dt) * 8);
}

// One entry of the block list for one key/value head.  blk_cb counts in units of
// BLK_WAVES * BLK_CT column tiles.
template <int GROUPS>
struct BlockShared {
  __attribute__((aligned(16))) bf16_t stage[GROUPS][BLK_STAGES][STAGE_ELEMS];   // K rows, then V^T rows
  int wave_range[GROUPS * BLK_WAVES][2];
  int work;
};
// what a lane of the second group hands over per column tile: its sums, the reference and its share of the total
#define MERGE_REGS (NT * 4 + 2)
static_assert(BLK_MAX_GROUPS == 1 || BLK_CT * MERGE_REGS * BLK_WAVES * 64 * 4 <= BLK_STAGES * STAGE_ELEMS * 2,
              "the second group's sums do not fit its stages");

template <int GROUPS>
__device__ __forceinline__ void attend_block(BlockShared<GROUPS>& sh, int item, int kvh, const bf16_t* __restrict__ q,
                                             const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
                                             const int* __restrict__ bt, int table_width,
                                             const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
                                             const int* __restrict__ blk_req, const int* __restrict__ blk_cb,
                                             bf16_t* __restrict__ out, int nq, int nkv, int ps, int window,
                                             float scale) {
  const int g = nq / nkv;
  const int wave_of_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int group = wave_of_all / BLK_WAVES, wave = wave_of_all % BLK_WAVES;
  const int r = blk_req[item], ct0 = (blk_cb[item] * BLK_WAVES + wave) * BLK_CT;
  const int ncols = (cu_q[r + 1] - cu_q[r]) * g;
  TileInfo t[BLK_CT];
  bf16x8_t qb[BLK_CT][KS];
  TileState st[BLK_CT];
  int lo = 0x7fffffff, hi = -1;
  Walk<BLK_CT> w;
#pragma unroll
  for (int i = 0; i < BLK_CT; ++i) {
    const bool exists = (ct0 + i) * 16 < ncols;   // a request's last block may be short of tiles
    t[i] = tile_info(cu_q, ctx_len, r, exists ? ct0 + i : 0, g, kvh, window);
    if (!exists) { t[i].valid = false; t[i].my_p = -1; }
    load_q(q, nq, t[i], qb[i]);
    init_state(st[i]);
    w.my_lo[i] = t[i].my_lo;
    w.my_p[i] = t[i].my_p;
    if (exists) {
      lo = t[i].lo_tile < lo ? t[i].lo_tile : lo;
      hi = t[i].hi_tile > hi ? t[i].hi_tile : hi;
    }
  }
  if (lane == 0) {
    sh.wave_range[wave_of_all][0] = lo;
    sh.wave_range[wave_of_all][1] = hi;
  }
  __syncthreads();
  int blo = 0x7fffffff, bhi = -1;
#pragma unroll
  for (int i = 0; i < GROUPS * BLK_WAVES; ++i) {
    blo = min(blo, sh.wave_range[i][0]);
    bhi = max(bhi, sh.wave_range[i][1]);
  }
  if (bhi < 0) return;  // uniform over the block
  blo = __builtin_amdgcn_readfirstlane(blo);
  bhi = __builtin_amdgcn_readfirstlane(bhi);
  w.key_begin = lo; w.key_end = hi;
  w.scale_log2 = scale * LOG2E; w.lg = lane >> 4; w.r = lane & 15;
  {  // the range every column of this wave sees
    int a = lo, b = hi;
#pragma unroll
    for (int i = 0; i < BLK_CT; ++i)
      if (w.my_p[i] >= 0) {
        a = max(a, w.my_lo[i]);
        b = min(b, w.my_p[i]);
      }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      a = max(a, __shfl_xor(a, o, QVL_WAVE));
      b = min(b, __shfl_xor(b, o, QVL_WAVE));
    }
    w.all_lo = __builtin_amdgcn_readfirstlane(a);   // the same in every lane: compared in scalar registers
    w.all_hi = __builtin_amdgcn_readfirstlane(b);
  }
  BlockLoader<GROUPS> ld;
  ld.bt = bt + (size_t)r * table_width;
  ld.table_width = table_width; ld.ps = ps; ld.wave = wave;
  // this group's blocks are kb0, kb0 + GROUPS, ...: nblk of them; every group goes round the
  // loop (and through its barrier) as often as the first
  const int kb0 = (blo >> 5) + group, all_blocks = (bhi >> 5) - (blo >> 5) + 1;
  const int nblk = (all_blocks - group + GROUPS - 1) / GROUPS;
  const int rounds = (all_blocks + GROUPS - 1) / GROUPS;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&sh.stage[group][0][0];
  StagePages pg;
  ld.start(kc, vc, kb0, nkv, kvh);
  ld.next_pages(pg);
  // the queries are in their registers before the first asynchronous load is issued: from here to
  // the end of the walk the compiler finds nothing of its own to wait for in vmcnt
  wait_loads<0>();
  int issued = 0;   // blocks whose loads are issued; pg holds the pages of the next one
#pragma unroll
  for (int d = 0; d < BLK_STAGES - 1; ++d)
    if (issued < nblk) {
      ld.issue(pg, lds0 + (uint32_t)(issued % BLK_STAGES) * (STAGE_ELEMS * 2));
      ++issued;
      if (issued < nblk) ld.next_pages(pg);
    }
  // the rounds in which this wave's columns see keys of the block: i_first .. i_last (block kb0 + GROUPS i
  // holds keys 32 kb .. 32 kb + 31; a wave without tiles has lo > hi and takes part in none)
  const int lo_s = __builtin_amdgcn_readfirstlane(lo), hi_s = __builtin_amdgcn_readfirstlane(hi);
  const int i_first = lo_s > hi_s ? rounds : ((lo_s >> 5) - kb0 + GROUPS - 1 < 0 ? 0 : ((lo_s >> 5) - kb0 + GROUPS - 1) / GROUPS);
  const int i_last = lo_s > hi_s || (hi_s >> 5) < kb0 ? -1 : ((hi_s >> 5) - kb0) / GROUPS;
  // One round: wait for block i, issue the loads of the block BLK_STAGES - 1 ahead, compute block i.
  // In a steady round that block exists, so two blocks are in flight behind block i and nothing has
  // to be asked (the table entry looked up for the block after the walk's last is never used).
  auto round = [&](int i, auto steady_round) {
    constexpr bool steady = decltype(steady_round)::value;
    if constexpr (steady) {
      wait_loads<2 * WAVE_LOADS>();
    } else {
      // block i has landed when only the loads of the blocks issued after it are outstanding
      const int later = issued - 1 - i;
      if (later >= 2) wait_loads<2 * WAVE_LOADS>();
      else if (later == 1) wait_loads<WAVE_LOADS>();
      else wait_loads<0>();
    }
    __syncthreads();   // everybody's part of block i is there, and everybody has left block i - 1
    if (steady || issued < nblk) {
      ld.issue(pg, lds0 + (uint32_t)(issued % BLK_STAGES) * (STAGE_ELEMS * 2));   // into the stage of block i - 1
      ++issued;
      if (steady || issued < nblk) ld.next_pages(pg);
    }
    if (i >= i_first && i <= i_last) {
      const bf16_t* stage = sh.stage[group][i % BLK_STAGES];
      if constexpr (BLK_CT >= 3) {
        w.compute_streamed(kb0 + GROUPS * i, qb, stage, stage + K_LOADS * 512, st);
      } else {
        BlockRegs ops;
        operands_from_lds(stage, stage + K_LOADS * 512, ops);
        w.template compute<true>(kb0 + GROUPS * i, qb, ops, st);
      }
    }
  };
  int i = 0;
  for (; i < nblk - (BLK_STAGES - 1); ++i) round(i, std::true_type{});
  for (; i < rounds; ++i) round(i, std::false_type{});
  if (GROUPS > 1) {
    // The second group's sums reach the first through the second group's stages, which nobody reads
    // or fills any more: word (tile, register, wave, lane), so every lane finds its partner's.
    float* hand = reinterpret_cast<float*>(&sh.stage[GROUPS - 1][0][0]);
    __syncthreads();
    if (group > 0) {
#pragma unroll
      for (int i = 0; i < BLK_CT; ++i) {
        float* mine = hand + ((size_t)i * MERGE_REGS * BLK_WAVES + wave) * 64 + lane;
#pragma unroll
        for (int dt = 0; dt < NT; ++dt)
#pragma unroll
          for (int j = 0; j < 4; ++j) mine[(dt * 4 + j) * BLK_WAVES * 64] = st[i].acc[dt][j];
        mine[(NT * 4) * BLK_WAVES * 64] = st[i].m;
        mine[(NT * 4 + 1) * BLK_WAVES * 64] = st[i].acc[NT][0];
      }
    }
    __syncthreads();
    if (group > 0) return;
#pragma unroll
    for (int i = 0; i < BLK_CT; ++i) {
      const float* theirs = hand + ((size_t)i * MERGE_REGS * BLK_WAVES + wave) * 64 + lane;
      const float m_b = theirs[(NT * 4) * BLK_WAVES * 64], l_b = theirs[(NT * 4 + 1) * BLK_WAVES * 64];
      const float m = fmaxf(st[i].m, m_b);
      const float ref = m == -INFINITY ? 0.f : m;   // a column without keys: both sides are zero
      const float sa = __builtin_amdgcn_exp2f(st[i].m - ref), sb = __builtin_amdgcn_exp2f(m_b - ref);
      st[i].acc[NT][0] = st[i].acc[NT][0] * sa + l_b * sb;
#pragma unroll
      for (int dt = 0; dt < NT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          st[i].acc[dt][j] = st[i].acc[dt][j] * sa + theirs[(dt * 4 + j) * BLK_WAVES * 64] * sb;
    }
  }
  const int lg = lane >> 4;
#pragma unroll
  for (int i = 0; i < BLK_CT; ++i) {
    const float total = st[i].acc[NT][0];
    if (!t[i].valid) continue;
    const float inv = 1.0f / total;
    bf16_t* orow = out + ((size_t)t[i].token * nq + t[i].head) * HD;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) {
      const int d = dt * 16 + 4 * lg;
      uint2 wv;
      wv.x = pack2(st[i].acc[dt][0] * inv, st[i].acc[dt][1] * inv);
      wv.y = pack2(st[i].acc[dt][2] * inv, st[i].acc[dt][3] * inv);
      *reinterpret_cast<uint2*>(orow + d) = wv;
    }
  }
}

// The workgroups take (entry, head) pairs from queues in global memory until these are empty: the
// host lists the entries longest walk first, so the long walks start at once and the short ones
// fill in behind them, whatever mix of requests the step has.  Workgroups go to the 8 XCDs in
// turn; when the key/value heads divide 8 there is a queue per head and a workgroup serves the
// head of its XCD first (that XCD's L2 then holds one head's keys) and the others when its own
// queue is empty.  queue[i] is the next entry of queue i, queue[QUEUE_DONE] counts the workgroups
// that have found every queue empty; the last of them puts all counters back to zero for the
// next launch (launches that share the counters must not overlap).
#define QUEUE_DONE 8
#define QUEUE_INTS 16
#if HD <= 128
#define BLK_PER_CU 2   // of the plain kind (GROUPS = 1); the kind with two groups fills a compute unit alone
#else
#define BLK_PER_CU 1
#endif
template <int GROUPS>
__global__ __launch_bounds__(64 * BLK_WAVES * GROUPS, GROUPS == 1 ? BLK_PER_CU : 1) void attn_mfma_block_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int* __restrict__ bt, int table_width, const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    const int* __restrict__ blk_req, const int* __restrict__ blk_cb, int num_blocks, bf16_t* __restrict__ out, int nq,
    int nkv, int ps, int window, float scale, int* __restrict__ queue) {
  __shared__ BlockShared<GROUPS> sh;
  const bool per_head = 8 % nkv == 0;
  const int queues = per_head ? nkv : 1;
  const int per_queue = per_head ? num_blocks : num_blocks * nkv;
  const int home = (blockIdx.x & 7) % queues;
  for (int turn = 0; turn < queues; ++turn) {
    const int qi = (home + turn) % queues;
    for (;;) {
      if (threadIdx.x == 0) sh.work = atomicAdd(&queue[qi], 1);
      __syncthreads();
      const int work = __builtin_amdgcn_readfirstlane(sh.work);   // the same for all: keep it scalar
      if (work >= per_queue) break;  // uniform over the block; every workgroup gets here for every queue
      attend_block(sh, per_head ? work : work / nkv, per_head ? qi : work % nkv, q, kc, vc, bt, table_width, cu_q,
                   ctx_len, blk_req, blk_cb, out, nq, nkv, ps, window, scale);
      __syncthreads();               // everybody has read sh.work and is done with the stages
    }
    __syncthreads();
  }
  if (threadIdx.x == 0 && atomicAdd(&queue[QUEUE_DONE], 1) == (int)gridDim.x - 1) {
    for (int i = 0; i < queues; ++i) atomicExch(&queue[i], 0);  // nobody takes work any more
    atomicExch(&queue[QUEUE_DONE], 0);
  }
}

// ---- few tiles (decode): the waves of a block share one tile ---------------------------------
// The COOP_WAVES waves of a block take the tile's 32-key blocks in turn (wave w the blocks
// w, w + COOP_WAVES, ...), then merge their sums and statistics through LDS in wave order.  With
// nsplit > 1 the key range is further cut among blocks (grid.z); each block then writes its
// merged partial to scratch.  The splits are merged by the block that finishes last (one counter
// per (tile, kv head) tells a block whether it is that one), or, for callers without counters, by
// a second kernel.
// Blocks of one tile may run on different XCDs, whose L2 caches do not see each other's lines: the
// partial results are stored and loaded at device scope (they go through to memory), every thread
// waits for its stores before the block's barrier, and only then is the counter raised, by a
// relaxed device-scope atomic.  No fence is used (a device-scope fence writes a whole L2 back).
// The last block leaves the counter at zero for the next launch.
// scratch layout per (tile, kv head, split): 16 columns x PART_COLS floats (HD sums, m, l, and
// padding that keeps every column 16-byte aligned).
#define PART_COLS (HD + 4)
#define PART_STRIDE (16 * PART_COLS)
#if HD <= 128
#define COOP_WAVES 8
#else
#define COOP_WAVES 2
#endif

// Device-scope ("agent") stores and loads: visible across the XCDs' L2 caches.
__device__ __forceinline__ void store_device_scope(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_device_scope(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge the nsplit partial results of one (tile, kv head) and write the tile's rows of the output:
// thread -> (column, 4 channels); splits are summed in order.  ACROSS: the partial results were
// written by other blocks of the running kernel (device-scope loads); otherwise by a kernel before.
template <bool ACROSS>
__device__ __forceinline__ void merge_splits(const float* __restrict__ base, int nsplit, int r, int ct, int kvh, int g,
                                             const int* __restrict__ cu_q, bf16_t* __restrict__ out, int nq) {
  const Run run = run_of(cu_q, r);
  const int q0 = run.q0, qlen = run.qlen;
  for (int idx = threadIdx.x; idx < 16 * (HD / 4); idx += blockDim.x) {
    const int col = idx / (HD / 4), d = (idx - col * (HD / 4)) * 4;
    const int colg = ct * 16 + col;
    const int i = colg / g, gh = colg - i * g;
    if (i >= qlen) continue;
    auto ld = [&](const float* p) { return ACROSS ? load_device_scope(p) : *p; };
    // Eight splits at a time: their 48 values are asked for together (one trip to memory, not one
    // per split), then folded into the running sums against the running maximum, in split order.
    constexpr int AT_ONCE = 8;
    float m = -INFINITY, den = 0.f;
    float4 num = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < nsplit; s0 += AT_ONCE) {
      float pm[AT_ONCE], pl[AT_ONCE];
      float4 pn[AT_ONCE];
#pragma unroll
      for (int j = 0; j < AT_ONCE; ++j) {
        const int s = s0 + j < nsplit ? s0 + j : nsplit - 1;   // beyond the last: read it again, weight 0 below
        const float* p = base + (size_t)s * PART_STRIDE + col * PART_COLS;
        pm[j] = ld(p + HD);
        pl[j] = ld(p + HD + 1);
        pn[j] = float4{ld(p + d), ld(p + d + 1), ld(p + d + 2), ld(p + d + 3)};
      }
      float m_new = m;
#pragma unroll
      for (int j = 0; j < AT_ONCE; ++j)
        if (s0 + j < nsplit) m_new = fmaxf(m_new, pm[j]);
      const float keep = (m == -INFINITY) ? 0.f : exp2f(m - m_new);
      num.x *= keep; num.y *= keep; num.z *= keep; num.w *= keep;
      den *= keep;
      m = m_new;
#pragma unroll
      for (int j = 0; j < AT_ONCE; ++j) {
        const float wgt = (s0 + j < nsplit && pm[j] != -INFINITY) ? exp2f(pm[j] - m) : 0.f;
        num.x += wgt * pn[j].x; num.y += wgt * pn[j].y; num.z += wgt * pn[j].z; num.w += wgt * pn[j].w;
        den += wgt * pl[j];
      }
    }
    const float inv = 1.0f / den;
    uint2 wv;
    wv.x = pack2(num.x * inv, num.y * inv);
    wv.y = pack2(num.z * inv, num.w * inv);
    *reinterpret_cast<uint2*>(out + ((size_t)(q0 + i) * nq + kvh * g + gh) * HD + d) = wv;
  }
}

__global__ __launch_bounds__(64 * COOP_WAVES) void attn_mfma_coop_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int* __restrict__ bt, int table_width, const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    const int* __restrict__ tile_req, const int* __restrict__ tile_ct, bf16_t* __restrict__ out,
    float* __restrict__ scratch, int* __restrict__ counters, int nq, int nkv, int ps, int window, float scale,
    int nsplit, int keys_per_split) {
  __shared__ __attribute__((aligned(16))) float sm[COOP_WAVES][PART_STRIDE];
  __shared__ __attribute__((aligned(16))) char second_place[K_VIA_LDS ? COOP_WAVES : 1][K_VIA_LDS ? 32 * HD * 2 : 16];   // of staged keys
  __shared__ int is_last;
  const int tile = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lg = lane >> 4, c = lane & 15;
  const int g = nq / nkv;
  // without a tile list tile i is the only tile of request i
  const int r = tile_req ? tile_req[tile] : tile, ct = tile_req ? tile_ct[tile] : 0;
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
    // a wave's place in LDS holds its staged keys while it walks, its sums afterwards
    static_assert(!K_VIA_LDS || PART_STRIDE * 4 >= 32 * HD * 2, "a wave's place in LDS holds a block's keys");
    const uint32_t k_stage = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&sm[wave][0]);
    const uint32_t k_stage2 = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&second_place[K_VIA_LDS ? wave : 0][0]);
    attend<1>(kc, vc, bt + (size_t)r * table_width, table_width, nkv, kvh, ps, qb, &t.my_lo, &t.my_p, scale * LOG2E,
              first, last, wave, COOP_WAVES, &st, k_stage, K_VIA_LDS ? reinterpret_cast<const char*>(&sm[wave][0]) : nullptr,
              k_stage2, &second_place[K_VIA_LDS ? wave : 0][0]);
  }
  // every wave leaves its column sums in LDS: column c, channels dt*16 + 4*lg .. +3, then m and l
  float* mine = &sm[wave][c * PART_COLS];
#pragma unroll
  for (int dt = 0; dt < NT; ++dt)
    *reinterpret_cast<float4*>(mine + dt * 16 + 4 * lg) =
        float4{st.acc[dt][0], st.acc[dt][1], st.acc[dt][2], st.acc[dt][3]};
  const float total = sum_over_groups(st.l);
  if (lg == 0) {
    mine[HD] = st.m;
    mine[HD + 1] = total;
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
    const Run run = run_of(cu_q, r);
    const int q0 = run.q0, qlen = run.qlen;
    if (nsplit > 1) {
      float* part = scratch + (((size_t)tile * nkv + kvh) * nsplit + split) * PART_STRIDE + (size_t)col * PART_COLS;
      if (counters) {   // read by another block of this launch
        store_device_scope(part + d, num.x); store_device_scope(part + d + 1, num.y);
        store_device_scope(part + d + 2, num.z); store_device_scope(part + d + 3, num.w);
        if (d == 0) {
          store_device_scope(part + HD, m);
          store_device_scope(part + HD + 1, den);
        }
      } else {
        *reinterpret_cast<float4*>(part + d) = num;
        if (d == 0) {
          part[HD] = m;
          part[HD + 1] = den;
        }
      }
    } else if (i < qlen) {
      const float inv = 1.0f / den;
      uint2 wv;
      wv.x = pack2(num.x * inv, num.y * inv);
      wv.y = pack2(num.z * inv, num.w * inv);
      *reinterpret_cast<uint2*>(out + ((size_t)(q0 + i) * nq + kvh * g + gh) * HD + d) = wv;
    }
  }
  if (nsplit > 1 && counters) {
    // every thread's stores have arrived before anyone counts this block in
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      int* count = counters + tile * nkv + kvh;
      const int before = __hip_atomic_fetch_add(count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before == nsplit - 1;
      if (is_last) __hip_atomic_store(count, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (is_last)
      merge_splits<true>(scratch + ((size_t)tile * nkv + kvh) * nsplit * PART_STRIDE, nsplit, r, ct, kvh, g, cu_q, out, nq);
  }
}

__global__ void attn_mfma_merge_kernel(const float* __restrict__ scratch, const int* __restrict__ cu_q,
                                       const int* __restrict__ tile_req, const int* __restrict__ tile_ct,
                                       bf16_t* __restrict__ out, int nq, int nkv, int nsplit) {
  // one block per (tile, kv head)
  const int tile = blockIdx.x, kvh = blockIdx.y;
  merge_splits<false>(scratch + ((size_t)tile * nkv + kvh) * nsplit * PART_STRIDE, nsplit, tile_req ? tile_req[tile] : tile,
                      tile_req ? tile_ct[tile] : 0, kvh, nq / nkv, cu_q, out, nq);
}

static int check_common(int num_tiles, int nq, int nkv, int ps, int table_width) {
  if (num_tiles <= 0) return QVL_OK;
  if (nq <= 0 || nkv <= 0 || nq % nkv || ps <= 0 || ps % 16 || table_width <= 0) return QVL_ERR_SHAPE;
  if (nkv > 65535) return QVL_ERR_LIMIT;
  return -1;
}

// Column tiles per entry of the block list that qvl_attn_mfma_block expects, and how many of its
// workgroups a compute unit holds at a time.
extern "C" int qvl_attn_mfma_block_tiles() { return BLK_WAVES * BLK_CT; }
extern "C" int qvl_attn_mfma_block_per_cu() { return BLK_PER_CU; }
extern "C" int qvl_attn_mfma_block_max_groups() { return BLK_MAX_GROUPS; }
extern "C" int qvl_attn_mfma_queue_ints() { return QUEUE_INTS; }

extern "C" int qvl_attn_mfma_block(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                                   const void* cu_q, const void* ctx_len, const void* blk_req, const void* blk_cb,
                                   int num_blocks, void* out, int nq, int nkv, int ps, int window, float scale,
                                   void* queue, int max_workgroups, int groups, hipStream_t stream) {
  // queue: qvl_attn_mfma_queue_ints() ints, zero before the first launch that uses them.
  // groups: wave groups per workgroup, 1 .. qvl_attn_mfma_block_max_groups(); max_workgroups should
  // be what the device holds at a time (qvl_attn_mfma_block_per_cu() per compute unit with one group, one with two).
  const int c = check_common(num_blocks, nq, nkv, ps, table_width);
  if (c >= 0) return c;
  if (!(scale > 0.f) || !queue || max_workgroups <= 0) return QVL_ERR_SHAPE;
  if (groups < 1 || groups > BLK_MAX_GROUPS) return QVL_ERR_LIMIT;
  const long long total = (long long)num_blocks * nkv;
  if (total > 0x7fffffffLL) return QVL_ERR_LIMIT;
  const unsigned grid = (unsigned)(total < max_workgroups ? total : max_workgroups);
#define QVL_BLOCK_LAUNCH(G)                                                                                          \
  hipLaunchKernelGGL(attn_mfma_block_kernel<G>, dim3(grid), dim3(64 * BLK_WAVES * G), 0, stream, (const bf16_t*)q,    \
                     (const bf16_t*)kc, (const bf16_t*)vc, (const int*)bt, table_width, (const int*)cu_q,              \
                     (const int*)ctx_len, (const int*)blk_req, (const int*)blk_cb, num_blocks, (bf16_t*)out, nq, nkv, \
                     ps, window, scale, (int*)queue)
  if (groups == 1) QVL_BLOCK_LAUNCH(1);
#if BLK_MAX_GROUPS > 1
  else QVL_BLOCK_LAUNCH(2);
#endif
#undef QVL_BLOCK_LAUNCH
  return qvl_launch_status();
}

// Floats the scratch buffer of a split call must hold.
extern "C" long long qvl_attn_mfma_scratch_floats(int num_tiles, int nkv, int nsplit) {
  return (long long)num_tiles * nkv * nsplit * PART_STRIDE;
}

static int launch_coop(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                       const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                       int num_tiles, void* out, void* scratch, void* counters, int nq, int nkv, int ps, int window,
                       float scale, int nsplit, int keys_per_split, hipStream_t stream) {
  const int c = check_common(num_tiles, nq, nkv, ps, table_width);
  if (c >= 0) return c;
  if (nsplit <= 0 || nsplit > 65535 || (nsplit > 1 && (keys_per_split <= 0 || keys_per_split % 32 || !scratch)))
    return QVL_ERR_SHAPE;
  if (!(scale > 0.f)) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(attn_mfma_coop_kernel, dim3(num_tiles, nkv, nsplit), dim3(64 * COOP_WAVES), 0, stream,
                     (const bf16_t*)q, (const bf16_t*)kc, (const bf16_t*)vc, (const int*)bt, table_width,
                     (const int*)cu_q, (const int*)ctx_len, (const int*)tile_req, (const int*)tile_ct, (bf16_t*)out,
                     (float*)scratch, nsplit > 1 ? (int*)counters : nullptr, nq, nkv, ps, window, scale, nsplit,
                     keys_per_split);
  if (hipGetLastError() != hipSuccess) return QVL_ERR_LAUNCH;
  if (nsplit > 1 && !counters)
    hipLaunchKernelGGL(attn_mfma_merge_kernel, dim3(num_tiles, nkv), dim3(256), 0, stream, (const float*)scratch,
                       (const int*)cu_q, (const int*)tile_req, (const int*)tile_ct, (bf16_t*)out, nq, nkv, nsplit);
  return qvl_launch_status();
}

extern "C" int qvl_attn_mfma_coop(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                                  const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                                  int num_tiles, void* out, void* scratch, int nq, int nkv, int ps, int window,
                                  float scale, int nsplit, int keys_per_split, hipStream_t stream) {
  return launch_coop(q, kc, vc, bt, table_width, cu_q, ctx_len, tile_req, tile_ct, num_tiles, out, scratch, nullptr, nq,
                     nkv, ps, window, scale, nsplit, keys_per_split, stream);
}

// The same with the splits merged inside the one kernel, by the block of each (tile, kv head) that
// finishes last.  counters: num_tiles * nkv ints, zero before the launch; the launch leaves them at
// zero.  Launches that share counters or scratch must not overlap.
extern "C" int qvl_attn_mfma_coop_merged(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                                         const void* cu_q, const void* ctx_len, const void* tile_req,
                                         const void* tile_ct, int num_tiles, void* out, void* scratch, void* counters,
                                         int nq, int nkv, int ps, int window, float scale, int nsplit,
                                         int keys_per_split, hipStream_t stream) {
  if (nsplit > 1 && !counters) return QVL_ERR_SHAPE;
  return launch_coop(q, kc, vc, bt, table_width, cu_q, ctx_len, tile_req, tile_ct, num_tiles, out, scratch, counters, nq,
                     nkv, ps, window, scale, nsplit, keys_per_split, stream);
}

// ---------------------------------------------------------------------------------------------
// The same attention with the partial results of a split call in memory the library owns: the
// call allocates nothing (see attention_mfma.h).  The array below exists once per GPU the library
// runs on, for the life of the process.  In host code its name is only a handle: the device
// address is asked for once per device and kept, and only that address is ever handed to a kernel.
static __device__ __align__(256) float scratch[QVL_ATTN_STATIC_SCRATCH_FLOATS];

#define QVL_MAX_DEVICES 64
static std::atomic<float*> scratch_of_device[QVL_MAX_DEVICES];
static std::mutex scratch_lock;

// The current device's copy of the array, or nullptr (then *err says why).  After a device's first
// call this is one atomic load: the lock is taken only while an address is still unknown.
static float* static_scratch(int* err) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= QVL_MAX_DEVICES) {
    *err = QVL_ERR_LIMIT;
    return nullptr;
  }
  float* ptr = scratch_of_device[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  std::lock_guard<std::mutex> hold(scratch_lock);
  ptr = scratch_of_device[dev].load(std::memory_order_relaxed);
  if (!ptr) {
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
      (void)hipGetLastError();
      *err = QVL_ERR_LAUNCH;
      return nullptr;
    }
    scratch_of_device[dev].store(ptr, std::memory_order_release);
  }
  return ptr;
}

extern "C" long long qvl_attn_mfma_static_scratch_floats() { return QVL_ATTN_STATIC_SCRATCH_FLOATS; }

extern "C" int qvl_attn_mfma_coop_static_init() {
  int err = QVL_OK;
  return static_scratch(&err) ? QVL_OK : err;
}

extern "C" int qvl_attn_mfma_coop_static(const void* q, const void* kc, const void* vc, const void* bt,
                                         int table_width, const void* cu_q, const void* ctx_len,
                                         const void* tile_req, const void* tile_ct, int num_tiles, void* out, int nq,
                                         int nkv, int ps, int window, float scale, int nsplit, int keys_per_split,
                                         hipStream_t stream) {
  if (num_tiles < 0 || nkv <= 0 || nsplit <= 0) return QVL_ERR_SHAPE;
  if (nsplit > 1 && qvl_attn_mfma_scratch_floats(num_tiles, nkv, nsplit) > QVL_ATTN_STATIC_SCRATCH_FLOATS)
    return QVL_ERR_LIMIT;   // more partial results than the array holds: use qvl_attn_mfma_coop
  int err = QVL_OK;
  float* ptr = static_scratch(&err);
  if (!ptr) return err;
  // Every (tile, head, split) block writes all of its part before the merge kernel reads it, so
  // nothing of the array has to start at zero, whatever the call before left there.
  return launch_coop(q, kc, vc, bt, table_width, cu_q, ctx_len, tile_req, tile_ct, num_tiles, out, ptr, nullptr, nq, nkv,
                     ps, window, scale, nsplit, keys_per_split, stream);
}
