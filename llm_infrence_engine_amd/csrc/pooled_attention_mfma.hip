// Attention over a window of tokens and pooled blocks before it, on the matrix cores: the paged kernel of
// attention_mfma.hip (a wave owns NT*16 columns = (token, query head of a group) pairs of one (request, key/value head),
// S^T = K Q^T, float online softmax in log2 units, O^T += V^T P^T from transposed value pages, the waves of a block take
// a tile's key blocks in turn and merge through LDS) in a mode of its own, kept in a file of its own so that the other
// models' kernel stays as it is, instruction for instruction.
//
// Beside the window's tokens a column sees one pooled key and value for every whole block of `pool` tokens that lies
// before its window: entries 0 .. (pos - window + 1) / pool - 1 of a second set of pages (pk_pages, pvt_pages, through
// pool_table: entry b at index b).  The pooled entries are walked first, as blocks of 32 like any others and by the same
// waves in turn; only where a block's keys come from and which of them a column sees differ.  turn_back (may be null):
// float2 [tokens, D / 2], the cosine and sine of an angle per token and pair of neighbouring entries; the result's
// entries 2m, 2m + 1 are turned by minus that angle before they are stored.
#include "common.h"
#include "api.h"
#include <algorithm>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr float REF_SLACK = 8.0f;   // log2 units by which a column's maximum may run ahead of its reference

template <int D>
struct KeyBlock {          // one block of 32 keys as this lane sees it
  bf16x8 k[2][D / 32];     // [16-key subtile][32-dim step]
};
template <int CT>
struct ValueBlock {        // and its values, for the CT tiles of 16 dims that this block works out
  bf16x4 v[CT][2];         // [16-dim tile][subtile]: 4 keys of one dim; the two subtiles are one MFMA operand
};

// Page arithmetic: pages of a power of two (page_shift >= 0) need no division.
struct PageGeom {
  int size, shift;
  __device__ __forceinline__ int index(int key) const { return shift >= 0 ? key >> shift : key / size; }
  __device__ __forceinline__ int offset(int key) const { return shift >= 0 ? key & (size - 1) : key % size; }
};

// The pages of the two 16-key halves of the block at `base` (the same for every lane, so they are kept in
// scalar registers and so is all address arithmetic that follows from them); past the context: the null page.
__device__ __forceinline__ void pages_of(const int* __restrict__ table, int base, int key_hi, PageGeom pg,
                                         int* pages) {
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int kb = base + u * 16;
    pages[u] = kb <= key_hi ? __builtin_amdgcn_readfirstlane(table[pg.index(kb)]) : 0;
  }
}

// Where the two 16-key halves of a block start inside their page's part of one kv head: uniform values.
struct BlockPlace {
  size_t head[2];   // element offset of (page, kv head) in either pool
  int off[2];       // first key inside the page
};

__device__ __forceinline__ BlockPlace place_of(const int* pages, int base, int g, int nkv, PageGeom pg, int D) {
  BlockPlace bp;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    bp.head[u] = ((size_t)pages[u] * nkv + g) * pg.size * D;
    bp.off[u] = pg.offset(base + u * 16);
  }
  return bp;
}

template <int D>
__device__ __forceinline__ void load_keys(KeyBlock<D>& b, const bf16* __restrict__ k_pages, const BlockPlace& bp,
                                          int lane) {
  const int k_lane = (lane & 15) * D + (lane >> 4) * 8;   // this lane's key and dims inside a 16-key half
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const bf16* kp = k_pages + bp.head[u] + bp.off[u] * D;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) b.k[u][s] = *reinterpret_cast<const bf16x8*>(kp + k_lane + s * 32);
  }
}

template <int CT>
__device__ __forceinline__ void load_values(ValueBlock<CT>& b, const bf16* __restrict__ vt_pages,
                                            const BlockPlace& bp, PageGeom pg, int dim0, int lane) {
  const int v_lane = (dim0 + (lane & 15)) * pg.size + (lane >> 4) * 4;   // this lane's dim and keys inside a tile
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const bf16* vp = vt_pages + bp.head[u] + bp.off[u];
#pragma unroll
    for (int c = 0; c < CT; ++c) b.v[c][u] = *reinterpret_cast<const bf16x4*>((vp + c * 16 * pg.size) + v_lane);
  }
}

// Two waves of a wide tile on every SIMD (256 registers each) hide each other's waits; narrow tiles fit anyway.
//
// VS > 1 (narrow tiles only) shares one tile among VS blocks: each works out all scores and the whole softmax
// but only D / VS of the output's dims, so it reads all keys and 1 / VS of the values.  A compute unit draws
// its data at a small fraction of the chip's rate, so when a step has fewer tiles than the chip has units this
// shortens the longest chain without a second kernel; the blocks write disjoint dims and share nothing.
struct PoolArgs {
  const bf16* pk_pages;
  const bf16* pvt_pages;
  const int* pool_table;
  const float2* turn_back;
  int pool;
};

template <int D, int NT, int WAVES, bool SPLIT, int VS, bool SINK, bool POOL = false>
__global__ void __launch_bounds__(WAVES * MS_WAVE, (NT > 1 && !(POOL && D == 128) ? 2 : 1))
pooled_attention_mfma_kernel(const bf16* __restrict__ q, size_t q_stride, const bf16* __restrict__ k_pages,
                      const bf16* __restrict__ vt_pages, const int* __restrict__ block_table, int table_stride,
                      const int* __restrict__ table_rows, const int* __restrict__ q_start,
                      const int* __restrict__ context_lens, bf16* __restrict__ out, size_t out_stride,
                      float* __restrict__ part_o, float* __restrict__ part_ml, int nh, int nkv, int page_size,
                      int page_shift, float scale_log2e, int window, int min_blocks, int n_splits,
                      const float* __restrict__ sink, PoolArgs pa = PoolArgs{}) {
  static_assert(!POOL || (!SPLIT && !SINK), "pooled blocks come with the general shape and without a sink");
  // SPLIT: min_blocks and n_splits say how a request's key blocks are spread.  Else min_blocks != 0 asks for
  // the order of tiles in which a long tile's companion on its CU is a short one (see below), and n_splits is
  // the number of requests whose tiles the grid's second dimension runs over (0: one tile to a request)
  __shared__ float sm_m[WAVES][NT][16], sm_l[WAVES][NT][16];
  static_assert(VS == 1 || (NT == 1 && !SPLIT), "only narrow tiles of the general shape share their dims out");
  static_assert((D / 16) % VS == 0, "whole tiles of 16 dims to a block");
  constexpr int CT = D / 16 / VS;
  __shared__ f32x4 sm_o[WAVES > 1 ? WAVES - 1 : 1][CT][NT][MS_WAVE];
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);   // the same for the whole wave
  const int col16 = lane & 15, kq = lane >> 4;
  // general shape: grid (kv heads, column tiles of the whole step, blocks that share a tile's dims): blocks are
  // handed out with the kv head running fastest; split shape: grid (splits, kv heads, requests)
  const int g = SPLIT ? blockIdx.y : blockIdx.x;
  const int bx = SPLIT ? blockIdx.x : blockIdx.z;
  const int rep = nh / nkv;
  const PageGeom pg = {page_size, page_shift};
  // Which request, and which of its tiles.  A request owns ceil(columns / tile width) tiles, requests in order,
  // so the launch needs to know only how many tokens and requests a step has, not how the tokens are dealt out
  // (a captured graph serves every mix).  The waves of a block find their place alike: a lane per request
  // works out its tiles, a prefix sum over the wave and a vote say where this block's tile falls.
  int r, rank, n_tiles;
  if (SPLIT) {
    r = blockIdx.z; rank = 0; n_tiles = 1;
  } else if (n_splits == 0) {
    r = blockIdx.y; rank = 0; n_tiles = 1;
  } else if (n_splits == 1) {
    r = 0; rank = blockIdx.y;
    n_tiles = ((q_start[1] - q_start[0]) * rep + 16 * NT - 1) / (16 * NT);
    if (rank >= n_tiles) return;
  } else {
    const int flat = blockIdx.y;
    int before = 0;
    r = -1; rank = 0; n_tiles = 0;
    for (int base = 0; base < n_splits; base += MS_WAVE) {
      const int i = base + lane;
      int mine = 0;
      if (i < n_splits) mine = ((q_start[i + 1] - q_start[i]) * rep + 16 * NT - 1) / (16 * NT);
      int upto = mine;   // tiles of the requests base..i
#pragma unroll
      for (int o = 1; o < MS_WAVE; o <<= 1) {
        const int v = __shfl_up(upto, o, MS_WAVE);
        if (lane >= o) upto += v;
      }
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(flat < before + upto);
      if (hit) {
        const int first = __builtin_ctzll(hit);
        r = base + first;
        n_tiles = __shfl(mine, first, MS_WAVE);
        rank = flat - before - (__shfl(upto, first, MS_WAVE) - n_tiles);
        break;
      }
      before += __shfl(upto, MS_WAVE - 1, MS_WAVE);
    }
    if (r < 0) return;   // the grid has room for a partial tile of every request; this block is surplus
    r = __builtin_amdgcn_readfirstlane(r);
    rank = __builtin_amdgcn_readfirstlane(rank);
    n_tiles = __builtin_amdgcn_readfirstlane(n_tiles);
  }
  const int row = table_rows ? table_rows[r] : r;
  const int* table = block_table + (size_t)row * table_stride;
  const int* ptable = POOL ? pa.pool_table + (size_t)row * table_stride : nullptr;
  // Without a window a wave's first key block is known before the request's lengths are: ask for its page
  // ids at once, so that they travel together with the lengths instead of after them.
  int first_pages[2] = {0, 0};
  const bool early = !SPLIT && window <= 0;
  if (early) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
      first_pages[u] = __builtin_amdgcn_readfirstlane(table[min(pg.index(wave * 32 + u * 16), table_stride - 1)]);
  }
  const int q0 = q_start[r];
  const int qlen = q_start[r + 1] - q0;
  const int start_pos = context_lens[r] - qlen;
  const int ncols = qlen * rep;
  // Late tiles of a prompt see the most keys: they go first, so that the long ones do not finish last.  When
  // all blocks fit on the chip at once (two to a CU), only the later half goes first, latest tile first, and
  // then the earlier half, earliest first: blocks that start one round of the chip apart tend to share a CU, and
  // so a long tile's companion is a short one that soon leaves the SIMDs to it (2,048 tokens: 34.0 -> 29.4 us).
  const int dim0 = VS > 1 ? bx * CT * 16 : 0;   // the first of this block's output dims
  const int half = (!SPLIT && min_blocks) ? (n_tiles + 1) / 2 : n_tiles;
  const int tile = rank < half ? n_tiles - 1 - rank : rank - half;
  const int c0 = SPLIT ? 0 : tile * 16 * NT;
  if (c0 >= ncols) return;

  // key range of the tile: from the first column's window start to the last column's own position
  const int last_col = min(ncols, c0 + 16 * NT) - 1;
  int key_hi = start_pos + last_col / rep;
  int key_lo = 0;
  if (window > 0) key_lo = max(0, start_pos + c0 / rep - window + 1);
  int blk_begin = key_lo / 32, blk_end = key_hi / 32 + 1;
  // a block whose keys every column of the tile sees needs no mask: all keys at or before the first column's
  // position (and, with a window, after the last column's window start); tiles with idle columns always mask
  const int first_pos = start_pos + c0 / rep;
  const bool full_tile = c0 + 16 * NT <= ncols;
  if (SPLIT) {
    // every request spreads its own key blocks evenly over the splits (at least min_blocks each)
    const int per = max(min_blocks, (blk_end - blk_begin + n_splits - 1) / n_splits);
    blk_begin += bx * per;
    blk_end = min(blk_end, blk_begin + per);
    if (blk_begin >= blk_end) return;
  }

  // POOL: the pooled entries that the tile's last column sees come first, as the blocks vfirst .. blk_begin - 1
  const auto seen_blocks = [&](int p) { return POOL && p - window + 1 >= pa.pool ? (p - window + 1) / pa.pool : 0; };
  const int pool_hi = seen_blocks(key_hi) - 1;                 // the last pooled entry any column of the tile sees
  const int vfirst = blk_begin - (pool_hi + 32) / 32;          // (pool_hi = -1: no such block)
  const int pool_all = seen_blocks(first_pos);                 // entries below this one are seen by every column
  // where the keys of block blk come from: (first entry, last entry that may be read, pooled or not)
  const auto is_pooled = [&](int blk) { return POOL && blk < blk_begin; };
  const auto base_of = [&](int blk) { return is_pooled(blk) ? (blk - vfirst) * 32 : blk * 32; };

  // this lane's columns
  int pos[NT];   // -1: an idle column (sees no key; its result is not written)
  bf16x8 qv[NT][D / 32];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int c = c0 + t * 16 + col16;
    const int cc = min(c, ncols - 1);
    const int tok = q0 + cc / rep, head = g * rep + cc % rep;
    pos[t] = c < ncols ? start_pos + cc / rep : -1;
    const bf16* qp = q + (size_t)tok * q_stride + (size_t)head * D + kq * 8;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) qv[t][s] = *reinterpret_cast<const bf16x8*>(qp + s * 32);
  }

  int seen[POOL ? NT : 1];    // POOL: how many pooled entries each of this lane's columns sees
  if (POOL) {
#pragma unroll
    for (int t = 0; t < NT; ++t) seen[t] = seen_blocks(pos[t]);
  }

  // The sums of the exponentials come from the matrix cores too: one more product per column tile, of P^T with
  // a V^T of ones, gives every lane its columns' sums over all 32 keys of the block (of the same bfloat16 values
  // that the weighted sum of the values uses), where adding them up lane by lane took 32 additions and, at the
  // end, two exchanges between lanes; the matrix pipe has the time.
  // (The widest tile at head size 64 has no registers left for it and adds its exponentials up on the vector
  // pipe, a lane's share at a time, with two exchanges between lanes at the end.)
  constexpr bool SUMS_BY_MATRIX = !(D == 64 && NT == 4);
  float m[NT], lvec[NT];
  f32x4 o[CT][NT], lsum[SUMS_BY_MATRIX ? NT : 1];
  bf16x8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    m[t] = -INFINITY;
    lvec[t] = 0.f;
    if (SUMS_BY_MATRIX) lsum[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < CT; ++c) o[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // A sink is one more term of the denominator with no key and no value: the running softmax of one wave (the first
  // wave of the block, of the first split) starts as if it had already seen a key with that score, unscaled, and a
  // value of zero.  Everything after (moving the reference, merging waves and splits) treats it as any other term.
  if (SINK && wave == 0 && (!SPLIT || bx == 0)) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int cc = min(c0 + t * 16 + col16, ncols - 1);
      m[t] = sink[g * rep + cc % rep] * 1.4426950408889634f;
      lvec[t] = kq == 0 ? 1.0f : 0.f;
      if (SUMS_BY_MATRIX) lsum[t] = f32x4{1.f, 1.f, 1.f, 1.f};
    }
  }

  // A narrow tile (decode) has registers to spare and few waves to hide a wait behind: it fetches the next
  // block's values early, together with its keys.  A wide tile fetches values at the top of the pass that
  // uses them (the score products and the softmax run meanwhile, and so does the SIMD's other wave).
  constexpr bool VALUES_EARLY = NT == 1;
  KeyBlock<D> buf_k[2];
  ValueBlock<CT> buf_v[2];
  BlockPlace buf_at[2];
  if (vfirst + wave < blk_end) {
    KeyBlock<D>& cur_k = buf_k[0];
    ValueBlock<CT>& cur_v = buf_v[0];
    BlockPlace& cur_at = buf_at[0];
    const bool pooled = is_pooled(vfirst + wave);
    const int base = base_of(vfirst + wave);
    int pages[2];
    if (early) {  // blk_begin is 0 here; halves past the last key fall back to the null page
#pragma unroll
      for (int u = 0; u < 2; ++u) pages[u] = base + u * 16 <= key_hi ? first_pages[u] : 0;
    } else {
      pages_of(pooled ? ptable : table, base, pooled ? pool_hi : key_hi, pg, pages);
    }
    cur_at = place_of(pages, base, g, nkv, pg, D);
    load_keys<D>(cur_k, pooled ? pa.pk_pages : k_pages, cur_at, lane);
    if (VALUES_EARLY) load_values<CT>(cur_v, pooled ? pa.pvt_pages : vt_pages, cur_at, pg, dim0, lane);
  }
  // The page ids of a block are asked for one block before its keys are: the keys' loads then go out at the top of
  // an iteration instead of behind a table lookup (8,192 tokens of the 0.5B shape: 235 -> 232 us; 2,048 tokens at
  // head size 128: 99.9 -> 96.7 us).  (Keeping the loads of two blocks in flight for narrow tiles was measured and
  // dropped: a decode tile's time is what its CU can draw, 102 KB at about 43 GB/s at 640 keys, not its waits.)
  int ahead_pages[2] = {0, 0};
  if (vfirst + wave + WAVES < blk_end) {
    const bool pooled = is_pooled(vfirst + wave + WAVES);
    pages_of(pooled ? ptable : table, base_of(vfirst + wave + WAVES), pooled ? pool_hi : key_hi, pg, ahead_pages);
  }
  // One block of 32 keys: the step works on the buffers it is handed as current and fills those it is handed
  // as next; the loop below calls it with the two sets of buffers in turn, so nothing is copied between them.
  auto step = [&](int blk, KeyBlock<D>& cur_k, ValueBlock<CT>& cur_v, BlockPlace& cur_at, KeyBlock<D>& nxt_k,
                  ValueBlock<CT>& nxt_v, BlockPlace& nxt_at) __attribute__((always_inline)) {
    const bool pooled = is_pooled(blk);
    const int base = base_of(blk);
    const int hi = pooled ? pool_hi : key_hi;      // the last entry of this block's source that may be read
    if (!VALUES_EARLY) load_values<CT>(cur_v, pooled ? pa.pvt_pages : vt_pages, cur_at, pg, dim0, lane);
    if (blk + WAVES < blk_end) {
      const bool npooled = is_pooled(blk + WAVES);
      nxt_at = place_of(ahead_pages, base_of(blk + WAVES), g, nkv, pg, D);
      load_keys<D>(nxt_k, npooled ? pa.pk_pages : k_pages, nxt_at, lane);
      if (VALUES_EARLY) load_values<CT>(nxt_v, npooled ? pa.pvt_pages : vt_pages, nxt_at, pg, dim0, lane);
      if (blk + 2 * WAVES < blk_end) {
        const bool apooled = is_pooled(blk + 2 * WAVES);
        pages_of(apooled ? ptable : table, base_of(blk + 2 * WAVES), apooled ? pool_hi : key_hi, pg, ahead_pages);
      }
    }

    // scores: s[u][t] holds keys base + u*16 + kq*4 + (0..3) of column t*16 + col16
    f32x4 s[2][NT];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur_k.k[u][ks], qv[t][ks], acc, 0, 0, 0);
        s[u][t] = acc;
      }

    // values past the last visible key may be anything a reused page still holds: make them zero
    if (base + 31 > hi) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (base + u * 16 + kq * 4 + i > hi) {
#pragma unroll
            for (int c = 0; c < CT; ++c) cur_v.v[c][u][i] = (__bf16)0.0f;
          }
    }

    const bool unmasked = pooled ? full_tile && base + 31 < pool_all
                                 : full_tile && base + 31 <= first_pos && (window <= 0 || base > key_hi - window);
    bf16x8 p[NT];
    float corr[NT], bmax[NT];
    bool moved = false;
    // the block's maxima of the raw scores (the scale is positive, so they are the maxima of the scaled ones
    // too); one branch for the whole tile, so that what follows is straight-line code for all its columns
    if (unmasked) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float bm = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) bm = fmaxf(bm, s[u][t][i]);
        bmax[t] = bm;
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float bm = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = base + u * 16 + kq * 4 + i;
            const bool see = pooled ? key < seen[t]
                                    : key <= pos[t] && (window <= 0 || key > pos[t] - window);
            const float v = see ? s[u][t][i] : -INFINITY;
            s[u][t][i] = v;
            bm = fmaxf(bm, v);
          }
        bmax[t] = bm;
      }
    }
    float m_safe[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float bm = bmax[t];
      bm = fmaxf(bm, __shfl_xor(bm, 16, MS_WAVE));
      bm = fmaxf(bm, __shfl_xor(bm, 32, MS_WAVE));
      bm *= scale_log2e;
      // m is the reference that the exponents are taken against, not necessarily the maximum: it follows the
      // maximum only when that has run ahead by more than REF_SLACK (a factor 2^REF_SLACK in the terms, far
      // inside float's range), so that the accumulators are rescaled rarely.  Any reference gives the same
      // softmax; all lanes of a column decide alike because bm is the same in all of them.
      const bool step = bm > m[t] + REF_SLACK;
      const float m_new = step ? bm : m[t];
      corr[t] = step ? fast_exp2(m[t] - m_new) : 1.0f;   // m = -inf: 0
      moved |= step;
      m[t] = m_new;
      m_safe[t] = m_new == -INFINITY ? 0.f : m_new;
    }
    if (NT == 1 || __builtin_amdgcn_ballot_w64(moved) != 0) {   // the same branch for the whole wave
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (SUMS_BY_MATRIX) lsum[t] *= corr[t]; else lvec[t] *= corr[t];
#pragma unroll
        for (int c = 0; c < CT; ++c) o[c][t] *= corr[t];
      }
    }
    // column by column, so that the products of one column run on the matrix cores while the next column's
    // exponentials are taken
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = fast_exp2(fmaf(s[u][t][i], scale_log2e, -m_safe[t]));
          if (!SUMS_BY_MATRIX) lvec[t] += e;
          p[t][u * 4 + i] = (__bf16)e;
        }
      if (SUMS_BY_MATRIX) lsum[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p[t], lsum[t], 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        bf16x8 vv;
#pragma unroll
        for (int i = 0; i < 4; ++i) { vv[i] = cur_v.v[c][0][i]; vv[4 + i] = cur_v.v[c][1][i]; }
        o[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, p[t], o[c][t], 0, 0, 0);
      }
    }
  };
  for (int blk = vfirst + wave; blk < blk_end; blk += 2 * WAVES) {
    step(blk, buf_k[0], buf_v[0], buf_at[0], buf_k[1], buf_v[1], buf_at[1]);
    if (blk + WAVES < blk_end) step(blk + WAVES, buf_k[1], buf_v[1], buf_at[1], buf_k[0], buf_v[0], buf_at[0]);
  }

  float l[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (SUMS_BY_MATRIX) {
      l[t] = lsum[t][0];   // every row of the product of ones is the column's sum
    } else {               // a column's sum is spread over the four lane groups
      l[t] = lvec[t] + __shfl_xor(lvec[t], 16, MS_WAVE);
      l[t] += __shfl_xor(l[t], 32, MS_WAVE);
    }
  }
  if (WAVES > 1) {
    // merge the waves' partial results (each relative to its own maximum) in wave order
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (kq == 0) { sm_m[wave][t][col16] = m[t]; sm_l[wave][t][col16] = l[t]; }
      if (wave > 0) {
#pragma unroll
        for (int c = 0; c < CT; ++c) sm_o[wave - 1][c][t][lane] = o[c][t];
      }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float big = m[t];
      for (int w = 1; w < WAVES; ++w) big = fmaxf(big, sm_m[w][t][col16]);
      const float safe = big == -INFINITY ? 0.f : big;
      const float f0 = fast_exp2(m[t] - safe);
      float lsum = l[t] * f0;
#pragma unroll
      for (int c = 0; c < CT; ++c) o[c][t] *= f0;
      for (int w = 1; w < WAVES; ++w) {
        const float f = fast_exp2(sm_m[w][t][col16] - safe);
        lsum += f * sm_l[w][t][col16];
#pragma unroll
        for (int c = 0; c < CT; ++c) o[c][t] += sm_o[w - 1][c][t][lane] * f;
      }
      m[t] = big;
      l[t] = lsum;
    }
  }

#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const float lt = l[t];
    if (pos[t] < 0) continue;
    const int c = c0 + t * 16 + col16;   // worked out again rather than kept through the loop
    const int tok = q0 + c / rep, head = g * rep + c % rep;
    if (SPLIT) {
      // unnormalised: O, the running maximum (log2 units) and the sum; the combine kernel weighs the splits
      const size_t slot = ((size_t)r * nh + head) * n_splits + bx;
      float* po = part_o + slot * D + kq * 4;
#pragma unroll
      for (int c = 0; c < CT; ++c) *reinterpret_cast<f32x4*>(po + c * 16) = o[c][t];
      if (kq == 0) { part_ml[slot * 2] = m[t]; part_ml[slot * 2 + 1] = lt; }
    } else {
      const float inv = 1.0f / lt;
      bf16* op = out + (size_t)tok * out_stride + (size_t)head * D + dim0 + kq * 4;
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        bf16x4 w;
        if (POOL && pa.turn_back) {     // a lane's four dims are two pairs of neighbours
#pragma unroll
          for (int i = 0; i < 4; i += 2) {
            const float2 cs = pa.turn_back[(size_t)tok * (D / 2) + ((dim0 + c * 16 + kq * 4 + i) >> 1)];
            const float a = o[c][t][i] * inv, b = o[c][t][i + 1] * inv;
            w[i] = (__bf16)(a * cs.x + b * cs.y);
            w[i + 1] = (__bf16)(b * cs.x - a * cs.y);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) w[i] = (__bf16)(o[c][t][i] * inv);
        }
        *reinterpret_cast<bf16x4*>(op + c * 16) = w;
      }
    }
  }
}

inline int page_shift_of(int page_size) {   // log2 of a power of two, else -1
  if (page_size & (page_size - 1)) return -1;
  int sh = 0;
  while ((1 << sh) < page_size) ++sh;
  return sh;
}

template <int D, int NT, int WAVES, int VS>
int launch_pooled(const bf16* q, size_t q_stride, const bf16* k, const bf16* vt, const int* table, int table_stride,
                  const int* table_rows, const int* q_start, const int* ctx, bf16* out, size_t out_stride,
                  int n_requests, int n_tokens, int max_q_len, int nh, int nkv, int page_size, float scale,
                  int window, PoolArgs pa, hipStream_t stream) {
  const int rep = nh / nkv;
  const long long per_request = ((long long)max_q_len * rep + 16 * NT - 1) / (16 * NT);
  long long tiles = (long long)n_tokens * rep / (16 * NT) + n_requests;
  if (tiles > per_request * n_requests) tiles = per_request * n_requests;
  if (tiles > 65535) return MS_UNSUPPORTED;   // grid.y
  const int scan = per_request == 1 ? 0 : n_requests;
  dim3 grid(nkv, (unsigned)tiles, VS), block(WAVES * MS_WAVE);
  pooled_attention_mfma_kernel<D, NT, WAVES, false, VS, false, true><<<grid, block, 0, stream>>>(q, q_stride, k, vt, table, table_stride, table_rows, q_start, ctx, out, out_stride, nullptr, nullptr, nh, nkv, page_size, page_shift_of(page_size), scale * 1.4426950408889634f, window, 0, scan, nullptr, pa);
  return ms_launch_status();
}

}  // namespace

// A window of `window` tokens and pooled blocks of `pool` tokens before it (see POOL above).  As ms_paged_attention_mfma,
// plus pk_pages [P2, nkv, page_size, d], pvt_pages [P2, nkv, d, page_size] (entry b of a request at index b of its row of
// pool_table, int32 [rows, table_stride]) and turn_back (may be null) float [n_tokens, d / 2, 2], (cos, sin) per token and pair.
extern "C" int ms_pooled_attention_mfma(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                                        const int* block_table, const void* pk_pages, const void* pvt_pages,
                                        const int* pool_table, int table_stride, const int* table_rows,
                                        const int* q_start, const int* context_lens, const float* turn_back, void* out,
                                        long long out_stride, int n_requests, int n_tokens, int max_q_len, int num_heads,
                                        int num_kv_heads, int head_dim, int page_size, float scale, int window, int pool,
                                        hipStream_t stream) {
  if (n_requests <= 0 || max_q_len <= 0 || n_tokens <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || table_stride <= 0 || window <= 0 || pool <= 0 ||
      pk_pages == nullptr || pvt_pages == nullptr || pool_table == nullptr)
    return MS_BAD_ARG;
  if (!(scale > 0.f)) return MS_BAD_ARG;
  if (!ms_attention_mfma_supported(head_dim, page_size)) return MS_UNSUPPORTED;
  if (q_stride % 8 || out_stride % 4 || ((uintptr_t)q % 16) || ((uintptr_t)out % 8)) return MS_UNSUPPORTED;
  if (n_requests > 65535 || num_kv_heads > 65535) return MS_UNSUPPORTED;
  if ((uintptr_t)turn_back % 8) return MS_BAD_ARG;
  const PoolArgs pa = {(const bf16*)pk_pages, (const bf16*)pvt_pages, pool_table, (const float2*)turn_back, pool};
#define GO(D, NT, WV) return launch_pooled<D, NT, WV, 1>((const bf16*)q, q_stride, (const bf16*)k_pages, (const bf16*)vt_pages, block_table, table_stride, table_rows, q_start, context_lens, (bf16*)out, out_stride, n_requests, n_tokens, max_q_len, num_heads, num_kv_heads, page_size, scale, window, pa, stream)
  const int cols = max_q_len * (num_heads / num_kv_heads);
  if (cols > 16) {
    if (head_dim == 32) GO(32, 2, 4);
    if (head_dim == 64) GO(64, 2, 4);
    GO(128, 2, 4);
  }
  if (head_dim == 32) GO(32, 1, 8);
  if (head_dim == 64) GO(64, 1, 8);
  GO(128, 1, 4);     // four waves: one to a SIMD, with registers for both kinds of blocks
#undef GO
}
