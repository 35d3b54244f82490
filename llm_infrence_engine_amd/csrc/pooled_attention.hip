// Attention over a sliding window of tokens plus one pooled key and value for every whole block of older tokens, with
// neighbouring entries of q, k and v turned by the position and the result turned back.
//
// A token at position i sees the tokens j with 0 <= i - j < size and, beside them, block b (the tokens b P .. b P + P - 1)
// once the whole block lies before the window: b P + P - 1 <= i - size.  A block's key is the mean of its P keys as the
// pages hold them, its value the mean of its P values; tokens and blocks share one softmax.  Tokens that have left the
// window and whose block is not whole yet are not seen.
//
// Pages: tokens in [page][kv head][slot][width] through the request's row of `table`; blocks, one entry each (entry b
// at index b), in pages of the same shape through the row of `pool_table`.  v_transposed: both kinds of value pages are
// [page][kv head][width][slot] instead (what the matrix-core kernel reads as an operand as it lies).
//
// ms_pairs_rotate_store   q, k in place over their first rot_dims entries (pair m = entries 2m, 2m + 1, angle
//                         pos * inv_freq[m]), v over all its dv entries (angle pos * inv_freq_v[m]); k and v go to the
//                         token pages at the token's slot.
// ms_pool_store           for every token that ends a block (pool slot >= 0): the means of the block's P keys and values,
//                         read back from the token pages, into the pooled pages.
// ms_pooled_attention     one wave per (token, query head): float scores, running maximum, sums; the output's pairs are
//                         turned by -pos * inv_freq_v[m] before they are stored.
#include "common.h"
#include "api.h"

namespace {

constexpr int PA_WAVES = 4;
constexpr int PA_MAX_D = 256;

template <typename T>
__global__ void __launch_bounds__(256)
pairs_rotate_store_kernel(T* __restrict__ qkv, size_t stride, const int* __restrict__ positions,
                          const float* __restrict__ inv_freq, const float* __restrict__ inv_freq_v,
                          const int* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages, int n_tokens,
                          int nh, int nkv, int d, int dv, int rot_dims, int page_size, int v_transposed) {
  const int pairs_q = nh * d / 2, pairs_k = nkv * d / 2, pairs_v = nkv * dv / 2;
  const int per_token = pairs_q + pairs_k + pairs_v;
  const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= (long long)n_tokens * per_token) return;
  const int n = (int)(item / per_token);
  int p = (int)(item - (long long)n * per_token);
  const int pos = positions[n];
  T* row = qkv + (size_t)n * stride;
  int head, m, width, rot;
  T* src;
  T* dst = nullptr;
  size_t dst_step = 1;      // from an entry to its neighbour in the destination
  const float* freq;
  const int slot = slots ? slots[n] : -1;
  if (p < pairs_q + pairs_k) {
    const bool is_k = p >= pairs_q;
    if (is_k) p -= pairs_q;
    head = p / (d / 2); m = p - head * (d / 2); width = d; rot = rot_dims; freq = inv_freq;
    src = row + (is_k ? (size_t)nh * d : 0) + (size_t)head * d + 2 * m;
    if (is_k) {
      if (slot >= 0) dst = k_pages + (((size_t)(slot / page_size) * nkv + head) * page_size + slot % page_size) * d + 2 * m;
    } else {
      dst = src;
    }
  } else {
    p -= pairs_q + pairs_k;
    head = p / (dv / 2); m = p - head * (dv / 2); width = dv; rot = dv; freq = inv_freq_v;
    src = row + (size_t)(nh + nkv) * d + (size_t)head * dv + 2 * m;
    if (slot >= 0) {
      const size_t at = ((size_t)(slot / page_size) * nkv + head) * page_size;
      if (v_transposed) { dst = v_pages + (at * dv + (size_t)2 * m * page_size) + slot % page_size; dst_step = page_size; }
      else dst = v_pages + (at + slot % page_size) * dv + 2 * m;
    }
  }
  (void)width;
  if (dst == nullptr) return;
  float a = to_float(src[0]), b = to_float(src[1]);
  if (2 * m < rot) {
    float sn, cs;
    sincosf((float)pos * freq[m], &sn, &cs);
    const float ra = a * cs - b * sn, rb = b * cs + a * sn;
    a = ra; b = rb;
  } else if (dst == src) {
    return;
  }
  dst[0] = from_float<T>(a);
  dst[dst_step] = from_float<T>(b);
}

// one wave per (token, kv head); only tokens that end a block work
template <typename T>
__global__ void __launch_bounds__(256)
pool_store_kernel(const T* __restrict__ k_pages, const T* __restrict__ v_pages, const int* __restrict__ table,
                  int table_stride, const int* __restrict__ table_rows, const int* __restrict__ token_req,
                  const int* __restrict__ positions, const int* __restrict__ pool_slots, T* __restrict__ pk_pages,
                  T* __restrict__ pv_pages, int n_tokens, int nkv, int d, int dv, int page_size, int pool, int v_transposed) {
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const long long item = (long long)blockIdx.x * (blockDim.x / MS_WAVE) + threadIdx.x / MS_WAVE;
  if (item >= (long long)n_tokens * nkv) return;
  const int n = (int)(item / nkv), h = (int)(item - (long long)n * nkv);
  const int slot = pool_slots[n];
  if (slot < 0) return;
  const int pos = positions[n];
  const int req = token_req[n];
  const int* tab = table + (size_t)(table_rows ? table_rows[req] : req) * table_stride;
  const float inv = 1.0f / (float)pool;
  const size_t phead = ((size_t)(slot / page_size) * nkv + h) * page_size;
  const int poff = slot % page_size;
  for (int i = lane; i < d + dv; i += MS_WAVE) {
    const bool key = i < d;
    const int e = key ? i : i - d, w = key ? d : dv;
    const T* pages = key ? k_pages : v_pages;
    const bool flip = !key && v_transposed;
    float s = 0.f;
    for (int j = pos - pool + 1; j <= pos; ++j) {
      const size_t head = ((size_t)tab[j / page_size] * nkv + h) * page_size;
      const int off = j % page_size;
      s += to_float(flip ? pages[head * w + (size_t)e * page_size + off] : pages[(head + off) * w + e]);
    }
    T* dst = key ? pk_pages : pv_pages;
    dst[flip ? phead * w + (size_t)e * page_size + poff : (phead + poff) * w + e] = from_float<T>(s * inv);
  }
}

// the keys first .. last (entries of `tab`'s pages) join the running softmax of the wave's (token, head)
template <typename T>
__device__ __forceinline__ void attend_span(const float* __restrict__ qs, const T* __restrict__ k_pages,
                                            const T* __restrict__ v_pages, const int* __restrict__ tab, int first, int last,
                                            int nkv, int kvh, int d, int dv, int page_size, int v_transposed, int lane,
                                            float& m, float& l, float (&acc)[PA_MAX_D / MS_WAVE]) {
  for (int base = first; base <= last; base += MS_WAVE) {
    const int j = base + lane;
    const bool valid = j <= last;
    size_t row = 0;
    float s = -INFINITY;
    if (valid) {
      row = ((size_t)tab[j / page_size] * nkv + kvh) * page_size + (j % page_size);
      const T* kp = k_pages + row * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(kp[i]), dot);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);      // 0 while m is still -inf
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < PA_MAX_D / MS_WAVE; ++c) acc[c] *= corr;
    const int count = min(MS_WAVE, last - base + 1);
    for (int jj = 0; jj < count; ++jj) {
      const float pj = __shfl(p, jj, MS_WAVE);
      const unsigned lo = __shfl((unsigned)(row & 0xffffffffu), jj, MS_WAVE), hi = __shfl((unsigned)(row >> 32), jj, MS_WAVE);
      const size_t vrow = ((size_t)hi << 32) | lo;
      const T* vp = v_transposed ? v_pages + (vrow / page_size) * page_size * dv + vrow % page_size : v_pages + vrow * dv;
      const size_t vs = v_transposed ? page_size : 1;
#pragma unroll
      for (int c = 0; c < PA_MAX_D / MS_WAVE; ++c) {
        const int i = lane + c * MS_WAVE;
        if (i < dv) acc[c] = fmaf(pj, to_float(vp[i * vs]), acc[c]);
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(PA_WAVES * MS_WAVE)
pooled_attention_kernel(const T* __restrict__ q, size_t q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                        const int* __restrict__ table, const T* __restrict__ pk_pages, const T* __restrict__ pv_pages,
                        const int* __restrict__ pool_table, int table_stride, const int* __restrict__ table_rows,
                        const int* __restrict__ n_live_tokens, const int* __restrict__ token_req,
                        const int* __restrict__ positions, const float* __restrict__ inv_freq_v, T* __restrict__ out,
                        size_t out_stride, int n_tokens, int nh, int nkv, int d, int dv, int page_size, float scale,
                        int size, int pool, int v_transposed) {
  __shared__ float qs[PA_WAVES][PA_MAX_D];
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const long long item = (long long)blockIdx.x * PA_WAVES + wave;
  if (item >= (long long)n_tokens * nh) return;      // whole waves leave; no block-wide barrier below
  const int n = (int)(item / nh), h = (int)(item - (long long)n * nh);
  if (n_live_tokens && n >= *n_live_tokens) return;
  const int kvh = h / (nh / nkv);
  const int pos = positions[n];
  const int req = token_req[n];
  const size_t trow = (size_t)(table_rows ? table_rows[req] : req) * table_stride;
  const T* qp = q + (size_t)n * q_stride + (size_t)h * d;
  for (int i = lane; i < d; i += MS_WAVE) qs[wave][i] = to_float(qp[i]) * scale;
  __builtin_amdgcn_wave_barrier();

  float m = -INFINITY, l = 0.f;
  float acc[PA_MAX_D / MS_WAVE];
#pragma unroll
  for (int c = 0; c < PA_MAX_D / MS_WAVE; ++c) acc[c] = 0.f;
  const int first = pos - size + 1 > 0 ? pos - size + 1 : 0;
  const int n_blocks = pool > 0 && pos - size + 1 > 0 ? (pos - size + 1) / pool : 0;
  if (n_blocks > 0)
    attend_span<T>(qs[wave], pk_pages, pv_pages, pool_table + trow, 0, n_blocks - 1, nkv, kvh, d, dv, page_size, v_transposed, lane, m, l, acc);
  attend_span<T>(qs[wave], k_pages, v_pages, table + trow, first, pos, nkv, kvh, d, dv, page_size, v_transposed, lane, m, l, acc);

  T* op = out + (size_t)n * out_stride + (size_t)h * dv;
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < PA_MAX_D / MS_WAVE; ++c) {
    const int i = lane + c * MS_WAVE;
    float mine = acc[c] * inv;
    if (inv_freq_v) {       // the pair (2m, 2m + 1) lies in neighbouring lanes; turned by -pos * f_m
      const float other = __shfl_xor(mine, 1, MS_WAVE);
      float sn = 0.f, cs = 1.f;
      if (i < dv) sincosf((float)pos * inv_freq_v[i >> 1], &sn, &cs);
      mine = (i & 1) ? mine * cs - other * sn : mine * cs + other * sn;
    }
    if (i < dv) op[i] = from_float<T>(mine);
  }
}

}  // namespace

extern "C" int ms_pairs_rotate_store(void* qkv, long long stride, const int* positions, const float* inv_freq,
                                     const float* inv_freq_v, const int* slots, void* k_pages, void* v_pages, int n_tokens,
                                     int num_heads, int num_kv_heads, int head_dim, int value_dim, int rot_dims,
                                     int page_size, int v_transposed, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || value_dim <= 0 || (head_dim & 1) || (value_dim & 1) ||
      rot_dims < 0 || (rot_dims & 1) || rot_dims > head_dim || page_size <= 0 ||
      stride < (long long)(num_heads + num_kv_heads) * head_dim + (long long)num_kv_heads * value_dim)
    return MS_BAD_ARG;
  const long long items = (long long)n_tokens * ((num_heads + num_kv_heads) * head_dim + num_kv_heads * value_dim) / 2;
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
#define LAUNCH(T) pairs_rotate_store_kernel<T><<<grid, block, 0, stream>>>((T*)qkv, (size_t)stride, positions, inv_freq, inv_freq_v, slots, (T*)k_pages, (T*)v_pages, n_tokens, num_heads, num_kv_heads, head_dim, value_dim, rot_dims, page_size, v_transposed)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

extern "C" int ms_pool_store(const void* k_pages, const void* v_pages, const int* table, int table_stride,
                             const int* table_rows, const int* token_req, const int* positions, const int* pool_slots,
                             void* pk_pages, void* pv_pages, int n_tokens, int num_kv_heads, int head_dim, int value_dim,
                             int page_size, int pool, int v_transposed, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (num_kv_heads <= 0 || head_dim <= 0 || value_dim <= 0 || page_size <= 0 || pool <= 0 || table_stride <= 0)
    return MS_BAD_ARG;
  const long long items = (long long)n_tokens * num_kv_heads;
  dim3 grid((unsigned)((items + 3) / 4)), block(256);
#define LAUNCH(T) pool_store_kernel<T><<<grid, block, 0, stream>>>((const T*)k_pages, (const T*)v_pages, table, table_stride, table_rows, token_req, positions, pool_slots, (T*)pk_pages, (T*)pv_pages, n_tokens, num_kv_heads, head_dim, value_dim, page_size, pool, v_transposed)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

extern "C" int ms_pooled_attention(const void* q, long long q_stride, const void* k_pages, const void* v_pages,
                                   const int* table, const void* pk_pages, const void* pv_pages, const int* pool_table,
                                   int table_stride, const int* table_rows, const int* n_live_tokens, const int* token_req,
                                   const int* positions, const float* inv_freq_v, void* out, long long out_stride,
                                   int n_tokens, int num_heads, int num_kv_heads, int head_dim, int value_dim,
                                   int page_size, float scale, int size, int pool, int v_transposed, int dtype,
                                   hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || page_size <= 0 || table_stride <= 0 ||
      size <= 0 || pool < 0 || (pool > 0 && (pk_pages == nullptr || pv_pages == nullptr || pool_table == nullptr)) ||
      (inv_freq_v != nullptr && (value_dim & 1)))
    return MS_BAD_ARG;
  if (head_dim <= 0 || head_dim > PA_MAX_D || value_dim <= 0 || value_dim > PA_MAX_D) return MS_UNSUPPORTED;
  const long long items = (long long)n_tokens * num_heads;
  dim3 grid((unsigned)((items + PA_WAVES - 1) / PA_WAVES)), block(PA_WAVES * MS_WAVE);
#define LAUNCH(T) pooled_attention_kernel<T><<<grid, block, 0, stream>>>((const T*)q, (size_t)q_stride, (const T*)k_pages, (const T*)v_pages, table, (const T*)pk_pages, (const T*)pv_pages, pool_table, table_stride, table_rows, n_live_tokens, token_req, positions, inv_freq_v, (T*)out, (size_t)out_stride, n_tokens, num_heads, num_kv_heads, head_dim, value_dim, page_size, scale, size, pool, v_transposed)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
