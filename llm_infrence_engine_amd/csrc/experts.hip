// Kernels of a feed-forward made of routed experts, all driven by device data so that a step can be captured:
//   route    per token: softmax over the router's outputs, the `top` largest of (score + correction), their scores
//   align    rows (token, choice) grouped by expert into tiles of TILE rows, each tile of one expert
//   grouped  out[row] = act(W[expert of the row's tile] . in[row]) for every tile, gathered / scattered by the rows' list
//   combine  out[n] = sum_j weight[n, j] * (expert j's row, or the token's input for an identity expert)
//                     (+ sigmoid(gate[n]) * shared[n])
// and the exact gelu, z/2 (1 + erf(z / sqrt 2)).  Router scores, weights and all sums are float.
#include "common.h"
#include "api.h"

namespace {

constexpr int ROUTE_MAX_PER_LANE = 16;     // router outputs a lane holds: up to 1024 outputs
constexpr int ROUTE_MAX_TOP = 32;

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f)); }

template <typename T>
__global__ void gelu_kernel(const T* __restrict__ x, T* __restrict__ out, size_t total) {
  constexpr int V = 16 / sizeof(T);     // values in 16 bytes
  struct alignas(16) Pack { T v[V]; };
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t packs = (((size_t)x | (size_t)out) & 15) == 0 ? total / V : 0;   // 16 bytes a lane where both are aligned
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < packs; i += stride) {
    Pack p = reinterpret_cast<const Pack*>(x)[i];
#pragma unroll
    for (int j = 0; j < V; ++j) p.v[j] = from_float<T>(gelu_erf(to_float(p.v[j])));
    reinterpret_cast<Pack*>(out)[i] = p;
  }
  for (size_t i = packs * V + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
    out[i] = from_float<T>(gelu_erf(to_float(x[i])));
}

// One wave per token.  Ties go to the lower index.  sigmoid_scores: every score is the sigmoid of its own logit
// instead of the softmax over all of them.
__global__ void __launch_bounds__(256)
moe_route_kernel(const float* __restrict__ logits, size_t ld, const float* __restrict__ correction, int n_tokens,
                 int n_out, int top, int* __restrict__ ids, float* __restrict__ weights, int sigmoid_scores) {
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int n = blockIdx.x * (blockDim.x / MS_WAVE) + threadIdx.x / MS_WAVE;
  if (n >= n_tokens) return;
  const float* z = logits + (size_t)n * ld;
  float s[ROUTE_MAX_PER_LANE], c[ROUTE_MAX_PER_LANE];
  float big = -INFINITY;
#pragma unroll
  for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
    const int e = lane + i * MS_WAVE;
    s[i] = e < n_out ? z[e] : -INFINITY;
    big = fmaxf(big, s[i]);
  }
  big = wave_max(big);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
    const int e = lane + i * MS_WAVE;
    s[i] = e < n_out ? (sigmoid_scores ? 1.0f / (1.0f + expf(-s[i])) : expf(s[i] - big)) : 0.f;
    sum += s[i];
  }
  sum = wave_sum(sum);
  const float inv = sigmoid_scores ? 1.0f : 1.0f / sum;
#pragma unroll
  for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
    const int e = lane + i * MS_WAVE;
    s[i] *= inv;
    c[i] = e < n_out ? s[i] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY, bs = 0.f;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i) {
      const int e = lane + i * MS_WAVE;
      if (c[i] > bv) { bv = c[i]; be = e; bs = s[i]; }   // a lane's indices rise with i: the first maximum stays
    }
#pragma unroll
    for (int o = MS_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, MS_WAVE), os = __shfl_xor(bs, o, MS_WAVE);
      const int oe = __shfl_xor(be, o, MS_WAVE);
      if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; bs = os; }
    }
    if (lane == 0) { ids[(size_t)n * top + j] = be; weights[(size_t)n * top + j] = bs; }
#pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; ++i)
      if (lane + i * MS_WAVE == be) c[i] = -INFINITY;
  }
}

// One block.  rows[cap] (cap = tiles * tile): for every tile its rows' flat index n * top + j, or -1; tile_expert[tiles]:
// the tile's expert, or -1 for a tile nobody uses.  Choices of experts >= n_experts (identities) take no row.
__global__ void __launch_bounds__(1024)
moe_align_kernel(const int* __restrict__ ids, int n_items, int n_experts, int tile, int tiles, int* __restrict__ rows,
                 int* __restrict__ tile_expert) {
  extern __shared__ int sh[];     // counts [n_experts], first row of each expert [n_experts + 1]
  int* count = sh;
  int* first = sh + n_experts;
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) count[e] = 0;
  for (int i = threadIdx.x; i < tiles * tile; i += blockDim.x) rows[i] = -1;
  for (int t = threadIdx.x; t < tiles; t += blockDim.x) tile_expert[t] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < n_items; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < n_experts; ++e) {
      first[e] = at;
      at += (count[e] + tile - 1) / tile * tile;
    }
    first[n_experts] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    for (int t = first[e] / tile; t < first[e + 1] / tile; ++t) tile_expert[t] = e;
    count[e] = 0;       // now the cursor within the expert's rows
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_items; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < n_experts) rows[first[e] + atomicAdd(&count[e], 1)] = i;
  }
}

// Vector-ALU product of every tile with its expert's matrix: float accumulation in the order of k, whatever the
// batch.  A block owns GM rows of a tile by GN output features; K walks in steps of GK through LDS.
constexpr int GM = 16, GN = 64, GK = 32;

template <typename T, typename TO>
__global__ void __launch_bounds__(256)
grouped_gemm_kernel(const T* __restrict__ in, size_t in_stride, const T* __restrict__ w, const int* __restrict__ rows,
                    const int* __restrict__ tile_expert, TO* __restrict__ out, size_t out_stride, int n_out, int K,
                    int in_div, int out_scatter, int act) {
  __shared__ float As[GM][GK + 1], Ws[GN][GK + 1];
  __shared__ int s_row[GM];
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int n0 = blockIdx.y * GN;
  const int tid = threadIdx.x;
  if (tid < GM) s_row[tid] = rows[tile * GM + tid];
  __syncthreads();
  const T* we = w + (size_t)e * n_out * K;
  const int r = tid / 16, cg = tid % 16;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += GK) {
    for (int i = tid; i < GM * GK; i += 256) {
      const int rr = i / GK, kk = i % GK;
      const int item = s_row[rr];
      float v = 0.f;
      if (item >= 0 && k0 + kk < K) {
        const size_t src = in_div > 0 ? (size_t)(item / in_div) : (size_t)(tile * GM + rr);
        v = to_float(in[src * in_stride + k0 + kk]);
      }
      As[rr][kk] = v;
    }
    for (int i = tid; i < GN * GK; i += 256) {
      const int cc = i / GK, kk = i % GK;
      Ws[cc][kk] = (n0 + cc < n_out && k0 + kk < K) ? to_float(we[(size_t)(n0 + cc) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      const float a = As[r][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = fmaf(a, Ws[cg + 16 * j][kk], acc[j]);
    }
    __syncthreads();
  }
  const int item = s_row[r];
  if (item < 0) return;
  const size_t dst = out_scatter ? (size_t)item : (size_t)(tile * GM + r);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = n0 + cg + 16 * j;
    if (c < n_out) out[dst * out_stride + c] = from_float<TO>(act ? gelu_erf(acc[j]) : acc[j]);
  }
}

// The same product on the matrix cores, bfloat16 in, K a multiple of 32.  A block owns one tile of 16 * NT rows and a slab
// of 128 output features, 32 to each of its four waves: the expert's rows are the A operand of
// v_mfma_f32_16x16x32_bf16 (a lane reads 16 bytes of a row), the tile's activations, gathered by the rows' list, the B
// operand; a lane then holds four neighbouring features of one row.  Every output sums over k in the same order whatever
// else is in the tile.  The grid runs over slabs first, so that neighbouring blocks read the same activations and
// different weights.
typedef __attribute__((ext_vector_type(8))) __bf16 gg_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 gg_bf16x4;
typedef __attribute__((ext_vector_type(4))) float gg_f32x4;
constexpr int GG_SLAB = 128;

template <int NT, typename TO>
__global__ void __launch_bounds__(256)
grouped_gemm_mfma_kernel(const bf16* __restrict__ in, size_t in_stride, const bf16* __restrict__ w,
                         const int* __restrict__ rows, const int* __restrict__ tile_expert, TO* __restrict__ out,
                         size_t out_stride, int n_out, int K, int in_div, int out_scatter, int act) {
  constexpr int TM = 16 * NT;
  const int tile = blockIdx.y;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int col = lane & 15, kq = lane >> 4;
  const int f0 = blockIdx.x * GG_SLAB + wave * 32;
  if (f0 >= n_out) return;
  const bf16* we = w + (size_t)e * n_out * K;
  const bf16* wrow[2];
  bool wlive[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int f = f0 + u * 16 + col;
    wlive[u] = f < n_out;
    wrow[u] = we + (size_t)(wlive[u] ? f : 0) * K + kq * 8;
  }
  const bf16* arow[NT];
  int item[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int p = tile * TM + t * 16 + col;
    item[t] = rows[p];
    const size_t src = in_div > 0 ? (size_t)(max(item[t], 0) / in_div) : (size_t)p;
    arow[t] = in + src * in_stride + kq * 8;
  }
  gg_f32x4 acc[2][NT];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[u][t] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
  const gg_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // a decode step is the stream of the chosen experts' matrices: four steps' loads in flight a wave
#pragma unroll 4
  for (int k = 0; k < K; k += 32) {
    gg_bf16x8 wv[2], av[NT];
#pragma unroll
    for (int u = 0; u < 2; ++u) wv[u] = wlive[u] ? *reinterpret_cast<const gg_bf16x8*>(wrow[u] + k) : zero;
#pragma unroll
    for (int t = 0; t < NT; ++t) av[t] = item[t] >= 0 ? *reinterpret_cast<const gg_bf16x8*>(arow[t] + k) : zero;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[u], av[t], acc[u][t], 0, 0, 0);
  }
  // lane holds out[row = t * 16 + col][feature f0 + u * 16 + kq * 4 + i], i = 0..3
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (item[t] < 0) continue;
    const size_t dst = out_scatter ? (size_t)item[t] : (size_t)(tile * TM + t * 16 + col);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int f = f0 + u * 16 + kq * 4;
      TO* op = out + dst * out_stride + f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = act ? gelu_erf(acc[u][t][i]) : acc[u][t][i];
        if (f + i < n_out) op[i] = from_float<TO>(v);
      }
    }
  }
}

// The product for tiles of 128 rows, for experts with many rows each (portions of prompts).  A block owns a tile and 256
// output features, 64 to each wave: 32 accumulator tiles a wave, so a row of the expert's matrix that a wave reads serves
// 128 rows of activations and the activations, which all waves need, are staged once a block through LDS (two buffers
// taken in turn, one barrier a step of 64 along K).  The next step's rows of the matrix and activations are asked for
// before the current step's products start.
constexpr int GW_NT = 8, GW_FT = 4, GW_TM = 16 * GW_NT, GW_SLAB = 64 * 4, GW_KS = 64, GW_PAD = 8;
constexpr int GW_PIECES = GW_TM * (GW_KS / 8) / 256;     // pieces of 16 bytes a thread stages a step

template <typename TO>
__global__ void __launch_bounds__(256, 2)
grouped_gemm_mfma_wide_kernel(const bf16* __restrict__ in, size_t in_stride, const bf16* __restrict__ w,
                              const int* __restrict__ rows, const int* __restrict__ tile_expert, TO* __restrict__ out,
                              size_t out_stride, int n_out, int K, int in_div, int out_scatter, int act) {
  __shared__ __align__(16) bf16 Bs[2][GW_TM][GW_KS + GW_PAD];
  __shared__ int s_item[GW_TM];
  const int tile = blockIdx.y;
  const int e = tile_expert[tile];
  if (e < 0 || (int)blockIdx.x * GW_SLAB >= n_out) return;   // an unused tile, or a slab that only pads the grid
  const int tid = threadIdx.x, lane = tid & (MS_WAVE - 1), wave = tid / MS_WAVE;
  const int col = lane & 15, kq = lane >> 4;
  if (tid < GW_TM) s_item[tid] = rows[tile * GW_TM + tid];
  __syncthreads();
  // staging: a row of a step is 128 bytes, eight pieces of 16; a thread brings four pieces
  const bf16* src[GW_PIECES];
  bool src_live[GW_PIECES];
  int st_row[GW_PIECES], st_part[GW_PIECES];
#pragma unroll
  for (int j = 0; j < GW_PIECES; ++j) {
    const int c = tid + j * 256;
    st_row[j] = c / (GW_KS / 8);
    st_part[j] = c % (GW_KS / 8);
    const int item = s_item[st_row[j]];
    src_live[j] = item >= 0;
    const size_t r = in_div > 0 ? (size_t)(max(item, 0) / in_div) : (size_t)(tile * GW_TM + st_row[j]);
    src[j] = in + r * in_stride + st_part[j] * 8;
  }
  const int f0 = blockIdx.x * GW_SLAB + wave * 64;
  const bf16* we = w + (size_t)e * n_out * K;
  const bf16* wrow[GW_FT];
  bool wlive[GW_FT];
#pragma unroll
  for (int u = 0; u < GW_FT; ++u) {
    const int f = f0 + u * 16 + col;
    wlive[u] = f < n_out;
    wrow[u] = we + (size_t)(wlive[u] ? f : 0) * K + kq * 8;
  }
  gg_f32x4 acc[GW_FT][GW_NT];
#pragma unroll
  for (int u = 0; u < GW_FT; ++u)
#pragma unroll
    for (int t = 0; t < GW_NT; ++t) acc[u][t] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
  const gg_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  gg_bf16x8 gb[GW_PIECES], wv[2][GW_FT], wn[2][GW_FT];
  // K is a multiple of 32: the last step may hold one half only
  auto ask = [&](int k, gg_bf16x8 (&wa)[2][GW_FT]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < GW_PIECES; ++j)
      gb[j] = (src_live[j] && k + st_part[j] * 8 < K) ? *reinterpret_cast<const gg_bf16x8*>(src[j] + k) : zero;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int u = 0; u < GW_FT; ++u)
        wa[h][u] = (wlive[u] && k + h * 32 < K) ? *reinterpret_cast<const gg_bf16x8*>(wrow[u] + k + h * 32) : zero;
  };
  auto put = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < GW_PIECES; ++j) *reinterpret_cast<gg_bf16x8*>(&Bs[buf][st_row[j]][st_part[j] * 8]) = gb[j];
  };
  ask(0, wv);
  put(0);
  __syncthreads();
  int cur = 0;
  for (int k = 0; k < K; k += GW_KS) {
    const bool more = k + GW_KS < K;
    if (more) ask(k + GW_KS, wn);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int t = 0; t < GW_NT; ++t) {
        const gg_bf16x8 bv = *reinterpret_cast<const gg_bf16x8*>(&Bs[cur][t * 16 + col][h * 32 + kq * 8]);
#pragma unroll
        for (int u = 0; u < GW_FT; ++u) acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[h][u], bv, acc[u][t], 0, 0, 0);
      }
    if (more) {
      put(cur ^ 1);
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int u = 0; u < GW_FT; ++u) wv[h][u] = wn[h][u];
    }
    __syncthreads();
    cur ^= 1;
  }
#pragma unroll
  for (int t = 0; t < GW_NT; ++t) {
    const int item = s_item[t * 16 + col];
    if (item < 0) continue;
    const size_t dst = out_scatter ? (size_t)item : (size_t)(tile * GW_TM + t * 16 + col);
#pragma unroll
    for (int u = 0; u < GW_FT; ++u) {
      const int f = f0 + u * 16 + kq * 4;
      TO* op = out + dst * out_stride + f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = act ? gelu_erf(acc[u][t][i]) : acc[u][t][i];
        if (f + i < n_out) op[i] = from_float<TO>(v);
      }
    }
  }
}

// out[n, :] = sum_j weights[n, j] * (ids[n, j] < n_experts ? part[n * top + j, :] : h[n, :]) + sigmoid(gate[n]) * shared[n, :]
template <typename T, typename TS>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ part, const int* __restrict__ ids, const float* __restrict__ weights,
                   const T* __restrict__ h, size_t h_stride, const TS* __restrict__ shared, const float* __restrict__ gate,
                   size_t gate_stride, float* __restrict__ out, int top, int n_experts, int H) {
  const int n = blockIdx.x;
  __shared__ int s_id[ROUTE_MAX_TOP];
  __shared__ float s_w[ROUTE_MAX_TOP];
  if ((int)threadIdx.x < top) {
    s_id[threadIdx.x] = ids[(size_t)n * top + threadIdx.x];
    s_w[threadIdx.x] = weights ? weights[(size_t)n * top + threadIdx.x] : 1.0f;
  }
  __syncthreads();
  float g = 0.f;
  if (shared) { const float z = gate[(size_t)n * gate_stride]; g = 1.0f / (1.0f + expf(-z)); }
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j) {
      const float v = s_id[j] < n_experts ? part[((size_t)n * top + j) * H + i] : to_float(h[(size_t)n * h_stride + i]);
      acc = fmaf(s_w[j], v, acc);
    }
    if (shared) acc = fmaf(g, to_float(shared[(size_t)n * H + i]), acc);
    out[(size_t)n * H + i] = acc;
  }
}

}  // namespace

extern "C" int ms_gelu(const void* x, void* out, long long total, int dtype, hipStream_t stream) {
  if (total <= 0) return MS_OK;
  int blocks = (int)((total / 4 + 255) / 256) + 1;
  if (blocks > 8192) blocks = 8192;
  if (dtype == MS_F32) gelu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, (float*)out, (size_t)total);
  else if (dtype == MS_BF16) gelu_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)x, (bf16*)out, (size_t)total);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_moe_route(const float* logits, long long ld, const float* correction, int n_tokens, int n_out, int top,
                            int* ids, float* weights, int sigmoid_scores, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (n_out <= 0 || top <= 0 || top > n_out) return MS_BAD_ARG;
  if (n_out > ROUTE_MAX_PER_LANE * MS_WAVE || top > ROUTE_MAX_TOP) return MS_UNSUPPORTED;
  moe_route_kernel<<<(n_tokens + 3) / 4, 256, 0, stream>>>(logits, (size_t)ld, correction, n_tokens, n_out, top, ids,
                                                           weights, sigmoid_scores);
  return ms_launch_status();
}

extern "C" int ms_moe_tile_rows() { return GM; }
extern "C" int ms_moe_wide_tile_rows() { return GW_TM; }

// tile: rows of a tile, 16 (the tile of every product here), or 128 or 256 (of the matrix-core products alone)
extern "C" int ms_moe_align(const int* ids, int n_items, int n_experts, int tile, int tiles, int* rows, int* tile_expert,
                            hipStream_t stream) {
  if (n_items <= 0 || tiles <= 0) return MS_OK;
  if (n_experts <= 0 || (tile != GM && tile != GW_TM && tile != ms_gemm_tiled_grouped_rows())) return MS_BAD_ARG;
  if (n_experts > 4096) return MS_UNSUPPORTED;
  if ((long long)tiles * tile < (long long)n_items + (long long)n_experts * (tile - 1)) return MS_BAD_ARG;
  moe_align_kernel<<<1, 1024, (2 * n_experts + 1) * sizeof(int), stream>>>(ids, n_items, n_experts, tile, tiles, rows,
                                                                          tile_expert);
  return ms_launch_status();
}

// Whether ms_grouped_gemm takes the product to the matrix cores (tiles of `tile` rows).
extern "C" int ms_grouped_gemm_mfma_ok(int K, long long in_stride, long long out_stride, int tile, int dtype, int out_dtype) {
  return dtype == MS_BF16 && K % 32 == 0 && in_stride % 8 == 0 && (tile == GM || tile == GW_TM) &&
         (out_dtype == MS_F32 || out_dtype == MS_BF16);
}

extern "C" int ms_grouped_gemm(const void* in, long long in_stride, const void* w, const int* rows, const int* tile_expert,
                               void* out, long long out_stride, int tiles, int tile, int n_out, int K, int in_div,
                               int out_scatter, int act, int dtype, int out_dtype, hipStream_t stream) {
  if (tiles <= 0) return MS_OK;
  if (n_out <= 0 || K <= 0 || in_div < 0) return MS_BAD_ARG;
  if (tile == ms_gemm_tiled_grouped_rows() || (tile * 2 == ms_gemm_tiled_grouped_rows() && K % 64 == 0 && dtype == MS_BF16)) {
    // wide tiles with K a multiple of 64: the tiled kernel, operands from memory straight to LDS
    const int rc = dtype == MS_BF16 ? ms_gemm_tiled_grouped(in, in_stride, w, rows, tile_expert, out, out_stride, tiles,
                                                            tile, n_out, K, in_div, out_scatter, act, out_dtype, stream)
                                    : MS_UNSUPPORTED;
    if (rc != MS_UNSUPPORTED || tile == ms_gemm_tiled_grouped_rows()) return rc;
  }
  if (ms_grouped_gemm_mfma_ok(K, in_stride, out_stride, tile, dtype, out_dtype) && ((uintptr_t)in % 16) == 0 &&
      ((uintptr_t)w % 16) == 0) {
    const int slab = tile == GM ? GG_SLAB : GW_SLAB;
    const int slabs = (n_out + slab - 1) / slab;
    if (tiles > 65535) return MS_UNSUPPORTED;
    dim3 grid(slabs, tiles), block(256);
#define LAUNCH_W(TO)                                                                                                  \
  grouped_gemm_mfma_wide_kernel<TO><<<grid, block, 0, stream>>>((const bf16*)in, (size_t)in_stride, (const bf16*)w, rows, \
                                                                tile_expert, (TO*)out, (size_t)out_stride, n_out, K,  \
                                                                in_div, out_scatter, act)
#define LAUNCH_M(NT, TO)                                                                                              \
  grouped_gemm_mfma_kernel<NT, TO><<<grid, block, 0, stream>>>((const bf16*)in, (size_t)in_stride, (const bf16*)w, rows, \
                                                               tile_expert, (TO*)out, (size_t)out_stride, n_out, K,   \
                                                               in_div, out_scatter, act)
    if (tile == GM && out_dtype == MS_F32) LAUNCH_M(1, float);
    else if (tile == GM) LAUNCH_M(1, bf16);
    else if (out_dtype == MS_F32) LAUNCH_W(float);
    else LAUNCH_W(bf16);
#undef LAUNCH_M
#undef LAUNCH_W
    return ms_launch_status();
  }
  if (tile != GM) return MS_UNSUPPORTED;
  const int cb = (n_out + GN - 1) / GN;
  if (cb > 65535) return MS_UNSUPPORTED;
  dim3 grid(tiles, cb), block(256);
#define LAUNCH(T, TO)                                                                                                 \
  grouped_gemm_kernel<T, TO><<<grid, block, 0, stream>>>((const T*)in, (size_t)in_stride, (const T*)w, rows,          \
                                                         tile_expert, (TO*)out, (size_t)out_stride, n_out, K, in_div, \
                                                         out_scatter, act)
  if (dtype == MS_F32 && out_dtype == MS_F32) LAUNCH(float, float);
  else if (dtype == MS_BF16 && out_dtype == MS_F32) LAUNCH(bf16, float);
  else if (dtype == MS_BF16 && out_dtype == MS_BF16) LAUNCH(bf16, bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

extern "C" int ms_moe_combine(const float* part, const int* ids, const float* weights, const void* h, long long h_stride,
                              const void* shared, int shared_dtype, const float* gate, long long gate_stride, float* out,
                              int n_tokens, int top, int n_experts, int hidden, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (top <= 0 || top > ROUTE_MAX_TOP || hidden <= 0 || (shared != nullptr && gate == nullptr)) return MS_BAD_ARG;
  dim3 grid(n_tokens), block(256);
#define LAUNCH(T, TS)                                                                                                \
  moe_combine_kernel<T, TS><<<grid, block, 0, stream>>>(part, ids, weights, (const T*)h, (size_t)h_stride,           \
                                                        (const TS*)shared, gate, (size_t)gate_stride, out, top,      \
                                                        n_experts, hidden)
  if (dtype == MS_F32) LAUNCH(float, float);
  else if (dtype == MS_BF16 && shared_dtype == MS_F32) LAUNCH(bf16, float);
  else if (dtype == MS_BF16) LAUNCH(bf16, bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
