// Layer norm with a weight and no bias on the float residual stream, the scaled sum that precedes it, and a token's
// own side input into the stream.
//   v = x[row] (+ scale o delta[row]);   out = w o (v - mean v) / sqrt(mean (v - mean v)^2 + eps)
// The row is held in LDS between the passes (mean, then the mean of the squared deviations, as the norm is defined; no
// E[v^2] - E[v]^2), so out may be x itself.  Everything is float; out is rounded once.
//
// Side input of layer i for token n (c = side_table[token, i d .. i d + d - 1], d small):
//   g = gelu_tanh(G v) o c;   y = P g;   x[n] = v + y / sqrt(mean y^2 + eps) o w_side
// one block per token: G [d, H] row by row over the waves, P [H, d] a row per thread.
#include "common.h"
#include "api.h"

namespace {

constexpr int LN_THREADS = 256;

template <typename TD>
__device__ __forceinline__ void load_row(float* __restrict__ row, const float* __restrict__ x, const TD* __restrict__ delta,
                                         const float* __restrict__ dscale, int H) {
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (delta) v += (dscale ? dscale[i] : 1.0f) * to_float(delta[i]);
    row[i] = v;
  }
}

template <typename TD, typename TO>
__global__ void __launch_bounds__(LN_THREADS)
layer_norm_kernel(float* __restrict__ x, const TD* __restrict__ delta, const float* __restrict__ dscale,
                  const float* __restrict__ w, const int* __restrict__ rows, TO* out, int H, float eps, int write_back) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const size_t src = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  float* xr = x + src * H;
  load_row<TD>(row, xr, delta ? delta + src * H : nullptr, dscale, H);
  __syncthreads();
  float s = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) s += row[i];
  const float mean = block_sum(s, red) / (float)H;
  float q = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) { const float d = row[i] - mean; q = fmaf(d, d, q); }
  const float inv = 1.0f / sqrtf(block_sum(q, red) / (float)H + eps);
  TO* o = out + (size_t)blockIdx.x * H;
  const bool same = (const void*)o == (const void*)xr;     // the norm in place: x takes the normed row, not the sum
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    if (delta && write_back && !same) xr[i] = row[i];
    if (w) o[i] = from_float<TO>((row[i] - mean) * inv * w[i]);
  }
}

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T, typename TD>
__global__ void __launch_bounds__(LN_THREADS)
token_side_kernel(float* __restrict__ x, const TD* __restrict__ delta, const float* __restrict__ dscale,
                  const int* __restrict__ token_ids, const T* __restrict__ table, size_t table_stride, int part,
                  const T* __restrict__ G, const T* __restrict__ P, const float* __restrict__ w, int H, int d, float eps) {
  extern __shared__ float sh[];
  float* row = sh;            // [H]
  float* y = sh + H;          // [H]
  float* g = sh + 2 * H;      // [d]
  __shared__ float red[16];
  const size_t n = blockIdx.x;
  float* xr = x + n * H;
  load_row<TD>(row, xr, delta ? delta + n * H : nullptr, dscale, H);
  __syncthreads();
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE, waves = blockDim.x / MS_WAVE;
  const T* c = table + (size_t)token_ids[n] * table_stride + (size_t)part * d;
  for (int j = wave; j < d; j += waves) {
    const T* gj = G + (size_t)j * H;
    float dot = 0.f;
    for (int i = lane; i < H; i += MS_WAVE) dot = fmaf(to_float(gj[i]), row[i], dot);
    dot = wave_sum(dot);
    if (lane == 0) g[j] = gelu_tanh(dot) * to_float(c[j]);
  }
  __syncthreads();
  float q = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const T* pi = P + (size_t)i * d;
    float v = 0.f;
    for (int j = 0; j < d; ++j) v = fmaf(to_float(pi[j]), g[j], v);
    y[i] = v;
    q = fmaf(v, v, q);
  }
  const float inv = 1.0f / sqrtf(block_sum(q, red) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) xr[i] = row[i] + y[i] * inv * w[i];
}

}  // namespace

// x float [N, H]; delta (may be null) [N, H] of `delta_dtype`, dscale (may be null) float [H]; w (null: only the sum)
// float [H]; rows (may be null) int32 [n_rows]: which rows of x; out [n_rows, H] of `out_dtype` (may be x for float).
extern "C" int ms_layer_norm(float* x, const void* delta, int delta_dtype, const float* dscale, const float* w,
                             const int* rows, void* out, int n_rows, int H, float eps, int write_back, int out_dtype,
                             hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (H <= 0 || (w != nullptr && out == nullptr)) return MS_BAD_ARG;
  if (H > 16384) return MS_UNSUPPORTED;
  const size_t lds = (size_t)H * sizeof(float);
#define LAUNCH(TD, TO)                                                                                               \
  layer_norm_kernel<TD, TO><<<dim3(n_rows), dim3(LN_THREADS), lds, stream>>>(x, (const TD*)delta, dscale, w, rows,   \
                                                                             (TO*)out, H, eps, write_back)
  const bool dbf = delta != nullptr && delta_dtype == MS_BF16;
  if (delta != nullptr && delta_dtype != MS_BF16 && delta_dtype != MS_F32) return MS_BAD_ARG;
  if (out_dtype == MS_F32) { if (dbf) LAUNCH(bf16, float); else LAUNCH(float, float); }
  else if (out_dtype == MS_BF16) { if (dbf) LAUNCH(bf16, bf16); else LAUNCH(float, bf16); }
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

// table [vocab, table_stride] and the matrices G [d, H], P [H, d] of `dtype`; token_ids int32 [N]; w float [H].
extern "C" int ms_token_side(float* x, const void* delta, int delta_dtype, const float* dscale, const int* token_ids,
                             const void* table, long long table_stride, int part, const void* G, const void* P,
                             const float* w, int n_tokens, int H, int d, float eps, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (H <= 0 || d <= 0 || part < 0 || (long long)(part + 1) * d > table_stride) return MS_BAD_ARG;
  if (2 * (size_t)H + d > 15000) return MS_UNSUPPORTED;     // 60 KB of LDS
  const size_t lds = (2 * (size_t)H + d) * sizeof(float);
#define LAUNCH(T, TD)                                                                                                \
  token_side_kernel<T, TD><<<dim3(n_tokens), dim3(LN_THREADS), lds, stream>>>(                                       \
      x, (const TD*)delta, dscale, token_ids, (const T*)table, (size_t)table_stride, part, (const T*)G, (const T*)P, w, H, d, eps)
  const bool dbf = delta != nullptr && delta_dtype == MS_BF16;
  if (delta != nullptr && delta_dtype != MS_BF16 && delta_dtype != MS_F32) return MS_BAD_ARG;
  if (dtype == MS_F32) { if (dbf) LAUNCH(float, bf16); else LAUNCH(float, float); }
  else if (dtype == MS_BF16) { if (dbf) LAUNCH(bf16, bf16); else LAUNCH(bf16, float); }
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
