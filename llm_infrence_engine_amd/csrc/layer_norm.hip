// Layer norm with a weight and an optional bias on the float residual stream, the scaled sum that precedes it, and the gate of a
// token's own side input into the stream.
//   v = x[row] (+ scale o delta[row]);   out = w o (v - mean v) / sqrt(mean (v - mean v)^2 + eps) (+ b)
// The row is held in LDS between the passes (mean, then the mean of the squared deviations, as the norm is defined; no
// E[v^2] - E[v]^2), so out may be x itself.  Everything is float; out is rounded once.  Without a weight the kernel is
// the scaled sum alone, and out (if given) takes the summed row rounded to its type: the operand of a product that reads
// the stream itself.
//
// ms_side_gate: g[n, j] = gelu_tanh(z[n, j]) * table[token[n], part d + j], what stands between the two small products
// of a layer's side input (z = G x before it, y = P g after it).
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
                  const float* __restrict__ w, const float* __restrict__ b, const int* __restrict__ rows, TO* out, int H, float eps,
                  int write_back) {
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
    if (w) o[i] = from_float<TO>(b ? fmaf((row[i] - mean) * inv, w[i], b[i]) : (row[i] - mean) * inv * w[i]);
    else if (out) o[i] = from_float<TO>(row[i]);
  }
}

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void __launch_bounds__(256)
side_gate_kernel(const T* __restrict__ z, size_t z_stride, const int* __restrict__ token_ids, const T* __restrict__ table,
                 size_t table_stride, int part, T* __restrict__ out, int n_tokens, int d) {
  const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= (long long)n_tokens * d) return;
  const int n = (int)(item / d), j = (int)(item - (long long)n * d);
  const float c = to_float(table[(size_t)token_ids[n] * table_stride + (size_t)part * d + j]);
  out[(size_t)n * d + j] = from_float<T>(gelu_tanh(to_float(z[(size_t)n * z_stride + j])) * c);
}

}  // namespace

// x float [N, H]; delta (may be null) [N, H] of `delta_dtype`, dscale (may be null) float [H]; w (null: only the sum)
// float [H], b (may be null; only with w) float [H]; rows (may be null) int32 [n_rows]: which rows of x; out [n_rows, H] of `out_dtype` (may be x for float).
extern "C" int ms_layer_norm(float* x, const void* delta, int delta_dtype, const float* dscale, const float* w,
                             const float* b, const int* rows, void* out, int n_rows, int H, float eps, int write_back, int out_dtype,
                             hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (H <= 0 || (w != nullptr && out == nullptr) || (b != nullptr && w == nullptr)) return MS_BAD_ARG;   // w null with out: the summed rows' rounded copy
  if (H > 16384) return MS_UNSUPPORTED;
  const size_t lds = (size_t)H * sizeof(float);
#define LAUNCH(TD, TO)                                                                                               \
  layer_norm_kernel<TD, TO><<<dim3(n_rows), dim3(LN_THREADS), lds, stream>>>(x, (const TD*)delta, dscale, w, b, rows, \
                                                                             (TO*)out, H, eps, write_back)
  const bool dbf = delta != nullptr && delta_dtype == MS_BF16;
  if (delta != nullptr && delta_dtype != MS_BF16 && delta_dtype != MS_F32) return MS_BAD_ARG;
  if (out_dtype == MS_F32) { if (dbf) LAUNCH(bf16, float); else LAUNCH(float, float); }
  else if (out_dtype == MS_BF16) { if (dbf) LAUNCH(bf16, bf16); else LAUNCH(float, bf16); }
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

// z [N, d] (rows z_stride apart), table [vocab, table_stride], out [N, d] of `dtype`; token_ids int32 [N].
extern "C" int ms_side_gate(const void* z, long long z_stride, const int* token_ids, const void* table, long long table_stride,
                            int part, void* out, int n_tokens, int d, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (d <= 0 || part < 0 || (long long)(part + 1) * d > table_stride || z_stride < d) return MS_BAD_ARG;
  const long long items = (long long)n_tokens * d;
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
  if (dtype == MS_F32) side_gate_kernel<float><<<grid, block, 0, stream>>>((const float*)z, (size_t)z_stride, token_ids, (const float*)table, (size_t)table_stride, part, (float*)out, n_tokens, d);
  else if (dtype == MS_BF16) side_gate_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)z, (size_t)z_stride, token_ids, (const bf16*)table, (size_t)table_stride, part, (bf16*)out, n_tokens, d);
  else return MS_BAD_ARG;
  return ms_launch_status();
}
