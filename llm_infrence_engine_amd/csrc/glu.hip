// Gated activations that stand between two products and have no place in a product's epilogue.
//
// ms_clamped_glu   gu [N, 2F] with gate and up interleaved (g0, u0, g1, u1, ...):
//                  g = min(g, limit); u = clamp(u, -limit, limit); out = g * sigmoid(alpha g) * (u + 1)
// ms_scaled_swiglu gu [rows, 2F] interleaved, one factor s per row (rows of routed experts: the token's weight for the
//                  expert, which scales what the expert reads; the two products are linear, so the factor is applied
//                  to their results): out = silu(s g) * (s u).  row_item[p] (may be null) names the factor of row p
//                  (factor[row_item[p]]; rows with row_item < 0 are left alone).
// ms_gelu_tanh_glu gu [N, 2F] interleaved: out = gelu_tanh(g) * u, gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// All work in float and round once.
#include "common.h"
#include "api.h"

namespace {

template <typename T>
__global__ void __launch_bounds__(256)
clamped_glu_kernel(const T* __restrict__ gu, size_t in_stride, T* __restrict__ out, size_t out_stride, int n_rows, int F,
                   float limit, float alpha) {
  const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= (long long)n_rows * F) return;
  const int n = (int)(item / F), f = (int)(item - (long long)n * F);
  const T* p = gu + (size_t)n * in_stride + 2 * (size_t)f;
  const float g = fminf(to_float(p[0]), limit);
  const float u = fminf(fmaxf(to_float(p[1]), -limit), limit);
  out[(size_t)n * out_stride + f] = from_float<T>(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
}

template <typename T>
__global__ void __launch_bounds__(256)
scaled_swiglu_kernel(const T* __restrict__ gu, size_t in_stride, const float* __restrict__ factor,
                     const int* __restrict__ row_item, T* __restrict__ out, size_t out_stride, int n_rows, int F) {
  const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= (long long)n_rows * F) return;
  const int n = (int)(item / F), f = (int)(item - (long long)n * F);
  int which = n;
  if (row_item) {
    which = row_item[n];
    if (which < 0) return;
  }
  const float s = factor ? factor[which] : 1.0f;
  const T* p = gu + (size_t)n * in_stride + 2 * (size_t)f;
  const float g = s * to_float(p[0]), u = s * to_float(p[1]);
  out[(size_t)n * out_stride + f] = from_float<T>(g / (1.0f + expf(-g)) * u);
}

template <typename T>
__global__ void __launch_bounds__(256)
gelu_tanh_glu_kernel(const T* __restrict__ gu, size_t in_stride, T* __restrict__ out, size_t out_stride, int n_rows, int F) {
  const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= (long long)n_rows * F) return;
  const int n = (int)(item / F), f = (int)(item - (long long)n * F);
  const T* p = gu + (size_t)n * in_stride + 2 * (size_t)f;
  const float g = to_float(p[0]), u = to_float(p[1]);
  const float act = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  out[(size_t)n * out_stride + f] = from_float<T>(act * u);
}

}  // namespace

extern "C" int ms_clamped_glu(const void* gu, long long in_stride, void* out, long long out_stride, int n_rows, int F,
                              float limit, float alpha, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (F <= 0 || in_stride < 2ll * F || out_stride < F) return MS_BAD_ARG;
  const long long items = (long long)n_rows * F;
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
  if (dtype == MS_F32) clamped_glu_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, (size_t)in_stride, (float*)out, (size_t)out_stride, n_rows, F, limit, alpha);
  else if (dtype == MS_BF16) clamped_glu_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)gu, (size_t)in_stride, (bf16*)out, (size_t)out_stride, n_rows, F, limit, alpha);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_scaled_swiglu(const void* gu, long long in_stride, const float* factor, const int* row_item, void* out,
                                long long out_stride, int n_rows, int F, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (F <= 0 || in_stride < 2ll * F || out_stride < F) return MS_BAD_ARG;
  const long long items = (long long)n_rows * F;
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
  if (dtype == MS_F32) scaled_swiglu_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, (size_t)in_stride, factor, row_item, (float*)out, (size_t)out_stride, n_rows, F);
  else if (dtype == MS_BF16) scaled_swiglu_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)gu, (size_t)in_stride, factor, row_item, (bf16*)out, (size_t)out_stride, n_rows, F);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_gelu_tanh_glu(const void* gu, long long in_stride, void* out, long long out_stride, int n_rows, int F,
                                int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (F <= 0 || in_stride < 2ll * F || out_stride < F) return MS_BAD_ARG;
  const long long items = (long long)n_rows * F;
  dim3 grid((unsigned)((items + 255) / 256)), block(256);
  if (dtype == MS_F32) gelu_tanh_glu_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, (size_t)in_stride, (float*)out, (size_t)out_stride, n_rows, F);
  else if (dtype == MS_BF16) gelu_tanh_glu_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)gu, (size_t)in_stride, (bf16*)out, (size_t)out_stride, n_rows, F);
  else return MS_BAD_ARG;
  return ms_launch_status();
}
