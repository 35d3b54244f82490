// What lies between the packed q/k/v projection and attention for heads that are normalised instead of rotated:
// the RMS norm of every query and key head (one weight per entry, shared by the heads), a query temperature that
// grows with the logarithm of the position,
//   q <- q * (1 + coef * ln(floor((p + 1) / every) + 1)),
// optionally a rotation of the first rot_dim entries of every q and k head (entry i with entry i + rot_dim / 2, by the
// angle position * inv_freq[i], after the norm), and the store of k and v into the cache pages.  `unit_norm`: heads are
// divided by their root mean square even where no weight is given.  Keys and values may have different sizes.
// qkv [N, nh * d + nkv * d + nkv * dv]; q and k are rewritten in place.  Norms, logarithm, temperature, angles, sines
// and cosines are float.
#include "common.h"
#include "api.h"

namespace {

constexpr int MAX_HEAD = 256;   // the longest head the rotation can hold in LDS (the attention kernels' own limit)

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_store_kernel(T* __restrict__ qkv, size_t stride, const float* __restrict__ q_w, const float* __restrict__ k_w,
                     float eps, const int* __restrict__ positions, float coef, int every,
                     const int* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages, long long items,
                     int nh, int nkv, int d, int dv, int page_size, int v_transposed, int unit_norm,
                     const float* __restrict__ inv_freq, int rot_dim) {
  __shared__ float head[4][MAX_HEAD];
  const int wave = threadIdx.x / MS_WAVE;
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const long long item = (long long)blockIdx.x * (blockDim.x / MS_WAVE) + threadIdx.x / MS_WAVE;
  if (item >= items) return;
  const int per_token = nh + 2 * nkv;
  const long long n = item / per_token;
  const int h = (int)(item - n * per_token);
  T* row = qkv + (size_t)n * stride;
  const int slot = slots ? slots[n] : -1;
  if (h < nh + nkv) {
    const bool is_q = h < nh;
    T* p = row + (size_t)h * d;   // k heads follow the q heads at the same width
    const float* w = is_q ? q_w : k_w;
    float mult = 1.f;
    if (w || unit_norm) {
      float ss = 0.f;
      for (int i = lane; i < d; i += MS_WAVE) { const float v = to_float(p[i]); ss = fmaf(v, v, ss); }
      ss = wave_sum(ss);
      mult = 1.0f / sqrtf(ss / (float)d + eps);
    }
    float temp = 1.f;
    if (is_q && coef != 0.f) temp = 1.0f + coef * logf((float)((positions[n] + 1) / every + 1));
    T* kp = nullptr;
    if (!is_q && k_pages && slot >= 0) {
      const int page = slot / page_size, off = slot % page_size;
      kp = k_pages + (((size_t)page * nkv + (h - nh)) * page_size + off) * d;
    }
    if (rot_dim > 0) {
      // the normed head waits in LDS: the two entries of a pair may belong to different lanes
      for (int i = lane; i < d; i += MS_WAVE) {
        float v = to_float(p[i]) * mult;
        if (w) v *= w[i];
        head[wave][i] = v * temp;
      }
      __builtin_amdgcn_wave_barrier();
      const int half = rot_dim / 2;
      const float pos = (float)positions[n];
      for (int i = lane; i < d; i += MS_WAVE) {
        float v = head[wave][i];
        if (i < rot_dim) {
          const int j = i < half ? i : i - half;
          float sn, cs;
          sincosf(pos * inv_freq[j], &sn, &cs);
          v = i < half ? head[wave][i] * cs - head[wave][i + half] * sn : head[wave][i] * cs + head[wave][i - half] * sn;
        }
        const T r = from_float<T>(v);
        p[i] = r;
        if (kp) kp[i] = r;
      }
    } else {
      for (int i = lane; i < d; i += MS_WAVE) {
        float v = to_float(p[i]) * mult;
        if (w) v *= w[i];
        const T r = from_float<T>(v * temp);
        p[i] = r;
        if (kp) kp[i] = r;
      }
    }
  } else if (v_pages && slot >= 0) {
    const int g = h - nh - nkv;
    const T* p = row + (size_t)(nh + nkv) * d + (size_t)g * dv;
    const int page = slot / page_size, off = slot % page_size;
    if (v_transposed) {
      T* vp = v_pages + ((size_t)page * nkv + g) * dv * page_size + off;
      for (int i = lane; i < dv; i += MS_WAVE) vp[(size_t)i * page_size] = p[i];
    } else {
      T* vp = v_pages + (((size_t)page * nkv + g) * page_size + off) * dv;
      for (int i = lane; i < dv; i += MS_WAVE) vp[i] = p[i];
    }
  }
}

}  // namespace

extern "C" int ms_qk_norm_store(void* qkv, long long stride, const float* q_weight, const float* k_weight, float eps,
                                const int* positions, float coef, int every, const int* slots, void* k_pages,
                                void* v_pages, int n_tokens, int num_heads, int num_kv_heads, int head_dim, int value_dim,
                                int page_size, int v_transposed, int unit_norm, const float* inv_freq, int rot_dim, int dtype,
                                hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || value_dim <= 0) return MS_BAD_ARG;
  if (coef != 0.f && (positions == nullptr || every <= 0)) return MS_BAD_ARG;
  if (rot_dim < 0 || rot_dim % 2 || rot_dim > head_dim || (rot_dim > 0 && (positions == nullptr || inv_freq == nullptr)))
    return MS_BAD_ARG;
  if (rot_dim > 0 && head_dim > MAX_HEAD) return MS_UNSUPPORTED;
  if ((k_pages != nullptr) != (v_pages != nullptr) || (k_pages != nullptr && (slots == nullptr || page_size <= 0)))
    return MS_BAD_ARG;
  const long long items = (long long)n_tokens * (num_heads + 2 * num_kv_heads);
  const int waves = 4;
  dim3 grid((unsigned)((items + waves - 1) / waves)), block(waves * MS_WAVE);
#define LAUNCH(T)                                                                                                    \
  qk_norm_store_kernel<T><<<grid, block, 0, stream>>>((T*)qkv, (size_t)stride, q_weight, k_weight, eps, positions,  \
                                                      coef, every, slots, (T*)k_pages, (T*)v_pages, items, num_heads, \
                                                      num_kv_heads, head_dim, value_dim, page_size, v_transposed, unit_norm, \
                                                      inv_freq, rot_dim)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
