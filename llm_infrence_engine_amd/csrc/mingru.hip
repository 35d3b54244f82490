// minGRU: a gated recurrence per channel whose gates read the current token only.
//   z = sigmoid(pz + bz);  u = px + bx;  c = u + 1/2 (u >= 0), sigmoid(u) (u < 0);
//   S_t = (1 - z) S_(t-1) + z c;   out = S_t * silu(pg)
// pz | px | pg are the three thirds of a row of one packed product [N, 3C].  S float [slots, C] is carried from step
// to step in the request's slot.  The gates, the candidate, the gate of the read-out and S are float.
//
// The recurrence is linear in S (S_t = a_t S_(t-1) + b_t), so a portion is walked a chunk of W x TPW tokens at a time by
// the W waves of a block, 64 channels a block: every wave loads its TPW tokens at once, folds them into one pair
// (A, B) with S_out = A S_in + B, the pairs of the waves before it give its S_in, and it then walks its tokens again
// from there.  A step of single tokens runs W = 1.
// A step is a ragged batch: request r owns the tokens q_start[r] .. q_start[r+1]-1 and the slot state_slots[r];
// requests without tokens are left alone.
#include "common.h"
#include "api.h"

namespace {

constexpr int GRU_TPW = 8;     // tokens a wave holds in registers

__device__ __forceinline__ float gru_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

template <typename T, int W>
__global__ void __launch_bounds__(W * MS_WAVE)
mingru_scan_kernel(const T* __restrict__ zxg, size_t in_stride, const float* __restrict__ bz, const float* __restrict__ bx,
                   float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
                   T* __restrict__ out, size_t out_stride, int C) {
  __shared__ float sA[W][MS_WAVE], sB[W][MS_WAVE];
  const int r = blockIdx.y;
  const int s0 = q_start[r], L = q_start[r + 1] - s0;
  if (L <= 0) return;
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int ch = blockIdx.x * MS_WAVE + lane;
  const bool live = ch < C;
  const int chl = live ? ch : 0;
  float* Sg = state + (size_t)state_slots[r] * C + chl;
  float S_in = live ? *Sg : 0.f;
  const float biz = bz ? bz[chl] : 0.f, bix = bx ? bx[chl] : 0.f;
  for (int c0 = 0; c0 < L; c0 += W * GRU_TPW) {
    const int t0 = c0 + wave * GRU_TPW;
    float a[GRU_TPW], b[GRU_TPW], gg[GRU_TPW];
    float A = 1.f, B = 0.f;
#pragma unroll
    for (int i = 0; i < GRU_TPW; ++i) {
      const int t = t0 + i;
      a[i] = 1.f; b[i] = 0.f; gg[i] = 0.f;
      if (t < L) {
        const T* p = zxg + (size_t)(s0 + t) * in_stride + chl;
        const float z = gru_sigmoid(to_float(p[0]) + biz);
        const float u = to_float(p[C]) + bix;
        const float g = to_float(p[2 * (size_t)C]);
        const float cand = u >= 0.f ? u + 0.5f : gru_sigmoid(u);
        a[i] = 1.f - z;
        b[i] = z * cand;
        gg[i] = g * gru_sigmoid(g);
      }
      B = fmaf(a[i], B, b[i]);
      A *= a[i];
    }
    float S = S_in;
    if (W > 1) {
      sA[wave][lane] = A; sB[wave][lane] = B;
      __syncthreads();
      float carry = S_in;
      for (int w2 = 0; w2 < W; ++w2) {
        if (w2 == wave) S = carry;
        carry = fmaf(sA[w2][lane], carry, sB[w2][lane]);
      }
      S_in = carry;
      __syncthreads();
    } else {
      S_in = fmaf(A, S_in, B);
    }
#pragma unroll
    for (int i = 0; i < GRU_TPW; ++i) {
      const int t = t0 + i;
      S = fmaf(a[i], S, b[i]);
      if (t < L && live) out[(size_t)(s0 + t) * out_stride + ch] = from_float<T>(S * gg[i]);
    }
  }
  if (wave == 0 && live) *Sg = S_in;
}

}  // namespace

// zxg [N, >= 3 C] with row stride in_stride; bz, bx float [C] (may be null); state float [slots, C]; out [N, C].
// long_portions: the step has portions of more than a few tokens.
extern "C" int ms_mingru_scan(const void* zxg, long long in_stride, const float* bz, const float* bx, float* state,
                              const int* q_start, const int* state_slots, void* out, long long out_stride,
                              int n_requests, int C, int long_portions, int dtype, hipStream_t stream) {
  if (n_requests <= 0) return MS_OK;
  if (C <= 0 || in_stride < 3ll * C || out_stride < C) return MS_BAD_ARG;
  if (n_requests > 65535) return MS_UNSUPPORTED;
  dim3 grid((C + MS_WAVE - 1) / MS_WAVE, n_requests);
#define LAUNCH(T, W)                                                                                                 \
  mingru_scan_kernel<T, W><<<grid, dim3(W * MS_WAVE), 0, stream>>>((const T*)zxg, (size_t)in_stride, bz, bx, state,  \
                                                                   q_start, state_slots, (T*)out, (size_t)out_stride, C)
  if (dtype == MS_F32) { if (long_portions) LAUNCH(float, 8); else LAUNCH(float, 1); }
  else if (dtype == MS_BF16) { if (long_portions) LAUNCH(bf16, 8); else LAUNCH(bf16, 1); }
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
