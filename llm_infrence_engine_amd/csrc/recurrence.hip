// Recurrences over a float state S [D, E] per request and head whose rows decay by a factor of their own (one per head
// and key channel, made from the token), and the small kernels around them.
//
// ms_decay_recurrence   S <- diag(w_t) S + k_t v_t^T with the read-out either after the write, o_t = S_t^T q_t, or
//                       (`bonus` u [H, D] given) before it with the current token weighted by u:
//                       o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t.  The decay comes from z [N, H * D] float (+ z_bias):
//                       kind 0: w = sigmoid(z)^(inv_tau) = exp(-softplus(-z) * inv_tau);  kind 1: w = exp(-exp(z)).
// ms_token_shift        out[m][n] = h[n] + (h'[n] - h[n]) o mu[m], h' the previous token's h (the request's state slot for
//                       the first token of a portion: zero at a request's start); then the state becomes the portion's last h.
// ms_pair_sum           x[n] += sa f(a[n]) + sb g(b[n]) on the float residual stream, f the identity or a[n] / rms(a[n]) o wa.
// ms_concat_rows        out[n] = [a[n] | b[n]] rounded to the products' type (a, b float).
// ms_tanh               x <- tanh(x) in place.
//
// A step is a ragged batch: request r owns the tokens q_start[r] .. q_start[r+1]-1 and the state slot state_slots[r];
// requests without tokens and tokens of no request pad a captured batch and are left alone.  States, decays and their
// exponentials, sums and norms are float in every mode.
#include "common.h"
#include "api.h"

namespace {

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// the sum over LPC neighbouring lanes (a power of two up to 16, groups aligned), every lane getting it
template <int LPC> __device__ __forceinline__ float group_sum(float v) {
  if (LPC >= 2) v += dpp_move<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  if (LPC >= 4) v += dpp_move<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  if (LPC >= 8) v += dpp_move<0x141>(v);    // row_half_mirror
  if (LPC >= 16) v += dpp_move<0x140>(v);   // row_mirror
  return v;
}

constexpr int REC_THREADS = 256;
constexpr int REC_CHUNK = 16;     // tokens staged at a time
constexpr int DPT = 16;           // rows of a column a lane holds

// Column j of S depends on no other column: LPC neighbouring lanes hold it (DPT rows each) for the whole portion.  A
// block owns REC_THREADS / LPC columns of one (request, head).  Tokens are staged a chunk at a time (q scaled, k, the
// decay worked out, v) as floats in LDS, then walked in order.
//
// A long portion is spread over blocks (MODE 1, then MODE 2; MODE 0 walks the whole portion in one block): the recurrence
// is linear in S, so a stretch of `stretch` tokens maps the state it starts from to diag(A) S + B, A the product of its
// decays and B what it leaves when started from zero.  MODE 1: every stretch but a portion's last walks from zero and
// leaves A and B in scratch; the last one's block puts a copy of the request's state there instead (its own pair is never
// asked for), so that the second launch, whose last stretch overwrites the state, reads the state from the copy whenever
// its blocks run.  MODE 2: every stretch folds the pairs of the stretches before it onto that copy, in order, walks from
// there and writes the read-outs; the last one stores the state.  blockIdx.z = request * stretches
// a request may have + the stretch's index.
template <typename T, int LPC, bool BONUS, int MODE>
__global__ void __launch_bounds__(REC_THREADS)
decay_recurrence_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, size_t q_stride,
                        size_t k_stride, size_t v_stride, const float* __restrict__ z, const float* __restrict__ z_bias,
                        int decay_kind, float inv_tau, const float* __restrict__ bonus, float q_scale,
                        float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
                        float* __restrict__ out, int H, int D, int E, int stretch, int max_stretches,
                        float* __restrict__ pair_a, float* __restrict__ pair_b) {
  constexpr int Dp = DPT * LPC, COLS = REC_THREADS / LPC;
  __shared__ __align__(16) float qs[REC_CHUNK * Dp];
  __shared__ __align__(16) float ks[REC_CHUNK * Dp];
  __shared__ __align__(16) float ws[REC_CHUNK * Dp];
  __shared__ float vs[REC_CHUNK * COLS];
  const int r = MODE == 0 ? blockIdx.z : blockIdx.z / max_stretches, h = blockIdx.y, col0 = blockIdx.x * COLS;
  const int piece = MODE == 0 ? 0 : blockIdx.z - r * max_stretches;
  const int s0 = q_start[r], L = q_start[r + 1] - s0;
  if (L <= 0) return;
  const int t_begin = MODE == 0 ? 0 : piece * stretch;
  const int t_end = MODE == 0 ? L : min(L, t_begin + stretch);
  if (t_begin >= L) return;
  const int tid = threadIdx.x, part = tid % LPC, my = tid / LPC, col = col0 + my;
  const bool live = col < E;
  float* Sg = state + (((size_t)state_slots[r] * H + h) * D) * E;
  float S[DPT], U[DPT], A[MODE == 1 ? DPT : 1];
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = part * DPT + ii;
    S[ii] = (MODE == 0 && live && i < D) ? Sg[(size_t)i * E + col] : 0.f;
    U[ii] = (BONUS && i < D) ? bonus[(size_t)h * D + i] : 0.f;
    if (MODE == 1) A[ii] = 1.f;
  }
  if (MODE == 1 && t_end == L) {      // a portion's last stretch: the state's copy
    const size_t at = ((size_t)r * max_stretches + piece) * H + h;
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = part * DPT + ii;
      if (live && i < D) pair_b[(at * D + i) * E + col] = Sg[(size_t)i * E + col];
    }
    return;
  }
  if (MODE == 2) {
    const size_t copy = ((size_t)r * max_stretches + (L - 1) / stretch) * H + h;
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = part * DPT + ii;
      if (live && i < D) S[ii] = pair_b[(copy * D + i) * E + col];
    }
    for (int c = 0; c < piece; ++c) {
      const size_t at = ((size_t)r * max_stretches + c) * H + h;
#pragma unroll
      for (int ii = 0; ii < DPT; ++ii) {
        const int i = part * DPT + ii;
        if (live && i < D) S[ii] = fmaf(pair_a[at * D + i], S[ii], pair_b[(at * D + i) * E + col]);
      }
    }
  }
  for (int c0 = t_begin; c0 < t_end; c0 += REC_CHUNK) {
    const int cn = min(REC_CHUNK, t_end - c0);
    __syncthreads();      // the chunk before has been walked
    for (int e = tid; e < cn * Dp; e += REC_THREADS) {
      const int t = e / Dp, i = e - t * Dp;
      float qv = 0.f, kv = 0.f, wv = 1.f;
      if (i < D) {
        const size_t n = (size_t)(s0 + c0 + t);
        qv = to_float(q[n * q_stride + (size_t)h * D + i]) * q_scale;
        kv = to_float(k[n * k_stride + (size_t)h * D + i]);
        float zz = z[n * (size_t)H * D + (size_t)h * D + i];
        if (z_bias) zz += z_bias[(size_t)h * D + i];
        wv = decay_kind == 0 ? expf(-softplus_f(-zz) * inv_tau) : expf(-expf(zz));
      }
      qs[e] = qv; ks[e] = kv; ws[e] = wv;
    }
    for (int e = tid; e < cn * COLS; e += REC_THREADS) {
      const int t = e / COLS, j = e - t * COLS;
      vs[e] = col0 + j < E ? to_float(v[(size_t)(s0 + c0 + t) * v_stride + (size_t)h * E + col0 + j]) : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < cn; ++t) {
      const float* qt = qs + t * Dp + part * DPT;
      const float* kt = ks + t * Dp + part * DPT;
      const float* wt = ws + t * Dp + part * DPT;
      const float vt = vs[t * COLS + my];
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DPT; ii += 4) {
        const float4 q4 = *reinterpret_cast<const float4*>(qt + ii);
        const float4 k4 = *reinterpret_cast<const float4*>(kt + ii);
        const float4 w4 = *reinterpret_cast<const float4*>(wt + ii);
        const float qq[4] = {q4.x, q4.y, q4.z, q4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float write = kk[j] * vt;
          if (MODE == 1) {
            S[ii + j] = fmaf(ww[j], S[ii + j], write);
            A[ii + j] *= ww[j];
          } else if (BONUS) {
            o4[j] = fmaf(fmaf(U[ii + j], write, S[ii + j]), qq[j], o4[j]);
            S[ii + j] = fmaf(ww[j], S[ii + j], write);
          } else {
            S[ii + j] = fmaf(ww[j], S[ii + j], write);
            o4[j] = fmaf(S[ii + j], qq[j], o4[j]);
          }
        }
      }
      if (MODE != 1) {
        const float o = group_sum<LPC>((o4[0] + o4[1]) + (o4[2] + o4[3]));
        if (live && part == 0) out[((size_t)(s0 + c0 + t) * H + h) * E + col] = o;
      }
    }
  }
  if (MODE == 1) {
    const size_t at = ((size_t)r * max_stretches + piece) * H + h;
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = part * DPT + ii;
      if (live && i < D) pair_b[(at * D + i) * E + col] = S[ii];
      if (blockIdx.x == 0 && my == 0 && i < D) pair_a[at * D + i] = A[ii];
    }
    return;
  }
  if (t_end < L) return;      // (MODE 2) only a portion's last stretch leaves the state
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = part * DPT + ii;
    if (live && i < D) Sg[(size_t)i * E + col] = S[ii];
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ h, size_t h_stride, const float* __restrict__ mu, const T* __restrict__ state,
                   const int* __restrict__ token_req, const int* __restrict__ q_start, const int* __restrict__ state_slots,
                   const int* __restrict__ n_live_tokens, T* __restrict__ out, int N, int W, int M) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  if (n_live_tokens && n >= *n_live_tokens) return;
  const int r = token_req[n];
  const float cur = to_float(h[(size_t)n * h_stride + c]);
  const float prev = n > q_start[r] ? to_float(h[(size_t)(n - 1) * h_stride + c]) : to_float(state[(size_t)state_slots[r] * W + c]);
  const float d = prev - cur;
  for (int m = 0; m < M; ++m)
    out[((size_t)m * N + n) * W + c] = from_float<T>(fmaf(d, mu[(size_t)m * W + c], cur));
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_update_kernel(const T* __restrict__ h, size_t h_stride, T* __restrict__ state, const int* __restrict__ q_start,
                          const int* __restrict__ state_slots, int W) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int end = q_start[r + 1];
  if (end <= q_start[r]) return;
  state[(size_t)state_slots[r] * W + c] = h[(size_t)(end - 1) * h_stride + c];
}

template <typename T>
__global__ void __launch_bounds__(256)
pair_sum_kernel(const T* __restrict__ a, const T* __restrict__ b, float sa, float sb, const float* __restrict__ wa,
                const float* __restrict__ wb, float eps, float* __restrict__ x, int W) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * W;
  float fa = sa, fb = sb;
  if (wa) {
    float s = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) { const float t = to_float(a[row + i]); s = fmaf(t, t, s); }
    fa = sa / sqrtf(block_sum(s, red) / (float)W + eps);
  }
  if (wb) {
    float s = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) { const float t = to_float(b[row + i]); s = fmaf(t, t, s); }
    fb = sb / sqrtf(block_sum(s, red) / (float)W + eps);
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float ta = to_float(a[row + i]) * fa * (wa ? wa[i] : 1.f);
    const float tb = to_float(b[row + i]) * fb * (wb ? wb[i] : 1.f);
    x[row + i] += ta + tb;
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, T* __restrict__ out, int Wa, int Wb) {
  const size_t n = blockIdx.x;
  T* o = out + n * (size_t)(Wa + Wb);
  for (int i = threadIdx.x; i < Wa; i += blockDim.x) o[i] = from_float<T>(a[n * Wa + i]);
  for (int i = threadIdx.x; i < Wb; i += blockDim.x) o[Wa + i] = from_float<T>(b[n * Wb + i]);
}

template <typename T>
__global__ void __launch_bounds__(256) tanh_kernel(T* __restrict__ x, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] = from_float<T>(tanhf(to_float(x[i])));
}

}  // namespace

// x <- tanh(x), in place; `total` values of `dtype`.
extern "C" int ms_tanh(void* x, long long total, int dtype, hipStream_t stream) {
  if (total <= 0) return MS_OK;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == MS_F32) tanh_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, (size_t)total);
  else if (dtype == MS_BF16) tanh_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)x, (size_t)total);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

// q, k [N, >= heads * dim] and v [N, >= heads * vdim] of `dtype`, rows q_stride / k_stride / v_stride elements apart;
// z float [N, heads * dim], z_bias (may be null) float [heads * dim]; bonus (may be null) float [heads * dim];
// state float [slots, heads, dim, vdim]; out float [N, heads * vdim].  max_stretches > 1: every portion is cut into
// stretches of `stretch` tokens (no portion has more than max_stretches of them) that run side by side in two launches;
// pair_a float [n_requests, max_stretches, heads, dim] and pair_b float [n_requests, max_stretches, heads, dim, vdim] are
// scratch.
extern "C" int ms_decay_recurrence(const void* q, const void* k, const void* v, long long q_stride, long long k_stride,
                                   long long v_stride, const float* z, const float* z_bias, int decay_kind, float inv_tau,
                                   const float* bonus, float q_scale, float* state, const int* q_start,
                                   const int* state_slots, float* out, int n_requests, int heads, int dim, int vdim,
                                   int stretch, int max_stretches, float* pair_a, float* pair_b, int dtype,
                                   hipStream_t stream) {
  if (n_requests <= 0) return MS_OK;
  if (heads <= 0 || dim <= 0 || vdim <= 0 || (decay_kind != 0 && decay_kind != 1)) return MS_BAD_ARG;
  if (q_stride < (long long)heads * dim || k_stride < (long long)heads * dim || v_stride < (long long)heads * vdim)
    return MS_BAD_ARG;
  if (dim > DPT * 16) return MS_UNSUPPORTED;
  const bool spread = max_stretches > 1;
  if (spread && (stretch <= 0 || pair_a == nullptr || pair_b == nullptr)) return MS_BAD_ARG;
  if (spread && (long long)n_requests * max_stretches > 65535) return MS_UNSUPPORTED;
  int lpc = 1;
  while (lpc * DPT < dim) lpc *= 2;
  const int cols = REC_THREADS / lpc;
  dim3 grid((unsigned)((vdim + cols - 1) / cols), (unsigned)heads, (unsigned)(n_requests * (spread ? max_stretches : 1)));
  dim3 block(REC_THREADS);
#define LAUNCH4(T, LPC, B, MODE)                                                                                     \
  decay_recurrence_kernel<T, LPC, B, MODE><<<grid, block, 0, stream>>>((const T*)q, (const T*)k, (const T*)v,        \
      (size_t)q_stride, (size_t)k_stride, (size_t)v_stride, z, z_bias, decay_kind, inv_tau, bonus, q_scale, state, q_start, \
      state_slots, out, heads, dim, vdim, stretch, max_stretches, pair_a, pair_b)
#define LAUNCH3(T, LPC, B)                                                                                           \
  do { if (spread) { LAUNCH4(T, LPC, B, 1); LAUNCH4(T, LPC, B, 2); } else LAUNCH4(T, LPC, B, 0); } while (0)
#define LAUNCH2(T, LPC) do { if (bonus) LAUNCH3(T, LPC, true); else LAUNCH3(T, LPC, false); } while (0)
#define LAUNCH(T)                                                                                                    \
  switch (lpc) {                                                                                                     \
    case 1: LAUNCH2(T, 1); break;                                                                                    \
    case 2: LAUNCH2(T, 2); break;                                                                                    \
    case 4: LAUNCH2(T, 4); break;                                                                                    \
    case 8: LAUNCH2(T, 8); break;                                                                                    \
    default: LAUNCH2(T, 16); break;                                                                                  \
  }
  if (dtype == MS_F32) { LAUNCH(float) }
  else if (dtype == MS_BF16) { LAUNCH(bf16) }
  else return MS_BAD_ARG;
#undef LAUNCH
#undef LAUNCH2
#undef LAUNCH3
#undef LAUNCH4
  return ms_launch_status();
}

// h [N, width] of `dtype` (rows h_stride apart), mu float [n_mixes, width], state [slots, width] of `dtype`,
// out [n_mixes, N, width] of `dtype`.
extern "C" int ms_token_shift(const void* h, long long h_stride, const float* mu, void* state, const int* token_req,
                              const int* q_start, const int* state_slots, const int* n_live_tokens, void* out,
                              int n_tokens, int n_requests, int width, int n_mixes, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || n_requests <= 0) return MS_OK;
  if (width <= 0 || n_mixes <= 0 || h_stride < width) return MS_BAD_ARG;
  dim3 grid((unsigned)n_tokens, (unsigned)((width + 255) / 256)), block(256);
  dim3 ugrid((unsigned)((width + 255) / 256), (unsigned)n_requests);
#define LAUNCH(T)                                                                                                    \
  token_shift_kernel<T><<<grid, block, 0, stream>>>((const T*)h, (size_t)h_stride, mu, (const T*)state, token_req,  \
                                                    q_start, state_slots, n_live_tokens, (T*)out, n_tokens, width,   \
                                                    n_mixes);                                                        \
  token_shift_update_kernel<T><<<ugrid, block, 0, stream>>>((const T*)h, (size_t)h_stride, (T*)state, q_start,       \
                                                            state_slots, width)
  if (dtype == MS_F32) { LAUNCH(float); }
  else if (dtype == MS_BF16) { LAUNCH(bf16); }
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

// a, b [n_rows, width] of `dtype`; norm_a / norm_b (may be null) float [width]; x float [n_rows, width].
extern "C" int ms_pair_sum(const void* a, const void* b, float scale_a, float scale_b, const float* norm_a,
                           const float* norm_b, float eps, float* x, int n_rows, int width, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (width <= 0) return MS_BAD_ARG;
  if (dtype == MS_F32)
    pair_sum_kernel<float><<<n_rows, 256, 0, stream>>>((const float*)a, (const float*)b, scale_a, scale_b, norm_a, norm_b, eps, x, width);
  else if (dtype == MS_BF16)
    pair_sum_kernel<bf16><<<n_rows, 256, 0, stream>>>((const bf16*)a, (const bf16*)b, scale_a, scale_b, norm_a, norm_b, eps, x, width);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_concat_rows(const float* a, const float* b, void* out, int n_rows, int width_a, int width_b,
                              int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (width_a <= 0 || width_b <= 0) return MS_BAD_ARG;
  if (out_dtype == MS_F32) concat_rows_kernel<float><<<n_rows, 256, 0, stream>>>(a, b, (float*)out, width_a, width_b);
  else if (out_dtype == MS_BF16) concat_rows_kernel<bf16><<<n_rows, 256, 0, stream>>>(a, b, (bf16*)out, width_a, width_b);
  else return MS_BAD_ARG;
  return ms_launch_status();
}
