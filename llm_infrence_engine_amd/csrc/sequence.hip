// Kernels of mixers that carry a fixed-size state from token to token instead of reading a cache of keys:
// a short causal convolution over time per channel (with the last taps - 1 inputs as state), the gated delta
// rule with one decay per head and key channel, and the gated RMS norm of its read-out.
// A step is a ragged batch: request r owns the tokens q_start[r] .. q_start[r+1]-1 (a portion of a prompt or
// one decoded token) and the state slot state_slots[r]; requests without tokens and tokens of no request pad a
// captured batch and are left alone.  All recurrences, decays, gates and norms are float in every mode.
#include "common.h"
#include "api.h"

namespace {

constexpr int MAX_TAPS = 8;

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ------------------------------------------------------------------------------------------------
// y[n, c] = act(sum_j w[c, j] * in(t - taps + 1 + j)) (+ x[n, c]), t the token's index within its portion;
// in(i) is the portion's own input for i >= 0 and the state (the taps - 1 inputs before the portion) for i < 0.
// mode 0: the sum; 1: x + the sum; 2: silu of the sum.  `bias` (may be null): one number per channel, added to the sum.
template <typename T>
__global__ void short_conv_kernel(const T* __restrict__ x, size_t x_stride, const float* __restrict__ w,
                                  const float* __restrict__ bias, const T* state, const int* __restrict__ token_req,
                                  const int* __restrict__ q_start, const int* __restrict__ state_slots,
                                  const int* __restrict__ n_live_tokens, T* __restrict__ out, size_t out_stride,
                                  int C, int taps, int mode, T* state_out) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  if (n_live_tokens && n >= *n_live_tokens) return;
  const int r = token_req[n];
  const int s = q_start[r];
  const int t = n - s;
  const T* st = state + (size_t)state_slots[r] * (taps - 1) * C;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int i = t - taps + 1 + j;
    const float v = i >= 0 ? to_float(x[(size_t)(s + i) * x_stride + c]) : to_float(st[(size_t)(taps - 1 + i) * C + c]);
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  if (mode == 1) acc += to_float(x[(size_t)n * x_stride + c]);
  else if (mode == 2) acc = acc * sigmoid_f(acc);
  out[(size_t)n * out_stride + c] = from_float<T>(acc);
  if (state_out) {
    // a step of single tokens: this thread is the only one that reads or writes its request's state of this channel,
    // so it moves the state on itself (one place up, the token's input last) and no second kernel is needed
    T* so = state_out + (size_t)state_slots[r] * (taps - 1) * C;
    T keep[MAX_TAPS];
#pragma unroll
    for (int i = 0; i < MAX_TAPS - 1; ++i)
      if (i < taps - 1) keep[i] = i + 1 < taps - 1 ? so[(size_t)(i + 1) * C + c] : x[(size_t)n * x_stride + c];
#pragma unroll
    for (int i = 0; i < MAX_TAPS - 1; ++i)
      if (i < taps - 1) so[(size_t)i * C + c] = keep[i];
  }
}

// After the convolution: the state of every request with tokens becomes its last taps - 1 inputs.
template <typename T>
__global__ void short_conv_update_kernel(const T* __restrict__ x, size_t x_stride, T* __restrict__ state,
                                         const int* __restrict__ q_start, const int* __restrict__ state_slots,
                                         int C, int taps) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = q_start[r], L = q_start[r + 1] - s;
  if (L <= 0) return;
  T* st = state + (size_t)state_slots[r] * (taps - 1) * C;
  T keep[MAX_TAPS];
  const int hist = taps - 1;
#pragma unroll
  for (int i = 0; i < MAX_TAPS - 1; ++i)
    if (i < hist) {
      const int src = L - hist + i;   // index within the portion; negative: still in the old state
      keep[i] = src >= 0 ? x[(size_t)(s + src) * x_stride + c] : st[(size_t)(src + hist) * C + c];
    }
#pragma unroll
  for (int i = 0; i < MAX_TAPS - 1; ++i)
    if (i < hist) st[(size_t)i * C + c] = keep[i];
}

// Sum over groups of LPC neighbouring lanes (LPC a power of two up to 16, groups aligned), every lane of a group
// getting the sum, by lane permutations inside the vector unit: within a quad lane ^ 1 and lane ^ 2, then the two
// quads of eight lanes mirrored onto each other (all lanes of a quad hold the same value by then).
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int LPC> __device__ __forceinline__ float group_sum(float v) {
  if (LPC >= 2) v += dpp_move<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  if (LPC >= 4) v += dpp_move<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  if (LPC >= 8) v += dpp_move<0x141>(v);    // row_half_mirror: lane i of eight <- lane 7 - i
  if (LPC >= 16) v += dpp_move<0x140>(v);   // row_mirror: lane i of sixteen <- lane 15 - i
  return v;
}

// ------------------------------------------------------------------------------------------------
// The gated delta rule.  Per request and head, S [D, E] float, token by token:
//   S <- g * S (row i by g_i);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// with q, k made unit vectors per head (q also times D^-1/2), beta = sigmoid(b) and
// g = exp(-exp(A_log_h) * softplus(a + dt_bias)).  Column j of S depends on no other column, so a column is
// held in the registers of LPC neighbouring lanes (DPT rows each) for the whole portion.  Tokens are staged a
// chunk at a time: the chunk's q, k (normalised), g, beta and v are worked out by all threads in parallel into
// LDS, then the chunk's tokens are walked in order.  The chunk is as long as LDS allows, up to 16 tokens.
constexpr int DELTA_CHUNK = 16;

// SINGLE: every request of the step has one token (a decode step).  Nothing is asked or fetched ahead then, which
// leaves registers for three blocks to a CU: the step is the read and the write of the states, and needs them in flight.
// SPLIT: the block has twice the threads; the first half walks the tokens of a chunk while the second half stages
// the next chunk into a second set of buffers (its arithmetic, the unit norms and the decays' exponentials, is as long
// as the walk over a chunk and shares nothing with it), so a chunk costs the longer of the two and one barrier.
template <typename T, int DPT, int LPC, bool SINGLE, bool SPLIT>
__global__ void __launch_bounds__(SPLIT ? 512 : 256, SINGLE ? 3 : 1)
gated_delta_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, size_t qkv_stride,
                   const float* __restrict__ a, int decay_per_channel, const T* __restrict__ b, size_t b_stride,
                   const float* __restrict__ A_log, const float* __restrict__ dt_bias, float* __restrict__ state,
                   const int* __restrict__ q_start, const int* __restrict__ state_slots, float* __restrict__ out,
                   int H, int G, int D, int E, int cols_per_block, int chunk) {
  extern __shared__ __align__(16) float lds[];
  constexpr int lpc = LPC;
  constexpr int Dp = DPT * LPC;             // padded key size
  float *qs, *ks, *gs, *vs, *bs;            // [chunk][Dp] three times, [chunk][cols_per_block], [chunk]
  const int buf_floats = (chunk * (3 * Dp + cols_per_block + 1) + 3) / 4 * 4;
  auto use_buffers = [&](int which) __attribute__((always_inline)) {
    qs = lds + (size_t)which * buf_floats;
    ks = qs + chunk * Dp;
    gs = ks + chunk * Dp;
    vs = gs + chunk * Dp;
    bs = vs + chunk * cols_per_block;
  };
  use_buffers(0);
  const int r = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * cols_per_block;
  const int kvh = h / (H / G);
  const int s0 = q_start[r], L = q_start[r + 1] - s0;
  if (L <= 0) return;
  const int nth = SPLIT ? blockDim.x / 2 : blockDim.x;      // threads of a role
  const bool producer = SPLIT && (int)threadIdx.x >= nth;
  const int tid = producer ? threadIdx.x - nth : threadIdx.x;   // the thread's place within its role
  const int part = tid % lpc, col = col0 + tid / lpc;
  const bool live = !producer && col < E && tid / lpc < cols_per_block;
  float* Sg = state + (((size_t)state_slots[r] * H + h) * D) * E;
  float S[DPT];
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = part * DPT + ii;
    S[ii] = (live && i < D) ? Sg[(size_t)i * E + col] : 0.f;
  }
  const float rate = expf(A_log[h]);
  const float q_scale = 1.0f / sqrtf((float)D);

  // Staging.  LT lanes share a token (the host makes the chunk no longer than the block has such groups): a lane
  // asks for all its entries of q, k, the decay's input, and its values of v at once, a chunk ahead, so that one trip
  // to memory serves a whole chunk and is over by the time the chunk before has been walked.
  constexpr int LT = Dp > 256 ? 64 : 16, EPL = (Dp + LT - 1) / LT, VPL = SINGLE ? 1 : 16 / LPC;   // a chunk has at most 16 / LPC values of v a lane   // a whole wave to a token of the longest keys
  const int tl = tid / LT, l16 = tid % LT;
  T qr[EPL], kr[EPL], vr[VPL], br = from_float<T>(0.f);   // as loaded: nothing waits for them before the staging
  float ar[EPL], dr[EPL];
  auto ask = [&](int c0) __attribute__((always_inline)) {
    const int cn = min(chunk, L - c0);
    if (tl < cn) {
      const size_t n = (size_t)(s0 + c0 + tl);
      const T* qp = q + n * qkv_stride + (size_t)kvh * D;
      const T* kp = k + n * qkv_stride + (size_t)kvh * D;
      // the decay's input: one number per head and key channel, or one per head that all its channels share
      const float* ap = decay_per_channel ? a + n * (size_t)H * D + (size_t)h * D : a + n * (size_t)H + h;
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int i = l16 + e * LT;
        const bool in = i < D;
        if (in) {
          qr[e] = qp[i]; kr[e] = kp[i];
          ar[e] = ap[decay_per_channel ? i : 0];
          dr[e] = dt_bias[decay_per_channel ? (size_t)h * D + i : (size_t)h];
        }
      }
      if (l16 == 0) br = b[n * b_stride + h];
    }
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e = tid + j * nth;
      if (e < cn * cols_per_block) {
        const int t = e / cols_per_block, jj = e - t * cols_per_block;
        if (col0 + jj < E) vr[j] = v[(size_t)(s0 + c0 + t) * qkv_stride + (size_t)h * E + col0 + jj];
      }
    }
  };
  constexpr bool ASK_AHEAD = DPT <= 32 && !SINGLE;   // the longest columns leave no registers to hold a chunk through the walk
  auto stage = [&](int c0) __attribute__((always_inline)) {
    const int cn = min(chunk, L - c0);
    if (tl < cn) {
      float sq = 0.f, sk = 0.f, qf[EPL], kf[EPL], af[EPL];
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const bool in = l16 + e * LT < D;
        qf[e] = in ? to_float(qr[e]) : 0.f;
        kf[e] = in ? to_float(kr[e]) : 0.f;
        af[e] = in ? ar[e] + dr[e] : 0.f;
        sq = fmaf(qf[e], qf[e], sq);
        sk = fmaf(kf[e], kf[e], sk);
      }
      sq = LT == 64 ? wave_sum(sq) : group_sum<16>(sq);
      sk = LT == 64 ? wave_sum(sk) : group_sum<16>(sk);
      const float iq = q_scale / sqrtf(sq + 1e-6f), ik = 1.0f / sqrtf(sk + 1e-6f);
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int i = l16 + e * LT;
        if (i < Dp) {
          const bool in = i < D;
          qs[tl * Dp + i] = qf[e] * iq;
          ks[tl * Dp + i] = kf[e] * ik;
          gs[tl * Dp + i] = in ? expf(-rate * softplus_f(af[e])) : 1.f;
        }
      }
      if (l16 == 0) bs[tl] = sigmoid_f(to_float(br));
    }
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e = tid + j * nth;
      if (e < cn * cols_per_block) {
        const int t = e / cols_per_block, jj = e - t * cols_per_block;
        vs[e] = col0 + jj < E ? to_float(vr[j]) : 0.f;
      }
    }
  };
  auto walk = [&](int c0) __attribute__((always_inline)) {
    const int cn = min(chunk, L - c0);
    // the rows of the next token's q, k and g are fetched from LDS while the current token is worked on (two sets of
    // registers taken in turn, so that nothing is copied); the two sums over a column run as four chains each
    struct Rows { float g[DPT], k[DPT], q[DPT]; };
    auto fetch = [&](Rows& r, int t) __attribute__((always_inline)) {
      const float* qt = qs + t * Dp + part * DPT;
      const float* kt = ks + t * Dp + part * DPT;
      const float* gt = gs + t * Dp + part * DPT;
#pragma unroll
      for (int ii = 0; ii < DPT; ii += 4) {
        const float4 g4 = *reinterpret_cast<const float4*>(gt + ii);
        const float4 k4 = *reinterpret_cast<const float4*>(kt + ii);
        const float4 q4 = *reinterpret_cast<const float4*>(qt + ii);
        r.g[ii] = g4.x; r.g[ii + 1] = g4.y; r.g[ii + 2] = g4.z; r.g[ii + 3] = g4.w;
        r.k[ii] = k4.x; r.k[ii + 1] = k4.y; r.k[ii + 2] = k4.z; r.k[ii + 3] = k4.w;
        r.q[ii] = q4.x; r.q[ii + 1] = q4.y; r.q[ii + 2] = q4.z; r.q[ii + 3] = q4.w;
      }
    };
    auto token = [&](const Rows& r, int t, float beta_t, float v_t) __attribute__((always_inline)) {
      float kv4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DPT; ii += 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          S[ii + j] *= r.g[ii + j];
          kv4[j] = fmaf(S[ii + j], r.k[ii + j], kv4[j]);
        }
      }
      const float kv = group_sum<LPC>((kv4[0] + kv4[1]) + (kv4[2] + kv4[3]));
      const float u = beta_t * (v_t - kv);
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DPT; ii += 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          S[ii + j] = fmaf(r.k[ii + j], u, S[ii + j]);
          o4[j] = fmaf(S[ii + j], r.q[ii + j], o4[j]);
        }
      }
      const float o_sum = group_sum<LPC>((o4[0] + o4[1]) + (o4[2] + o4[3]));
      if (live && part == 0) out[((size_t)(s0 + c0 + t) * H + h) * E + col] = o_sum;
    };
    constexpr bool AHEAD = DPT <= 32 && !SINGLE;    // the longest columns leave no registers for a second set of rows
    const int my_col = tid / lpc;
    if (AHEAD) {
      Rows ra, rb;
      fetch(ra, 0);
      for (int t = 0; t < cn; t += 2) {
        const float b0 = bs[t], v0 = vs[t * cols_per_block + my_col];
        const bool two = t + 1 < cn;
        if (two) fetch(rb, t + 1);
        token(ra, t, b0, v0);
        if (two) {
          const float b1 = bs[t + 1], v1 = vs[(t + 1) * cols_per_block + my_col];
          if (t + 2 < cn) fetch(ra, t + 2);
          token(rb, t + 1, b1, v1);
        }
      }
    } else {
      Rows ra;
      for (int t = 0; t < cn; ++t) {
        fetch(ra, t);
        token(ra, t, bs[t], vs[t * cols_per_block + my_col]);
      }
    }
  };
  if (SPLIT) {
    if (producer) {
      ask(0);
      stage(0);
      if (chunk < L) ask(chunk);
    }
    __syncthreads();
    int which = 0;
    for (int c0 = 0; c0 < L; c0 += chunk, which ^= 1) {
      if (producer) {
        if (c0 + chunk < L) {      // the walkers read the other set; the set written here was last read a barrier ago
          use_buffers(which ^ 1);
          stage(c0 + chunk);
          if (c0 + 2 * chunk < L) ask(c0 + 2 * chunk);
        }
      } else {
        use_buffers(which);
        walk(c0);
      }
      __syncthreads();
    }
  } else {
    if (ASK_AHEAD) ask(0);
    for (int c0 = 0; c0 < L; c0 += chunk) {
      if (!ASK_AHEAD) ask(c0);
      __syncthreads();   // the chunk before is done with the staging area
      stage(c0);
      __syncthreads();
      if (ASK_AHEAD && c0 + chunk < L) ask(c0 + chunk);
      walk(c0);
    }
  }
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = part * DPT + ii;
    if (live && i < D) Sg[(size_t)i * E + col] = S[ii];
  }
}

// ------------------------------------------------------------------------------------------------
// y[n, h, :] = o[n, h, :] / sqrt(mean(o[n, h, :]^2) + eps) * w[:] * act(gate[n, h, :]), act the sigmoid (gate_silu 0) or
// z * sigmoid(z) (1); one wave per (token, head).
template <typename T>
__global__ void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                       const T* __restrict__ gate, size_t gate_stride, T* __restrict__ out,
                                       long long items, int H, int E, float eps, int gate_silu, int weight_per_head,
                                       float scale) {
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const long long item = (long long)blockIdx.x * (blockDim.x / MS_WAVE) + threadIdx.x / MS_WAVE;
  if (item >= items) return;
  const long long n = item / H;
  const int h = (int)(item - n * H);
  const float* op = o + (size_t)item * E;
  float ss = 0.f;
  for (int i = lane; i < E; i += MS_WAVE) ss = fmaf(op[i], op[i], ss);
  ss = wave_sum(ss);
  const float inv = scale / sqrtf(ss / (float)E + eps);
  if (weight_per_head) w += (size_t)h * E;
  const T* gp = gate + (size_t)n * gate_stride + (size_t)h * E;
  T* yp = out + (size_t)item * E;
  for (int i = lane; i < E; i += MS_WAVE) {
    const float z = to_float(gp[i]);
    yp[i] = from_float<T>(op[i] * inv * w[i] * (gate_silu ? z * sigmoid_f(z) : sigmoid_f(z)));
  }
}

// ------------------------------------------------------------------------------------------------
// The xIELU activation with its two learned numbers (p, q):  z > 0: softplus(p) z^2 + z/2;
// z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2.
template <typename T>
__global__ void xielu_kernel(const T* __restrict__ x, const float* __restrict__ pq, T* __restrict__ out, size_t total) {
  const float ap = softplus_f(pq[0]), an = 0.5f + softplus_f(pq[1]);
  constexpr int V = 16 / sizeof(T);     // values in 16 bytes
  struct alignas(16) Pack { T v[V]; };
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t packs = (((size_t)x | (size_t)out) & 15) == 0 ? total / V : 0;   // 16 bytes a lane where both are aligned
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < packs; i += stride) {
    Pack p = reinterpret_cast<const Pack*>(x)[i];
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float z = to_float(p.v[j]);
      p.v[j] = from_float<T>(z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(an, expm1f(z) - z, 0.5f * z));
    }
    reinterpret_cast<Pack*>(out)[i] = p;
  }
  for (size_t i = packs * V + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const float z = to_float(x[i]);
    out[i] = from_float<T>(z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(an, expm1f(z) - z, 0.5f * z));
  }
}

}  // namespace

extern "C" int ms_short_conv(const void* x, long long x_stride, const float* w, const float* bias, void* state,
                             const int* token_req,
                             const int* q_start, const int* state_slots, const int* n_live_tokens, void* out,
                             long long out_stride, int n_tokens, int n_requests, int channels, int taps, int mode,
                             int update_state, int single_tokens, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (channels <= 0 || taps < 1 || mode < 0 || mode > 2 || n_requests <= 0) return MS_BAD_ARG;
  if (taps > MAX_TAPS) return MS_UNSUPPORTED;
  const int threads = channels >= 256 ? 256 : 64;
  const int cblocks = (channels + threads - 1) / threads;
  if (cblocks > 65535 || n_requests > 65535) return MS_UNSUPPORTED;
  dim3 block(threads), grid(n_tokens, cblocks), ugrid(cblocks, n_requests);
#define LAUNCH(T)                                                                                                       \
  do {                                                                                                                  \
    const bool fused = update_state && single_tokens && taps > 1;                                                       \
    short_conv_kernel<T><<<grid, block, 0, stream>>>((const T*)x, (size_t)x_stride, w, bias, (const T*)state, token_req, \
                                                     q_start, state_slots, n_live_tokens, (T*)out, (size_t)out_stride, \
                                                     channels, taps, mode, fused ? (T*)state : nullptr);               \
    if (update_state && taps > 1 && !fused)                                                                             \
      short_conv_update_kernel<T><<<ugrid, block, 0, stream>>>((const T*)x, (size_t)x_stride, (T*)state, q_start,      \
                                                               state_slots, channels, taps);                            \
  } while (0)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

extern "C" int ms_gated_delta(const void* q, const void* k, const void* v, long long qkv_stride, const float* a,
                              int decay_per_channel, const void* b, long long b_stride, const float* A_log, const float* dt_bias,
                              float* state, const int* q_start, const int* state_slots, float* out, int n_requests,
                              int heads, int kv_heads, int dim, int vdim, int single_tokens, int dtype,
                              hipStream_t stream) {
  if (n_requests <= 0) return MS_OK;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0) return MS_BAD_ARG;
  if (dim > 512 || n_requests > 65535 || heads > 65535) return MS_UNSUPPORTED;
  // lanes a column of the state is spread over (lpc) and rows each of them holds (dpt): sixteen rows a lane where the
  // key size allows, so that a token costs a lane few dependent operations and a head's columns spread over many waves
  int lpc, dpt;
  if (dim <= 8) { lpc = 1; dpt = 8; }
  else if (dim <= 16) { lpc = 1; dpt = 16; }
  else if (dim <= 32) { lpc = 2; dpt = 16; }
  else if (dim <= 64) { lpc = 4; dpt = 16; }
  else if (dim <= 128) { lpc = 8; dpt = 16; }
  else if (dim <= 256) { lpc = 8; dpt = 32; }
  else { lpc = 8; dpt = 64; }
  int threads = vdim * lpc;
  threads = threads >= 256 ? 256 : ((threads + MS_WAVE - 1) / MS_WAVE) * MS_WAVE;
  const int cols = threads / lpc;
  dim3 grid((vdim + cols - 1) / cols, heads, n_requests), block(threads);
  const int stagers = dpt * lpc > 256 ? 64 : 16;    // lanes that stage a token
  int chunk = DELTA_CHUNK < threads / stagers ? DELTA_CHUNK : threads / stagers;
  const size_t per_token = (3 * (size_t)dpt * lpc + cols + 1) * sizeof(float);
  while (chunk > 1 && chunk * per_token > 65536) chunk /= 2;
  const size_t lds = ((chunk * per_token / sizeof(float) + 3) / 4 * 4) * sizeof(float);   // one set of buffers
  if (lds > 65536) return MS_UNSUPPORTED;
#define LAUNCH1(T, DPT, LPC, ONE, TWO)                                                                                  \
  gated_delta_kernel<T, DPT, LPC, ONE, TWO><<<grid, dim3(threads * ((TWO) ? 2 : 1)), lds * ((TWO) ? 2 : 1), stream>>>(  \
      (const T*)q, (const T*)k, (const T*)v, (size_t)qkv_stride, a, decay_per_channel, (const T*)b, (size_t)b_stride,  \
      A_log, dt_bias,                                                                                                   \
      state, q_start, state_slots, out, heads, kv_heads, dim, vdim, cols, chunk)
#define LAUNCH(T, DPT, LPC)                                                                                             \
  do {                                                                                                                  \
    if (single_tokens && DPT <= 16) LAUNCH1(T, DPT, LPC, (DPT <= 16), false);                                           \
    else if (DPT <= 16 && 2 * lds <= 65536) LAUNCH1(T, DPT, LPC, false, (DPT <= 16));                                   \
    else LAUNCH1(T, DPT, LPC, false, false);                                                                            \
  } while (0)
#define BY_DPT(T)                                                                                                       \
  do {                                                                                                                  \
    if (dpt == 8) LAUNCH(T, 8, 1);                                                                                      \
    else if (dpt == 16 && lpc == 1) LAUNCH(T, 16, 1);                                                                   \
    else if (dpt == 16 && lpc == 2) LAUNCH(T, 16, 2);                                                                   \
    else if (dpt == 16 && lpc == 4) LAUNCH(T, 16, 4);                                                                   \
    else if (dpt == 16) LAUNCH(T, 16, 8);                                                                               \
    else if (dpt == 32) LAUNCH(T, 32, 8);                                                                               \
    else LAUNCH(T, 64, 8);                                                                                              \
  } while (0)
  if (dtype == MS_F32) BY_DPT(float);
  else if (dtype == MS_BF16) BY_DPT(bf16);
  else return MS_BAD_ARG;
#undef BY_DPT
#undef LAUNCH
#undef LAUNCH1
  return ms_launch_status();
}

extern "C" int ms_gated_head_norm(const float* o, const float* weight, const void* gate, long long gate_stride,
                                  void* out, int n_tokens, int heads, int vdim, float eps, int gate_silu,
                                  int weight_per_head, float scale, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (heads <= 0 || vdim <= 0) return MS_BAD_ARG;
  const long long items = (long long)n_tokens * heads;
  const int waves = 4;
  dim3 grid((unsigned)((items + waves - 1) / waves)), block(waves * MS_WAVE);
  if (dtype == MS_F32)
    gated_head_norm_kernel<float><<<grid, block, 0, stream>>>(o, weight, (const float*)gate, (size_t)gate_stride,
                                                              (float*)out, items, heads, vdim, eps, gate_silu,
                                                              weight_per_head, scale);
  else if (dtype == MS_BF16)
    gated_head_norm_kernel<bf16><<<grid, block, 0, stream>>>(o, weight, (const bf16*)gate, (size_t)gate_stride,
                                                             (bf16*)out, items, heads, vdim, eps, gate_silu,
                                                             weight_per_head, scale);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_xielu(const void* x, const float* pq, void* out, long long total, int dtype, hipStream_t stream) {
  if (total <= 0) return MS_OK;
  int blocks = (int)((total / 4 + 255) / 256) + 1;
  if (blocks > 8192) blocks = 8192;
  if (dtype == MS_F32) xielu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, pq, (float*)out, (size_t)total);
  else if (dtype == MS_BF16) xielu_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)x, pq, (bf16*)out, (size_t)total);
  else return MS_BAD_ARG;
  return ms_launch_status();
}
