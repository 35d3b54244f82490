// minGRU: a gated recurrence per channel whose gates read the current token only.
//   z = sigmoid(pz + bz);  u = px + bx;  c = u + 1/2 (u >= 0), sigmoid(u) (u < 0);
//   S_t = (1 - z) S_(t-1) + z c;   out = S_t * silu(pg)
// pz | px | pg are the three thirds of a row of one packed product [N, 3C].  S float [slots, C] is carried from step
// to step in the request's slot.  The gates, the candidate, the gate of the read-out and S are float.
//
// The recurrence is linear in S (S_t = a_t S_(t-1) + b_t), so a portion is walked a chunk of W x TPW tokens at a time by
// the W waves of a block, 64 channels a block: every wave loads its TPW tokens at once, folds them into one pair
// (A, B) with S_out = A S_in + B, the pairs of the waves before it give its S_in, and it then walks its tokens again
// from there.  A step of single tokens runs W = 1.  A portion longer than a chunk is spread over blocks, a chunk each, in two
// launches (fold every chunk; then start every chunk from the chunks before it and walk it), so that one long prompt fills
// the chip instead of channels / 64 blocks.
// A step is a ragged batch: request r owns the tokens q_start[r] .. q_start[r+1]-1 and the slot state_slots[r];
// requests without tokens are left alone.
#include "common.h"
#include "api.h"

namespace {

constexpr int GRU_TPW = 8;     // tokens a wave holds in registers

__device__ __forceinline__ float gru_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

// MODE 0: a block walks its request's whole portion, chunk after chunk.  MODE 1 and 2 spread a long portion's chunks
// over blocks (blockIdx.y: the chunk), in two launches: 1 folds every chunk into one pair (A, B) per channel and leaves
// it, and the state the portion starts from, in `scratch`; 2 gives every chunk its start from the pairs of the chunks
// before it, walks it, and the last chunk's block stores the state.
// scratch: float [R][n_chunks][2][C] pairs, then [R][C] starting states.
template <typename T, int W, int MODE>
__global__ void __launch_bounds__(W * MS_WAVE)
mingru_scan_kernel(const T* __restrict__ zxg, size_t in_stride, const float* __restrict__ bz, const float* __restrict__ bx,
                   float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
                   T* __restrict__ out, size_t out_stride, int C, float* __restrict__ scratch, int n_chunks, int n_requests) {
  __shared__ float sA[W][MS_WAVE], sB[W][MS_WAVE];
  constexpr int CHUNK = W * GRU_TPW;
  const int r = MODE ? blockIdx.z : blockIdx.y;
  const int s0 = q_start[r], L = q_start[r + 1] - s0;
  const int first = MODE ? blockIdx.y * CHUNK : 0;
  if (L <= 0 || first >= L) return;
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int ch = blockIdx.x * MS_WAVE + lane;
  const bool live = ch < C;
  const int chl = live ? ch : 0;
  float* Sg = state + (size_t)state_slots[r] * C + chl;
  float* pairs = MODE ? scratch + ((size_t)r * n_chunks) * 2 * C : nullptr;
  float* init = MODE ? scratch + (size_t)n_requests * n_chunks * 2 * C + (size_t)r * C + chl : nullptr;
  float S_in = 0.f;
  if (MODE == 0) S_in = live ? *Sg : 0.f;
  if (MODE == 1 && first == 0 && wave == 0 && live) *init = *Sg;
  if (MODE == 2) {
    S_in = live ? *init : 0.f;
    for (int c = 0; c < (int)blockIdx.y; ++c) S_in = fmaf(pairs[(size_t)c * 2 * C + chl], S_in, pairs[(size_t)c * 2 * C + C + chl]);
  }
  const float biz = bz ? bz[chl] : 0.f, bix = bx ? bx[chl] : 0.f;
  const int end = MODE ? min(L, first + CHUNK) : L;
  for (int c0 = first; c0 < end; c0 += CHUNK) {
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
      if (MODE == 1) {           // the chunk's own pair, by its first wave
        if (wave == 0 && live) {
          float At = 1.f, Bt = 0.f;
          for (int w2 = 0; w2 < W; ++w2) { Bt = fmaf(sA[w2][lane], Bt, sB[w2][lane]); At *= sA[w2][lane]; }
          pairs[(size_t)blockIdx.y * 2 * C + ch] = At;
          pairs[(size_t)blockIdx.y * 2 * C + C + ch] = Bt;
        }
        return;
      }
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
  if (wave == 0 && live && end == L) *Sg = S_in;
}

}  // namespace

// Tokens a block folds at once in the spread form; scratch floats the spread form needs for portions of up to max_q_len.
extern "C" int ms_mingru_chunk() { return 8 * GRU_TPW; }

// zxg [N, >= 3 C] with row stride in_stride; bz, bx float [C] (may be null); state float [slots, C]; out [N, C].
// max_q_len: the longest portion, or more.  Portions longer than a chunk are spread over blocks when `scratch` (float
// [(n_requests * ceil(max_q_len / chunk) * 2 + n_requests) * C]) is given.
extern "C" int ms_mingru_scan(const void* zxg, long long in_stride, const float* bz, const float* bx, float* state,
                              const int* q_start, const int* state_slots, void* out, long long out_stride,
                              int n_requests, int C, int max_q_len, float* scratch, int dtype, hipStream_t stream) {
  if (n_requests <= 0) return MS_OK;
  if (C <= 0 || in_stride < 3ll * C || out_stride < C || max_q_len <= 0) return MS_BAD_ARG;
  if (n_requests > 65535) return MS_UNSUPPORTED;
  const int chunk = ms_mingru_chunk();
  const int n_chunks = (max_q_len + chunk - 1) / chunk;
  const unsigned cb = (C + MS_WAVE - 1) / MS_WAVE;
#define LAUNCH(T, W, MODE, GRID)                                                                                     \
  mingru_scan_kernel<T, W, MODE><<<GRID, dim3(W * MS_WAVE), 0, stream>>>((const T*)zxg, (size_t)in_stride, bz, bx, state, \
                                                                         q_start, state_slots, (T*)out, (size_t)out_stride, C, \
                                                                         scratch, n_chunks, n_requests)
#define BY_SHAPE(T)                                                                                                  \
  do {                                                                                                               \
    if (scratch != nullptr && n_chunks > 1 && n_chunks <= 65535) {                                                   \
      LAUNCH(T, 8, 1, dim3(cb, n_chunks, n_requests));                                                               \
      LAUNCH(T, 8, 2, dim3(cb, n_chunks, n_requests));                                                               \
    } else if (max_q_len > GRU_TPW) LAUNCH(T, 8, 0, dim3(cb, n_requests));                                           \
    else LAUNCH(T, 1, 0, dim3(cb, n_requests));                                                                      \
  } while (0)
  if (dtype == MS_F32) BY_SHAPE(float);
  else if (dtype == MS_BF16) BY_SHAPE(bf16);
  else return MS_BAD_ARG;
#undef BY_SHAPE
#undef LAUNCH
  return ms_launch_status();
}
