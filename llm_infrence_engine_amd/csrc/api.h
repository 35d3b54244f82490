// C entry points of the gfx950 kernel library.  Every function enqueues work on `stream` and returns
// 0, or a non-zero code (see common.h) without launching when it refuses its arguments.  Pointers are
// device pointers; matrices are row-major.  `dtype` is 0 for float and 1 for bfloat16.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

int ms_embed(const int* ids, const void* table, float* out, int n_tokens, int hidden, float scale, int dtype,
             hipStream_t stream);

int ms_rms_norm(float* x, const void* delta, int delta_dtype, int n_partials, long long partial_stride,
                const float* weight, const int* rows, void* out, int n_rows, int hidden, float eps, int write_back,
                int dtype, hipStream_t stream);

// the same rows normalised once and scaled twice: out1 = w1 * n(x (+ delta)), out2 = w2 * n(x (+ delta)); the sum is kept in x
int ms_rms_norm_pair(float* x, const void* delta, int delta_dtype, const float* w1, const float* w2, void* out1, void* out2,
                     int n_rows, int hidden, float eps, int dtype, hipStream_t stream);

int ms_bias_add(void* x, const float* bias, int n_rows, int width, int dtype, hipStream_t stream);

// tables / slots: host arrays of n_groups device pointers (block table int32 [table rows, table_stride], slot
// mapping int32 [n_rows]); table_rows int32 [n_rows]: the table's row of each row of the batch; draw_index int32
// [n_rows] (may be null): counted up by one for every live row.  At most ms_max_cache_groups() groups.
int ms_max_cache_groups();
int ms_decode_advance(const int* prev_tokens, int* token_ids, int* positions, int* context_lens, const int* n_live,
                      const int* table_rows, int* draw_index, const int* const* tables, int* const* slots,
                      const int* strides, int n_groups, int table_stride, int page_size, int n_rows, hipStream_t stream);

// Block tables kept on the device: tables[g][index[g][i]] = value[g][i] for i < counts[g] (counts: device ints),
// every index at most once per group; max_updates bounds counts, table_elems bounds the indices.
int ms_table_update(int* const* tables, const int* const* index, const int* const* value, const int* counts,
                    int n_groups, int max_updates, long long table_elems, hipStream_t stream);

// rows[i] of a [n, row_bytes] tensor become zero (row_bytes a multiple of 4), i < n_rows; `count` (null: n_rows)
// is a device int that may ask for fewer.
int ms_zero_rows(void* base, long long row_bytes, const int* rows, const int* count, int n_rows, hipStream_t stream);

// A plain streaming read of `bytes` for bandwidth measurements; sink: unsigned [ms_read_probe_blocks()].
int ms_read_probe_blocks();
int ms_read_probe(const void* base, long long bytes, unsigned* sink, hipStream_t stream);

int ms_residual_add(float* x, const void* delta, long long total, int dtype, hipStream_t stream);

int ms_silu_mul(const void* gate_up, void* out, int n_tokens, int intermediate, int dtype, hipStream_t stream);

int ms_rope_store(void* qkv, const float* bias, const int* positions, const float* inv_freq, const int* slot_mapping, void* k_pages,
                  void* v_pages, int n_tokens, int num_heads, int num_kv_heads, int head_dim, int rot_dim,
                  int page_size, int v_transposed, int dtype, hipStream_t stream);

// table float [n_tokens, half, 2] = (cos, sin) of float(positions[n]) * inv_freq[j]
int ms_rope_table(const int* positions, const float* inv_freq, float* table, int n_tokens, int half, hipStream_t stream);

int ms_gemm_generic(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, long long lda,
                    long long ldw, long long ldc, int in_dtype, int out_dtype, int accumulate, hipStream_t stream);

int ms_gemm_skinny(const void* A, long long lda, const void* W, long long ldw, const float* bias, void* out,
                   long long ldo, int M, int N, int K, int epilogue, int out_dtype, hipStream_t stream);

void ms_gemm_skinny_force(int ntile, int waves, int token_groups);
void ms_attention_mfma_force(int nt, int waves, int dim_shares);

int ms_gemm_stream(const void* A, long long lda, const int* rows, const float* norm_w, float eps, const void* W,
                   long long ldw, const float* bias, void* out, long long ldo, int M, int N, int K, int epilogue,
                   int out_dtype, int norm, int any_shape, hipStream_t stream);

int ms_gemm_panel(const void* A, long long lda, const int* rows, const float* norm_w, float eps, const void* W,
                   long long ldw, const float* bias, void* out, long long ldo, int M, int N, int K, int epilogue,
                   int out_dtype, int norm, int any_shape, hipStream_t stream);

int ms_gemm_panel_splitk_parts(int M, int N, int K);
int ms_gemm_panel_splitk(const void* A, long long lda, const void* W, long long ldw, const float* bias, void* out,
                         long long ldo, int M, int N, int K, int epilogue, int out_dtype, void* partial, int parts,
                         hipStream_t stream);

// Many rows (prompt portions): the tiled matrix-core product, bfloat16 in and out, with the gated activation
// as epilogue 1; K a multiple of 64 (ms_gemm_tiled_force: measurements, 0 leaves the choice of tile, 1 to 5 force one;
// ms_gemm_tiled_pays: whether the gated product is faster here than as library product and activation kernel).
int ms_gemm_tiled(const void* A, long long lda, const void* W, long long ldw, void* out, long long ldo, int M, int N,
                  int K, int epilogue, hipStream_t stream);
void ms_gemm_tiled_force(int tile);
void ms_gemm_tiled_force_xcd_split(int xm);   // measurements: rows of XCDs over the tiles (1, 2, 4, 8); 0 leaves the choice
int ms_gemm_tiled_pays(int M, int N, int K);
int ms_gemm_tiled_plain_pays(int M, int N, int K);   // the same question for a plain product (epilogue 0)

// The q/k/v product of many tokens with bias, rotation (whole heads, pairs (j, j + d/2)) and the store of k and v
// into the cache pages as its epilogue: A [M, lda] bfloat16, W [(nh + 2 nkv) d, ldw], q_out [M, nh d] bfloat16;
// head_dim 64 or 128; rope_table float [M, d / 2, 2] from ms_rope_table.  Pages as in ms_rope_store.  ms_gemm_tiled_qkv_pays: where it beats product + rotation kernel.
int ms_gemm_tiled_qkv(const void* A, long long lda, const void* W, long long ldw, const float* bias,
                      const float* rope_table, const int* slot_mapping, void* q_out, void* k_pages, void* v_pages, int M,
                      int K, int nh, int nkv, int head_dim, int page_size, int v_transposed, hipStream_t stream);
int ms_gemm_tiled_qkv_pays(int M, int N, int K, int head_dim);

int ms_gemm_skinny_norm(const float* x, long long ldx, const int* rows, const float* norm_w, float eps, const void* W,
                        long long ldw, const float* bias, void* out, long long ldo, int M, int N, int K, int epilogue,
                        int out_dtype, hipStream_t stream);

void ms_qkv_rope_store_force(int pair8);

int ms_qkv_rope_store(const float* x, long long ldx, const float* norm_w, float eps, const void* W, const float* bias,
                      const int* positions, const float* inv_freq, const int* slot_mapping, void* q_out,
                      void* k_pages, void* v_pages, int M, int K, int num_heads, int num_kv_heads, int head_dim,
                      int page_size, int v_transposed, hipStream_t stream);

int ms_paged_attention_generic(const void* q, long long q_stride, const void* k_pages, const void* v_pages,
                               const int* block_table, int table_stride, const int* table_rows,
                               const int* n_live_tokens, const int* token_req, const int* positions,
                               void* out, long long out_stride, int n_tokens, int num_heads, int num_kv_heads,
                               int head_dim, int value_dim, int page_size, long long num_pages, float scale, int window,
                               int v_transposed, const float* sink, float softcap, const float* slopes, const void* gate,
                               long long gate_stride, float out_scale, int dtype, hipStream_t stream);

int ms_attention_mfma_supported(int head_dim, int page_size);

int ms_paged_attention_mfma(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                            const int* block_table, int table_stride, const int* table_rows, const int* q_start,
                            const int* context_lens, void* out, long long out_stride, int n_requests, int n_tokens,
                            int max_q_len, int num_heads, int num_kv_heads, int head_dim, int page_size, float scale,
                            int window, const float* sink, float softcap, const float* slopes, const void* gate,
                            long long gate_stride, float out_scale, hipStream_t stream);

int ms_paged_attention_mfma_decode(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                                   const int* block_table, int table_stride, const int* table_rows,
                                   const int* q_start, const int* context_lens, void* out, long long out_stride,
                                   void* part_o,
                                   void* part_ml, int n_requests, int num_heads, int num_kv_heads, int head_dim,
                                   int page_size, float scale, int window, int min_blocks, int n_splits,
                                   const float* sink, float softcap, const float* slopes, const void* gate,
                                   long long gate_stride, float out_scale, hipStream_t stream);

int ms_argmax(const float* logits, long long ld, int n_rows, int vocab, float* scratch_val, int* scratch_idx,
              int n_chunks, int* out, hipStream_t stream);

// The one entry point that allocates nothing.  It has no counterpart in the reference; it is for callers that
// cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  Same result as ms_argmax, but the stage-1 results live in a static device array of the library
// (256 KB on every GPU the library runs on, held until the process ends) instead of scratch_val / scratch_idx.
// The caller still passes logits and out; `stream` must belong to the current device.  Limits: n_rows <= 256
// and n_chunks <= 128 (ms_argmax_static_limits reports them); beyond them the call returns MS_UNSUPPORTED (2)
// and launches nothing.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (different
// streams or threads) race; calls on one stream, or ordered by events, do not.  Nothing in the array needs
// clearing between calls.  The array's address is looked up once per device, at the first call there or by
// ms_argmax_static_init() with that device current (call it before a stream capture starts).
int ms_argmax_static_init();
void ms_argmax_static_limits(int* max_rows, int* max_chunks);
int ms_argmax_static(const float* logits, long long ld, int n_rows, int vocab, int n_chunks, int* out,
                     hipStream_t stream);

// workspace: ms_sample_workspace_bytes(n_rows) bytes of device memory (any contents); use_top_k / use_top_p: 0 if
// no row has a top_k in (0, vocab) / a top_p below 1.
long long ms_sample_workspace_bytes(int n_rows);
int ms_sample(const float* logits, long long ld, int n_rows, int vocab, const float* temperature, const int* top_k,
              const float* top_p, const unsigned long long* seeds, const int* draw_index, int* out, void* workspace,
              int use_top_k, int use_top_p, hipStream_t stream);

// ---- mixers with a fixed-size state (csrc/sequence.hip).  A step's requests: tokens q_start[r]..q_start[r+1]-1, state
// slot state_slots[r]; token_req [n_tokens]; n_live_tokens (may be null): tokens from there on belong to no request.
// Short causal convolution per channel: w float [channels, taps] (last column: the current token), bias float [channels]
// or null, state
// [slots, taps - 1, channels] in `dtype`.  mode 0: the sum, 1: x + the sum, 2: silu(the sum).  out must not be x.
// With update_state the state becomes the last taps - 1 inputs of every request that has tokens (single_tokens: the
// caller knows that no request has more than one token, and the same kernel moves the state on).
int ms_short_conv(const void* x, long long x_stride, const float* w, const float* bias, void* state, const int* token_req,
                  const int* q_start, const int* state_slots, const int* n_live_tokens, void* out, long long out_stride,
                  int n_tokens, int n_requests, int channels, int taps, int mode, int update_state, int single_tokens,
                  int dtype, hipStream_t stream);

// Gated delta rule.  q, k [n, kv_heads * dim], v [n, heads * vdim], b [n, heads] in `dtype` (rows qkv_stride / b_stride
// apart); a: the decay's input before dt_bias, float [n, heads * dim] with dt_bias [heads * dim] (decay_per_channel: one
// decay per head and key channel) or float [n, heads] with dt_bias [heads] (one decay per head);
// state float [slots, heads, dim, vdim]; out float [n, heads * vdim].  single_tokens: the caller knows that no request
// has more than one token (a decode step).
int ms_gated_delta(const void* q, const void* k, const void* v, long long qkv_stride, const float* a,
                   int decay_per_channel, const void* b, long long b_stride, const float* A_log, const float* dt_bias, float* state, const int* q_start,
                   const int* state_slots, float* out, int n_requests, int heads, int kv_heads, int dim, int vdim,
                   int single_tokens, int dtype, hipStream_t stream);

// out[n, h, :] = o[n, h, :] / rms(o[n, h, :]) * weight * act(gate[n, h, :]), act the sigmoid or (gate_silu) z * sigmoid(z);
// o float, gate and out in `dtype`.  weight [vdim], shared by the heads, or with weight_per_head [heads * vdim]; `scale`
// multiplies every result.
int ms_gated_head_norm(const float* o, const float* weight, const void* gate, long long gate_stride, void* out,
                       int n_tokens, int heads, int vdim, float eps, int gate_silu, int weight_per_head, float scale,
                       int dtype, hipStream_t stream);

// xIELU with pq = (p, q) on the device.
int ms_xielu(const void* x, const float* pq, void* out, long long total, int dtype, hipStream_t stream);

// ---- attention through a latent (csrc/latent_attention.hip); strides in elements
int ms_head_matmul(const void* in, long long in_tok, long long in_head, const void* M, void* out, long long out_tok,
                   long long out_head, const void* gate, long long gate_tok, int n_tokens, int heads, int I, int J,
                   int dtype, int out_dtype, hipStream_t stream);
int ms_rms_norm_rows(const void* in, long long in_stride, const float* weight, void* out, long long out_stride, int n_rows,
                     int width, float eps, int dtype, hipStream_t stream);
int ms_rotary_pairs(const void* src, long long src_tok, long long src_head, void* dst, long long dst_tok,
                    long long dst_head, const int* positions, const float* inv_freq, int n_tokens, int heads, int width,
                    int dims, int dtype, hipStream_t stream);
int ms_latent_kv_store(const void* kv, long long kv_stride, const float* norm_w, float eps, const int* positions,
                       const float* inv_freq, const int* slots, void* c_pages, void* r_pages, void* ct_pages, int page_size,
                       int n_tokens, int C, int R, int dims, int dtype, hipStream_t stream);
int ms_latent_attention(const void* q, long long q_tok, long long q_head, const void* c_pages, const void* r_pages,
                        const int* block_table, int table_stride, const int* table_rows, const int* n_live_tokens,
                        const int* token_req, const int* positions, const float* sink, void* out, long long out_tok,
                        long long out_head, int n_tokens, int heads, int C, int R, int page_size, long long num_pages,
                        float scale, int window, int dtype, hipStream_t stream);

// the same on the matrix cores (csrc/latent_attention_mfma.hip): bfloat16, sizes ms_latent_attention_mfma_supported says
int ms_latent_attention_mfma_supported(int C, int R, int page_size);
int ms_latent_attention_mfma(const void* q, long long q_tok, long long q_head, const void* c_pages, const void* r_pages,
                             const void* ct_pages, const int* block_table, int table_stride, const int* table_rows,
                             const int* q_start, const int* context_lens, const float* sink, void* out, long long out_tok,
                             long long out_head, int n_requests, int max_q_len, int heads, int C, int R, int page_size,
                             long long num_pages, float scale, int window, hipStream_t stream);

// ---- layers that normalise a sublayer's output before it joins the residual stream (csrc/residual_norm.hip)
// x += w_post * rms_norm(y); then, if out is not null, out = w_next * rms_norm(x).  y [n, hidden] in y_dtype (rows y_stride
// apart), x float [n, hidden], out in out_dtype.
int ms_rms_norm_add(const void* y, long long y_stride, int y_dtype, const float* w_post, float eps_post, float* x,
                    const float* w_next, float eps_next, void* out, int out_dtype, int n_rows, int hidden,
                    hipStream_t stream);
// x[n, :] += kept[n, :] (if not null) + vec[:] (if not null)
int ms_add_rows(float* x, const float* kept, const float* vec, int n_rows, int hidden, hipStream_t stream);

// ---- heads normalised instead of rotated (csrc/qk_norm.hip): RMS norm of every q and k head with q_weight / k_weight
// [head_dim] (null: no norm), q times 1 + coef * ln(floor((p + 1) / every) + 1) (coef 0: none), k and v stored into pages
// (null: not stored); qkv [n, nh * head_dim + nkv * head_dim + nkv * value_dim].  unit_norm: the norm also without weights;
// rot_dim > 0: after the norm, entry i and entry i + rot_dim / 2 of every q and k head turn by position * inv_freq[i]
int ms_qk_norm_store(void* qkv, long long stride, const float* q_weight, const float* k_weight, float eps,
                     const int* positions, float coef, int every, const int* slots, void* k_pages, void* v_pages,
                     int n_tokens, int num_heads, int num_kv_heads, int head_dim, int value_dim, int page_size,
                     int v_transposed, int unit_norm, const float* inv_freq, int rot_dim, int dtype, hipStream_t stream);

// ---- the selective scan of a state-space mixer (csrc/scan.hip)
int ms_selective_scan(const void* x, long long x_stride, const float* dt_in, const float* dt_bias, const float* A,
                      const void* B, const void* C, long long bc_stride, const float* D, const void* z, long long z_stride,
                      float* state, const int* q_start, const int* state_slots, void* out, long long out_stride,
                      int n_requests, int channels, int states, int dtype, hipStream_t stream);

// ---- routed experts (csrc/experts.hip)
int ms_gelu(const void* x, void* out, long long total, int dtype, hipStream_t stream);
// softmax over logits[n, :n_out] (rows ld apart; sigmoid_scores: each logit's own sigmoid instead), the `top` largest of
// score + correction: ids / weights [n, top]
int ms_moe_route(const float* logits, long long ld, const float* correction, int n_tokens, int n_out, int top, int* ids,
                 float* weights, int sigmoid_scores, hipStream_t stream);
int ms_moe_tile_rows();
int ms_moe_wide_tile_rows();
// rows [tiles * tile] and tile_expert [tiles] from ids [n_items]; ids >= n_experts take no row; tile: ms_moe_tile_rows()
// or, for the matrix-core products alone, ms_moe_wide_tile_rows() or ms_gemm_tiled_grouped_rows()
int ms_moe_align(const int* ids, int n_items, int n_experts, int tile, int tiles, int* rows, int* tile_expert,
                 hipStream_t stream);
// the same product for tiles of ms_gemm_tiled_grouped_rows() rows, or half as many, on the tiled kernel
// (csrc/gemm_tiled.hip): K a multiple of 64
int ms_gemm_tiled_grouped_rows();
int ms_gemm_tiled_grouped(const void* A, long long lda, const void* W, const int* rows, const int* tile_expert, void* out,
                          long long ldo, int tiles, int tile_rows, int N, int K, int in_div, int out_scatter, int act,
                          int out_dtype, hipStream_t stream);

int ms_grouped_gemm_mfma_ok(int K, long long in_stride, long long out_stride, int tile, int dtype, int out_dtype);
// for every tile t with an expert e and each of its rows i (flat position p = t * tile + i, item = rows[p] >= 0):
// out[out_scatter ? item : p] = act(w[e] . in[in_div ? item / in_div : p]); w [experts, n_out, K]
int ms_grouped_gemm(const void* in, long long in_stride, const void* w, const int* rows, const int* tile_expert, void* out,
                    long long out_stride, int tiles, int tile, int n_out, int K, int in_div, int out_scatter, int act,
                    int dtype, int out_dtype, hipStream_t stream);
int ms_moe_combine(const float* part, const int* ids, const float* weights, const void* h, long long h_stride,
                   const void* shared, int shared_dtype, const float* gate, long long gate_stride, float* out,
                   int n_tokens, int top, int n_experts, int hidden, int dtype, hipStream_t stream);   // weights null: all 1

// ---- layer norm and the gate of a token's side input (csrc/layer_norm.hip)
int ms_layer_norm(float* x, const void* delta, int delta_dtype, const float* dscale, const float* w, const float* b, const int* rows,
                  void* out, int n_rows, int H, float eps, int write_back, int out_dtype, hipStream_t stream);
int ms_side_gate(const void* z, long long z_stride, const int* token_ids, const void* table, long long table_stride, int part,
                 void* out, int n_tokens, int d, int dtype, hipStream_t stream);
// ---- minGRU (csrc/mingru.hip)
int ms_mingru_chunk();
int ms_mingru_scan(const void* zxg, long long in_stride, const float* bz, const float* bx, float* state, const int* q_start,
                   const int* state_slots, void* out, long long out_stride, int n_requests, int C, int max_q_len,
                   float* scratch, int dtype, hipStream_t stream);
// ---- window + pooled blocks attention (csrc/pooled_attention.hip)
int ms_pairs_rotate_store(void* qkv, long long stride, const int* positions, const float* inv_freq, const float* inv_freq_v,
                          const int* slots, void* k_pages, void* v_pages, int n_tokens, int num_heads, int num_kv_heads,
                          int head_dim, int value_dim, int rot_dims, int page_size, int v_transposed, int dtype,
                          hipStream_t stream);
int ms_pool_store(const void* k_pages, const void* v_pages, const int* table, int table_stride, const int* table_rows,
                  const int* token_req, const int* positions, const int* pool_slots, void* pk_pages, void* pv_pages,
                  int n_tokens, int num_kv_heads, int head_dim, int value_dim, int page_size, int pool, int v_transposed,
                  int dtype, hipStream_t stream);
int ms_pooled_attention(const void* q, long long q_stride, const void* k_pages, const void* v_pages, const int* table,
                        const void* pk_pages, const void* pv_pages, const int* pool_table, int table_stride,
                        const int* table_rows, const int* n_live_tokens, const int* token_req, const int* positions,
                        const float* inv_freq_v, void* out, long long out_stride, int n_tokens, int num_heads,
                        int num_kv_heads, int head_dim, int value_dim, int page_size, float scale, int size, int pool,
                        int v_transposed, int dtype, hipStream_t stream);
// the same on the matrix cores (csrc/attention_mfma.hip): bfloat16, value pages transposed, keys and values of one size
int ms_pooled_attention_mfma(const void* q, long long q_stride, const void* k_pages, const void* vt_pages,
                             const int* block_table, const void* pk_pages, const void* pvt_pages, const int* pool_table,
                             int table_stride, const int* table_rows, const int* q_start, const int* context_lens,
                             const float* turn_back, void* out, long long out_stride, int n_requests, int n_tokens,
                             int max_q_len, int num_heads, int num_kv_heads, int head_dim, int page_size, float scale,
                             int window, int pool, hipStream_t stream);
// ---- gated activations (csrc/glu.hip)
int ms_clamped_glu(const void* gu, long long in_stride, void* out, long long out_stride, int n_rows, int F, float limit,
                   float alpha, int dtype, hipStream_t stream);
int ms_scaled_swiglu(const void* gu, long long in_stride, const float* factor, const int* row_item, void* out,
                     long long out_stride, int n_rows, int F, int dtype, hipStream_t stream);
int ms_gelu_tanh_glu(const void* gu, long long in_stride, void* out, long long out_stride, int n_rows, int F, int dtype,
                     hipStream_t stream);
// ---- recurrences with a decay per key channel, the previous token's input, sums of two mixers (csrc/recurrence.hip)
int ms_decay_recurrence(const void* q, const void* k, const void* v, long long q_stride, long long k_stride,
                        long long v_stride, const float* z, const float* z_bias, int decay_kind, float inv_tau,
                        const float* bonus, float q_scale, float* state, const int* q_start, const int* state_slots,
                        float* out, int n_requests, int heads, int dim, int vdim, int stretch, int max_stretches,
                        float* pair_a, float* pair_b, int dtype, hipStream_t stream);
int ms_token_shift(const void* h, long long h_stride, const float* mu, void* state, const int* token_req,
                   const int* q_start, const int* state_slots, const int* n_live_tokens, void* out, int n_tokens,
                   int n_requests, int width, int n_mixes, int dtype, hipStream_t stream);
int ms_pair_sum(const void* a, const void* b, float scale_a, float scale_b, const float* norm_a, const float* norm_b,
                float eps, float* x, int n_rows, int width, int dtype, hipStream_t stream);
int ms_tanh(void* x, long long total, int dtype, hipStream_t stream);
int ms_concat_rows(const float* a, const float* b, void* out, int n_rows, int width_a, int width_b, int out_dtype,
                   hipStream_t stream);

}  // extern "C"
