// C entry points of the kernel library (the switches that tests and tuning runs flip are
// declared apart, in api_test.h: nothing of the product calls them).  Every function launches on `stream`
// and returns ILLM_OK, ILLM_ERR_ARG (sizes or dtypes it does not take; nothing
// was launched), ILLM_ERR_LAUNCH or, where said, ILLM_ERR_SCRATCH.  Pointers are device pointers.  dtype codes:
// 0 = float32, 1 = bfloat16.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int illm_version();

// out[t, :] = table[tokens[t], :] as float32.
int illm_embed(const int32_t* tokens, const void* table, int table_dt, float* out,
               int T, int E, int V, void* stream);
// The same rows multiplied by `scale` (in float32).
int illm_embed_scaled(const int32_t* tokens, const void* table, int table_dt, float* out,
                      int T, int E, int V, float scale, void* stream);

// out[t, :] = table[tokens[t]] * scale + pairs[(prev * mul_prev + tokens[t] * mul_cur) mod buckets]
// + places[row_pos[t]]: prev is the token above in the step if it belongs to the same slot, else
// last_token[slot]; a row at position 0 takes pairs[buckets].  pairs, places may be null.  `remember`
// (one row a sequence): last_token[slot] = tokens[t] as well.
int illm_embed_pairs(const int32_t* tokens, const int32_t* row_pos, const int32_t* row_slot,
                     const void* table, int table_dt, const void* pairs, int pairs_dt,
                     const void* places, int places_dt, int32_t* last_token, float* out, int T, int E,
                     int V, int buckets, int mul_prev, int mul_cur, int n_places, float scale,
                     int remember, void* stream);
// last_token[seq_slot[b]] = the last token of sequence b's rows (cu [n_seqs + 1] row offsets).
int illm_remember_last(const int32_t* tokens, const int32_t* cu, const int32_t* seq_slot,
                       int32_t* last_token, int n_seqs, void* stream);

// out[i] = float32(a[i]) + float32(b[i]): the two outputs of a block whose parts read the same rows.
int illm_sum_rows(const void* a, int a_dt, const void* b, int b_dt, float* out, size_t n,
                  void* stream);
// out[i] = sa float32(a[i]) + sb float32(b[i]).
int illm_sum_rows_scaled(const void* a, int a_dt, float sa, const void* b, int b_dt, float sb,
                         float* out, size_t n, void* stream);

// out[i] = max(x[i], 0)^2.
int illm_relu_squared(const void* x, void* out, int dt, size_t n, void* stream);
// out[i] = 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))).
int illm_gelu_tanh(const void* x, void* out, int dt, size_t n, void* stream);

// Residual add and RMS norm.  in_row = row_idx ? row_idx[r] : r;
// v = x[in_row] (+ delta[in_row]); when delta is given and row_idx is not, v is
// written back to x.  out[r] = v * rsqrt(mean(v^2) + eps) * w.  delta may be `planes` >= 1
// arrays, plane_stride elements apart (the sums of a product whose K was split,
// illm_gemm_mid_bf16), which are added in order.
int illm_add_rmsnorm(float* x, const void* delta, int delta_dt, int planes, size_t plane_stride,
                     const void* w, int w_dt, void* out, int out_dt, const int32_t* row_idx,
                     int rows, int E, float eps, void* stream);

// The same with a second addend of delta's shape (may be null): v = x + (delta + delta2), the two
// outputs of a block whose parts read the same rows.
int illm_add2_rmsnorm(float* x, const void* delta, int delta_dt, int planes, size_t plane_stride,
                      const void* delta2, int delta2_dt, const void* w, int w_dt, void* out,
                      int out_dt, const int32_t* row_idx, int rows, int E, float eps, void* stream);

// The same with a second weight of w's dtype and a second output of out's (both null: none): the
// rows normed once and written under two norms' weights, for a block whose two parts each read a
// norm of their own of the same rows.
int illm_add2_rmsnorm_two(float* x, const void* delta, int delta_dt, int planes, size_t plane_stride,
                          const void* delta2, int delta2_dt, const void* w, const void* w2, int w_dt,
                          void* out, void* out2, int out_dt, const int32_t* row_idx, int rows, int E,
                          float eps, void* stream);

// out[t, f] = silu(gate_up[t, f]) * gate_up[t, F + f].
int illm_silu_mul(const void* gate_up, void* out, int dt, int T, int F, void* stream);

// Rotate q and k of packed rows [q (nh*hd) | k (nkv*hd) | v (nkv*hd)] in place by the
// angles of `cos_sin` ([max_pos][rot/2][2] float32; null: no rotation) at row_pos[t],
// pairing 0 = (i, i + hd/2), 1 = (2i, 2i+1), i < rot/2; then store k and v of each row in the
// paged cache of row_slot[t] (skipped when kcache is null).  With a ring of pages, slot_len
// (length of every slot after the step) lets rows that a later row of the same step would
// overwrite be skipped; it may be null when no sequence brings more than one row.
int illm_rope_store(void* qkv, int dt, const float* cos_sin, int max_pos, int rot, int pairing,
                    const int32_t* row_pos, const int32_t* row_slot, const int32_t* slot_len,
                    void* kcache, void* vcache, const int32_t* page_table, int table_stride,
                    int page_size, int ring, int T, int nh, int nkv, int hd, void* stream);

// Y[M, N] = X[M, K] . W[N, K]^T, float32 accumulation in a fixed order; any sizes.
int illm_gemm_generic(const void* X, int x_dt, const void* W, int w_dt, void* Y, int y_dt,
                      int M, int N, int K, void* stream);

// The same product for float32 X and W with K % 16 == 0 on the matrix cores' float32 instruction
// (float32 operands, products and sums), for many rows.
int illm_gemm_f32_mfma(const float* X, const float* W, void* Y, int y_dt, int M, int N, int K,
                       void* stream);

// The same product for M <= 128 rows of float32 X and W with K % 32 == 0, W read once, on the
// matrix cores' float32 instruction with operands straight from memory.
int illm_gemm_rows_f32_mfma(const float* X, const float* W, void* Y, int y_dt, int M, int N, int K,
                            void* stream);

// The same product for M <= 16 rows when X and W are float32 and K % 4 == 0: W is read once
// (decoding on the 32-bit path); plain float32 multiply-adds.
int illm_gemv_rows_f32(const float* X, const float* W, void* Y, int y_dt, int M, int N, int K,
                       void* stream);

// Causal attention over packed rows of whole prompts (keys and values of the step
// itself).  cu_seqlens[n_seqs + 1]; window <= 0: all earlier keys.
int illm_attn_prefill_generic(const void* qkv, void* out, int dt, const int32_t* cu_seqlens,
                              int n_seqs, int max_len, int nh, int nkv, int hd, float scale,
                              int window, void* stream);

// The same on the matrix cores for bfloat16 and head_dim % 16 == 0 (else ILLM_ERR_ARG).
int illm_attn_prefill_bf16(const void* qkv, void* out, const int32_t* cu_seqlens, int n_seqs,
                           int max_len, int nh, int nkv, int hd, float scale, int window,
                           void* stream);
// The same with a soft cap on the scores, cap tanh(score / cap) (cap <= 0: none).
int illm_attn_prefill_bf16_cap(const void* qkv, void* out, const int32_t* cu_seqlens, int n_seqs,
                           int max_len, int nh, int nkv, int hd, float scale, float cap, int window,
                           void* stream);

// The two above for steps whose rows go on from tokens the cache already holds (a prompt cut into
// several steps): keys and values are read from the paged cache, which must hold the step's own
// rows too by then; row r of sequence b stands at position seq_start[b] + r and sees the keys
// 0 .. its position of the sequence in seq_slot[b].  The bfloat16 kernel needs pages of a multiple
// of 64 rows.
int illm_attn_prefill_paged_generic(const void* qkv, void* out, int dt, const int32_t* cu_seqlens,
                                    const int32_t* seq_slot, const int32_t* seq_start,
                                    const void* kcache, const void* vcache,
                                    const int32_t* page_table, int table_stride, int page_size,
                                    int ring, int n_seqs, int max_len, int nh, int nkv, int hd,
                                    float scale, int window, void* stream);
int illm_attn_prefill_paged_bf16(const void* qkv, void* out, const int32_t* cu_seqlens,
                                 const int32_t* seq_slot, const int32_t* seq_start,
                                 const void* kcache, const void* vcache, const int32_t* page_table,
                                 int table_stride, int page_size, int ring, int n_seqs, int max_len,
                                 int nh, int nkv, int hd, float scale, int window, void* stream);
// The same with a soft cap on the scores, cap tanh(score / cap) (cap <= 0: none).
int illm_attn_prefill_paged_bf16_cap(const void* qkv, void* out, const int32_t* cu_seqlens,
                                 const int32_t* seq_slot, const int32_t* seq_start,
                                 const void* kcache, const void* vcache, const int32_t* page_table,
                                 int table_stride, int page_size, int ring, int n_seqs, int max_len,
                                 int nh, int nkv, int hd, float scale, float cap, int window, void* stream);

// One query row per sequence over the paged cache.  partial: float32
// [B][nh][nsplit][hd + 2] scratch.  seq_len[b] = keys of sequence b, the new one included.
int illm_attn_decode_generic(const void* qkv, void* out, int dt, const void* kcache,
                             const void* vcache, const int32_t* page_table, int table_stride,
                             int page_size, int ring, const int32_t* seq_slot,
                             const int32_t* seq_len, float* partial, int nsplit, int B, int nh,
                             int nkv, int hd, float scale, int window, void* stream);

// The same for bfloat16 with head_dim % 8 == 0 and page_size % 64 == 0 (anything else:
// ILLM_ERR_ARG); nsplit == 1 needs no `partial`.  `waves`: waves per block that share a key
// range and combine through LDS (clamped to what the head group's registers and LDS allow).
int illm_attn_decode_bf16(const void* qkv, void* out, const void* kcache, const void* vcache,
                          const int32_t* page_table, int table_stride, int page_size, int ring,
                          const int32_t* seq_slot, const int32_t* seq_len, float* partial,
                          int nsplit, int waves, int B, int nh, int nkv, int hd, float scale,
                          int window, void* stream);
// The same with a soft cap on the scores, cap tanh(score / cap) (cap <= 0: none).
int illm_attn_decode_bf16_cap(const void* qkv, void* out, const void* kcache, const void* vcache,
                          const int32_t* page_table, int table_stride, int page_size, int ring,
                          const int32_t* seq_slot, const int32_t* seq_len, float* partial,
                          int nsplit, int waves, int B, int nh, int nkv, int hd, float scale, float cap,
                          int window, void* stream);

// illm_attn_decode_bf16 for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid it): it has no counterpart in the
// reference.  The split results go through an array that the library holds on every GPU it runs
// on (ILLM_DECODE_SCRATCH_BYTES, until the process ends) instead of a `partial` argument; the call
// allocates and frees nothing.  B * nh * nsplit * (hd + 2) * 4 bytes must fit the array, else
// ILLM_ERR_SCRATCH (3) and nothing is launched; nsplit == 1 uses no scratch.  All calls on one GPU
// share the array, so calls that overlap on one GPU (two streams) race: run them one after the
// other.  Nothing needs clearing between calls: every entry that is read was written by the same
// call before.
#define ILLM_DECODE_SCRATCH_BYTES (4u << 20)
int illm_attn_decode_bf16_static(const void* qkv, void* out, const void* kcache,
                                 const void* vcache, const int32_t* page_table, int table_stride,
                                 int page_size, int ring, const int32_t* seq_slot,
                                 const int32_t* seq_len, int nsplit, int waves, int B, int nh,
                                 int nkv, int hd, float scale, int window, void* stream);

// Y[M, N] = X[M, K] . W[N, K]^T for bfloat16 X and W, 1 <= M <= 64, K % 8 == 0, on the
// matrix cores with float32 accumulation; Y float32 or bfloat16.
// ssq != null (M <= 16 only): X is bfloat16(x * norm weight) of residual rows x whose sums of
// squares lie in ssq[M][parts] (left by illm_gemm_skinny_add), and row m of the result is scaled
// by 1 / sqrt(sum_p ssq[m][p] / K + eps): the product of the RMS norm of x.
// Wt (here and below, may be null): a copy of W laid out for these kernels,
// [tile][K / 32][16 rows][32 k] with tile t holding the 16 rows that block t works on (plain
// product: rows 16 t ..; gate|up: 8 gate rows 8 t .. and the same 8 up rows; q|k|v: 8 rows of a
// head and their 8 rotation partners, then 16 rows per tile for v), rows beyond the matrix zero.
// Used when M <= 16 and K % 32 == 0; W itself is then not read.
int illm_gemm_skinny_bf16(const void* X, const void* W, const void* Wt, void* Y, int y_dt, int M,
                          int N, int K, const float* ssq, int parts, float eps, int waves_wanted,
                          void* stream);

// Y[M, N] (float32 residual rows) += X . W^T for M <= 16 bfloat16 rows.  nw != null (the weight of
// the RMS norm that follows, bfloat16 or float32 [N]): also xb[M, N] = bfloat16(Y * nw) and
// ssq_out[M][ceil(N / 16)], partial sums of Y^2, for a product that takes `ssq`.
int illm_gemm_skinny_add(const void* X, const void* W, const void* Wt, float* Y, int M, int N,
                         int K, const void* nw, int nw_dt, void* xb, float* ssq_out,
                         int waves_wanted, void* stream);

// Y = X[M, K] . W[N, K]^T for M up to 128 from the tiled copy Wt of W, K a
// multiple of 32, X shared by a block's waves through LDS.  splits == 1: Y is [M, N] of y_dt;
// splits > 1: K is cut into that many ranges and Y is float32 [splits][M][N], the planes to be
// added by the caller (illm_add_rmsnorm takes them).  illm_gemm_mid_splits: the splits to use.
int illm_gemm_mid_bf16(const void* X, const void* Wt, void* Y, int y_dt, int M, int N, int K,
                       int splits, void* stream);
int illm_gemm_mid_splits(int N, int K);

// Products of 1 to 128 bfloat16 rows (meant for 9 and more) from the tiled copy
// Wt of W, K a multiple of 64, X shared by a block's waves through LDS, K cut inside the block
// (csrc/gemm_rows.hip).  illm_gemm_rows_bf16: Y[M, N] = X . W^T (plain tiles), float32 or bfloat16.
// illm_gemm_rows_gateup_silu: Y[M, F] = silu(X . Wg^T) * (X . Wu^T) from the gate|up tiles.
// illm_qkv_rope_store_rows: as illm_qkv_rope_store_skinny, from the q|k|v tiles.  ssq (M <= 16
// only): as for illm_gemm_skinny_bf16.
int illm_gemm_rows_bf16(const void* X, const void* Wt, void* Y, int y_dt, int M, int N, int K,
                        const float* ssq, int parts, float eps, void* stream);
int illm_gemm_rows_gateup_silu(const void* X, const void* Wt, void* Y, int y_dt, int M, int F,
                               int K, const float* ssq, int parts, float eps, void* stream);
// The same with the clamped gate in place of SiLU where limit > 0: Y = g sigmoid(alpha g) (u + 1),
// g = min(gate, limit), u = clamp(up, -limit, limit) (limit 0: SiLU as above).
int illm_gemm_rows_gateup_act(const void* X, const void* Wt, void* Y, int y_dt, int M, int F, int K,
                              const float* ssq, int parts, float eps, float limit, float alpha,
                              void* stream);
int illm_qkv_rope_store_rows(const void* X, const void* Wt, void* Y, int M, int K,
                             const float* cos_sin, int max_pos, const int32_t* row_pos,
                             const int32_t* row_slot, void* kcache, void* vcache,
                             const int32_t* page_table, int table_stride, int page_size, int ring,
                             int nh, int nkv, int hd, const float* ssq, int parts, float eps,
                             void* stream);

// Y[M, F] = silu(X . Wg^T) * (X . Wu^T), W = [Wg | Wu] as [2F, K]; same limits as the skinny
// product, `ssq` included.  waves_wanted: waves per block (0: the default choice).
int illm_gemm_skinny_gateup_silu(const void* X, const void* W, const void* Wt, void* Y, int y_dt,
                                 int M, int F, int K, const float* ssq, int parts, float eps,
                                 int waves_wanted, void* stream);
// The same with the clamped gate where limit > 0 (as illm_gemm_rows_gateup_act).
int illm_gemm_skinny_gateup_act(const void* X, const void* W, const void* Wt, void* Y, int y_dt,
                                int M, int F, int K, const float* ssq, int parts, float eps,
                                int waves_wanted, float limit, float alpha, void* stream);

// Few bfloat16 rows (M <= 16, hd % 16 == 0): the q|k|v product, the rotation of q and k (pairs
// (i, i + hd/2), all dims) at row_pos[m], q into Y[M, (nh + 2 nkv) hd] (k and v parts untouched),
// k and v into the paged cache of row_slot[m], all in one kernel.  ssq: as for
// illm_gemm_skinny_bf16.  waves_wanted: waves per block (0: the default choice).
int illm_qkv_rope_store_skinny(const void* X, const void* W, const void* Wt, void* Y, int M, int K,
                               const float* cos_sin, int max_pos, const int32_t* row_pos,
                               const int32_t* row_slot, void* kcache, void* vcache,
                               const int32_t* page_table, int table_stride, int page_size, int ring,
                               int nh, int nkv, int hd, const float* ssq, int parts, float eps,
                               int waves_wanted, void* stream);

// out[b] = index of the largest logit of row b (lowest index on ties).  A row is cut into
// `parts` (1 to 64) that blocks of their own take; scratch: 2 x B x parts 32-bit words (may be
// null when parts == 1).
int illm_argmax(const float* logits, int32_t* out, void* scratch, int B, int V, int parts,
                void* stream);

// Temperature / top-k / top-p / repeat-penalty sampling, one draw per row.
// scratch: float32 [2][B][V].  last_tokens: [B][n_last] (-1 = empty) or null.
// counters[b]: index of the draw in the request's stream; seeds[b]: the request's seed.
int illm_sample(const float* logits, float* scratch, int32_t* out, int B, int V, float temp,
                int top_k, float top_p, float repeat_penalty, const int32_t* last_tokens,
                int n_last, const uint64_t* seeds, const int32_t* counters, void* stream);

// The same without top_k for rows of 16,384 ids and more, several blocks a row and a kernel a
// pass (illm_sample walks such a row with one block).  rows: B x ILLM_SAMPLE_LONG_ROW_BYTES bytes
// of device memory, 8-byte aligned, that the passes hand their results on through; nothing in it
// needs clearing.  Shorter rows: ILLM_ERR_ARG.
#define ILLM_SAMPLE_LONG_ROW_BYTES 73728
int illm_sample_long_row_bytes(void);          // ILLM_SAMPLE_LONG_ROW_BYTES, for callers that cannot read this file
int illm_sample_long(const float* logits, float* scratch, void* rows, int32_t* out, int B, int V,
                     float temp, float top_p, float repeat_penalty, const int32_t* last_tokens,
                     int n_last, const uint64_t* seeds, const int32_t* counters, void* stream);

// ---- latent attention (csrc/latent_attention.hip).  A token keeps one normed latent row c [R] and one
// rotated key part kr [dr] shared by all heads, together one row [R + dr] of the paged cache
// [page][row in page][R + dr]; head h's key is [W_uk,h c | kr], its value W_uv,h c.
//
// Rows y [T, ncols] = [q: H (dn + dr) | down: R + dr | gate: H ...]: the first R of `down` are
// RMS-normed (float32 statistics, weight norm_w, eps), the last dr and the last dr of every q head
// are rotated in pairs (2i, 2i+1), i < rot/2, by cos_sin ([max_pos][rot/2][2] float32; null: no
// rotation) at row_pos[t]; q is rotated in place; the normed latent and the rotated key part go
// to the cache row of (row_slot[t], row_pos[t]) (null cache: nowhere) and to c_out [T, R] and
// kr_out [T, dr] (either may be null).  slot_len, ring: as for illm_rope_store.  cache_t (may be
// null): a second copy of the latent alone, laid out [page][R][row in page], for
// illm_latent_attn_decode_mfma.
int illm_latent_rope_store(void* y, int dt, int ncols, int T, int H, int dn, int dr, int R, int rot,
                           const float* cos_sin, int max_pos, const void* norm_w, int norm_dt,
                           float eps, const int32_t* row_pos, const int32_t* row_slot,
                           const int32_t* slot_len, void* cache, const int32_t* page_table,
                           int table_stride, int page_size, int ring, void* c_out, void* kr_out,
                           void* cache_t, void* stream);

// Packed rows [q heads | k heads | v heads] with every head P wide (zeros beyond a head's own
// dims) for the prompt attention kernels: q from y, keys [kvu's key part (dn) | kr (dr)], values
// kvu's value part (dv); kvu [T, H dn + H dv] = c . [W_uk ; W_uv]^T.
int illm_latent_pack(const void* y, int dt, int ncols, const void* kvu, const void* kr, void* out,
                     int T, int H, int dn, int dr, int dv, int P, void* stream);

// out[t, h dv + v] = attn[t, h P + v] * sigmoid(y[t, gate_off + h]).
int illm_latent_gate(const void* attn, const void* y, int dt, int ncols, int gate_off, void* out,
                     int T, int H, int dv, int P, void* stream);

// qa[b, h] = [W_uk,h^T q_h (R) | rotated part of q_h (dr)] as [B, H, R + dr] of qa_dt (float32
// sums), q from y.
int illm_latent_absorb_q(const void* y, int dt, int ncols, const void* wuk, int w_dt, void* qa,
                         int qa_dt, int B, int H, int dn, int dr, int R, void* stream);

// Both in one launch, for rows that will walk the cache (single tokens): illm_latent_rope_store's
// norm, rotation and store of the latent and the key part (no slot_len, no c_out / kr_out), and
// illm_latent_absorb_q with the query's rot part rotated on its way (y keeps the unrotated query).
int illm_latent_store_absorb(void* y, int dt, int ncols, int B, int H, int dn, int dr, int R, int rot,
                             const float* cos_sin, int max_pos, const void* norm_w, int norm_dt,
                             float eps, const int32_t* row_pos, const int32_t* row_slot, void* cache,
                             const int32_t* page_table, int table_stride, int page_size, int ring,
                             void* cache_t, const void* wuk, int w_dt, void* qa, int qa_dt,
                             void* stream);

// One token per sequence over the latent cache: scores qa[b, h] . cache row, softmax over the
// keys the token sees (all, or the last `window`), sums of latent rows.  Token b sees
// seq_len[b] + len_more keys, itself included.  partial: float32 [B][H][nsplit][R + 4] = (sums,
// max, weight, two unused) per range of keys.  R <= 1024.
int illm_latent_attn_decode(const float* qa, const void* cache, int dt, const int32_t* page_table,
                            int table_stride, int page_size, int ring, const int32_t* seq_slot,
                            const int32_t* seq_len, int len_more, float* partial, int nsplit, int B,
                            int H, int R, int dr, float scale, int window, void* stream);

// The same on the matrix cores for a bfloat16 cache with R % 16 == 0, (R + dr) % 8 == 0 and pages of
// a multiple of 32 rows; cache_t: the transposed copy that illm_latent_rope_store keeps; qa in
// bfloat16.
int illm_latent_attn_decode_mfma(const void* qa, const void* cache, const void* cache_t,
                                 const int32_t* page_table, int table_stride, int page_size,
                                 int ring, const int32_t* seq_slot, const int32_t* seq_len,
                                 int len_more, float* partial, int nsplit, int B, int H, int R,
                                 int dr, float scale, int window, void* stream);

// out[b, h dv + v] = (W_uv[h dv + v, :] . combined sums of (b, h)) * sigmoid(y[b, gate_off + h]).
int illm_latent_merge_up(const float* partial, int nsplit, const void* wuv, int w_dt, const void* y,
                         int dt, int ncols, int gate_off, void* out, int B, int H, int R, int dv,
                         void* stream);

// ---- routed feed-forward (csrc/moe.hip).  Pair p = t * top + k is token t's k-th choice.
// z [T, NE] = x [T, K] . w [NE, K]^T for a float32 matrix of few rows (a router's), x of x_dt:
// float32 products and sums.
int illm_few_outputs_f32(const void* x, int x_dt, const float* w, float* z, int T, int NE, int K,
                         void* stream);

// idx, wt [T, top]: the `top` outputs of z [T, NE] (float32) with the largest softmax(z) + corr
// (corr may be null), in falling order, and their softmax values.  NE <= 512.
// score_kind 0: softmax over all outputs; 1: every output's sigmoid.
int illm_moe_route(const float* z, const void* corr, int corr_dt, int T, int NE, int top,
                   int32_t* idx, float* wt, int score_kind, void* stream);

// order [NP]: the pairs whose choice is below NEr, grouped by choice; tiles [3 max_tiles + 1]:
// (expert, first place in order, rows <= tile_rows) per tile and, last, their number.
// max_tiles >= min(NP, NP / tile_rows + NEr).  NEr <= 512.  illm_moe_tile_rows(): the tile rows
// that illm_moe_rows takes (illm_moe_rows_mfma: 16, 32 or 64).
int illm_moe_tile_rows(void);
int illm_moe_group(const int32_t* idx, int NP, int NEr, int32_t* order, int32_t* tiles,
                   int max_tiles, int tile_rows, void* stream);

// Y[p] = X[p / x_div] . W[e_p]^T for every grouped pair p (W [experts][N][K]); gated: W
// [experts][2 N][K] = [gate | up] rows and Y[p] = silu(X Wg^T) * (X Wu^T).  Y [NP, N] of dt.
// act_kind (gated only) 0: silu(g) * u; 1: with g = min(g, limit), u = clamp(u, -limit, limit):
// g * sigmoid(1.702 g) * (u + 1).  row_w (may be null; gated only): a weight per pair that
// multiplies the pair's X row (applied to the two products, which is the same).
int illm_moe_rows(const void* X, int x_div, const void* W, int dt, int gated, const int32_t* order,
                  const int32_t* tiles, int max_tiles, void* Y, int N, int K, int act_kind,
                  float limit, const float* row_w, void* stream);

// The same for bfloat16 with K % 32 == 0 and tiles of up to 16, 32 or 64 rows, on the matrix cores.
int illm_moe_rows_mfma(const void* X, int x_div, const void* W, int gated, int tile_rows,
                       const int32_t* order, const int32_t* tiles, int max_tiles, void* Y, int N,
                       int K, int act_kind, float limit, const float* row_w, void* stream);

// out[t] = sum_k wt[t, k] * (idx[t, k] < NEr ? Y[t top + k] : h[t]) (+ g * shared[t], with
// g = sigmoid(h[t] . sg), or 1 if sg is null; shared may be null), float32 [T, E].  wt null: every
// weight 1.
int illm_moe_combine(const void* h, int dt, const int32_t* idx, const float* wt, const void* Y,
                     const void* shared, const void* sg, int sg_dt, float* out, int T, int E, int top,
                     int NEr, void* stream);

// ---- several residual streams (streams.hip)
// x float32 [T, S, E].  If y1: x_t <- sum_s mix[s, t] x_s + outw[t] (ya y1 (+ yb y2)) for every
// stream t (written back unless row_idx); then u = sum_s read[s] x_s (read null: weights 1) and
// h[r] = u / sqrt(mean(u^2) + eps) * w for every row (or those row_idx names).  S <= 8.
int illm_stream_mix_norm(float* x, int S, const void* y1, int y1_dt, float ya, const void* y2,
                         int y2_dt, float yb, const float* mix, const float* outw,
                         const float* read, const void* w, int w_dt, void* h, int h_dt,
                         const int32_t* row_idx, int rows, int E, float eps, void* stream);
// out[t, s, :] = table[tokens[t], :] * scale for every stream s < S.
int illm_embed_streams(const int32_t* tokens, const void* table, int table_dt, float* out, int T,
                       int E, int V, int S, float scale, void* stream);

// ---- the gated delta rule (delta_rule.hip)
int illm_delta_prepare(const void* P, int p_dt, int p_stride, int b_off, const void* A, int a_dt,
                       int a_stride, int a_off, const float* conv_w, int taps, void* tail,
                       int tail_dt, const int32_t* row_slot, const float* a_log,
                       const float* dt_bias, float* qn, float* kn, float* vv, float* beta,
                       float* dec, int T, int G, int H, int dk, int dv, int DW, int update_tail,
                       void* stream);
int illm_delta_conv_tail(const void* P, int p_dt, int p_stride, void* tail, int tail_dt,
                         const int32_t* cu, const int32_t* seq_slot, int n_seqs, int C, int taps,
                         void* stream);
int illm_delta_scan(const float* qn, const float* kn, const float* vv, const float* beta,
                    const float* dec, int DW, float* state, const int32_t* cu,
                    const int32_t* seq_slot, float* o, int n_seqs, int max_rows, int G, int H, int dk,
                    int dv, void* stream);
int illm_delta_finish(const float* o, const void* w, int w_dt, const void* Z, int z_dt, int z_stride,
                      int z_off, int gate_kind, void* out, int out_dt, int T, int H, int dv,
                      float eps, void* stream);

// ---- attention with a soft cap on the scores and value heads of their own width (attention_capped.hip)
int illm_kv_store2(const void* rows, int dt, int row_len, int k_off, int v_off,
                   const int32_t* row_pos, const int32_t* row_slot, void* kcache, void* vcache,
                   const int32_t* page_table, int table_stride, int page_size, int ring, int T,
                   int nkv, int dk, int dv, void* stream);
int illm_attn_cap_rows(const void* q, int q_stride, void* out, int dt, const int32_t* cu,
                       const int32_t* seq_slot, const int32_t* seq_start, const void* kcache,
                       const void* vcache, const int32_t* page_table, int table_stride,
                       int page_size, int ring, int n_seqs, int max_rows, int nh, int nkv, int dk,
                       int dv, float scale, float cap, int window, const float* slopes, int chunk,
                       const void* gate, int gate_stride, int gate_off, int gate_heads, float* lse, void* stream);
int illm_attn_cap_decode(const void* q, int q_stride, void* out, int dt, const void* kcache,
                         const void* vcache, const int32_t* page_table, int table_stride,
                         int page_size, int ring, const int32_t* seq_slot, const int32_t* seq_len,
                         float* partial, int nsplit, int B, int nh, int nkv, int dk, int dv,
                         float scale, float cap, int window, const float* slopes, int chunk,
                         const void* gate, int gate_stride, int gate_off, int gate_heads, float* lse, void* stream);
// The two calls above also take: `slopes` float32 [nh] (null: none), score -= slopes[h] (i - j);
// `chunk` > 0, a row sees only the keys j with floor(j / chunk) = floor(i / chunk); `gate` (null: none),
// rows [., gate_stride] of the queries' dtype, out *= sigmoid(gate[row, gate_off + h dv + d]) (with
// `gate_heads` gate[row, gate_off + h]); `lse` (null: none), float32 [rows, nh]: max + log(sum) of each
// softmax (single tokens: with nsplit >= 2).
// In place: q and k of rows [q (nh dk) | .. k at k_off | v at v_off] each divided by the root mean
// square over all their heads and multiplied by qw, kw (null: untouched); v <- (1 - lam[0]) v +
// lam[0] first[row, first_off ..] (lam null: untouched); k and v stored in the paged cache (null: not).
int illm_qkv_norm_mix_store(void* rows, int dt, int row_len, int k_off, int v_off, const void* qw,
                            const void* kw, int w_dt, float eps, const float* lam, const void* first,
                            int first_stride, int first_off, const int32_t* row_pos,
                            const int32_t* row_slot, void* kcache, void* vcache,
                            const int32_t* page_table, int table_stride, int page_size, int ring,
                            int T, int nh, int nkv, int dk, int dv, void* stream);

// ---- what stands around the plain gated recurrence (linear_scan.hip, delta_rule.hip)
// The scan of illm_delta_scan with a choice of rule: `correct` 1, the delta rule; 0, the plain gated
// rule S <- diag(g) S + k (beta v)^T, o = S^T q.
int illm_gated_scan(const float* qn, const float* kn, const float* vv, const float* beta,
                    const float* dec, int DW, float* state, const int32_t* cu,
                    const int32_t* seq_slot, float* o, int n_seqs, int max_rows, int G, int H, int dk,
                    int dv, int correct, void* stream);
// A state-space mixer's inputs from U [T, u_stride]: columns x_off.. = x (H dv) | B (G N) | C (G N)
// through the short convolution (conv_w float32 [C, taps], conv_b [C], tail [slots, taps - 1, C] of
// U's dtype) and SiLU into vv, kn, qn; beta = softplus(U[dt_off + h] + dt_bias[h]),
// dec = exp(-exp(a_log[h]) beta).
int illm_ssm_prepare(const void* U, int dt, int u_stride, int x_off, int dt_off, const float* conv_w,
                     const float* conv_b, int taps, void* tail, const int32_t* row_slot,
                     const float* a_log, const float* dt_bias, float* qn, float* kn, float* vv,
                     float* beta, float* dec, int T, int G, int H, int N, int dv, int update_tail,
                     void* stream);
// out = rms_norm over `norm_groups` equal parts of ((o + D x) silu(Z[z_off ..])) times w.
int illm_ssm_finish(const float* o, const float* x, const float* D, const void* Z, int z_dt,
                    int z_stride, int z_off, const void* w, int w_dt, void* out, int out_dt, int T,
                    int H, int dv, int norm_groups, float eps, void* stream);
// A matrix memory's inputs from U [T, u_stride] = [q (H dk) | k (H dk) | v (H dv) | ..]: qn = q dk^-1/2,
// kn, vv [T, H, dv + 1] (v and a column of ones); the gates i = cap tanh((U[i_off + h] + i_bias) / cap),
// f = logsigmoid(cap tanh((U[f_off + h] + f_bias) / cap)) against the running maximum m (m_state
// [slots, H], kept): dec = exp(f + m_before - m), beta = exp(i - m), em = exp(-m).
int illm_memory_prepare(const void* U, int dt, int u_stride, int i_off, int f_off, const float* i_bias,
                        const float* f_bias, float cap, float* m_state, const int32_t* cu,
                        const int32_t* seq_slot, float* qn, float* kn, float* vv, float* beta,
                        float* dec, float* em, int T, int n_seqs, int H, int dk, int dv, void* stream);
// o [T, H, dv + 1] (the last column n . q): y = o / (max(|n . q|, em) + 1e-6), then per head
// y / sqrt(mean y^2 + eps) * w[h dv + j] * sigmoid(Z[z_off + h dv + j]).
int illm_memory_finish(const float* o, const float* em, const void* w, int w_dt, const void* Z,
                       int z_dt, int z_stride, int z_off, void* out, int out_dt, int T, int H, int dv,
                       float eps, void* stream);

// ---- short causal convolutions with a kept tail, a sublayer's own norm, a clamped gate (short_conv.hip)
// y(t) = (add_input ? in(t) : 0) + bias[c] + sum_j w[c, j] in(t - (taps - 1 - j)), in(t) = X[t, x_off + c]
// (+ in_bias[c]); inputs before a step's first row from tail [slots, taps - 1, C]; `update_tail` (one
// row a sequence) moves the tail on in the same launch.  w float32 [C, taps]; bias, in_bias may be null.
int illm_short_conv(const void* X, int x_dt, int x_stride, int x_off, const float* in_bias,
                    const float* w, const float* bias, int taps, void* tail, int tail_dt,
                    const int32_t* row_slot, int add_input, void* out, int out_dt, int out_stride,
                    int T, int C, int update_tail, void* stream);
// The last taps - 1 inputs of every sequence of a step into the tail.
int illm_short_conv_tail(const void* X, int x_dt, int x_stride, int x_off, const float* in_bias,
                         void* tail, int tail_dt, const int32_t* cu, const int32_t* seq_slot,
                         int n_seqs, int C, int taps, void* stream);
// out[r] = gain * a[r] / sqrt(mean(a[r]^2) + eps) * w, float32.
int illm_rms_rows_gain(const void* a, int a_dt, const void* w, int w_dt, float* out, int rows, int E,
                       float eps, float gain, void* stream);
// x <- x + gain * a / sqrt(mean(a^2) + post_eps) * post_w (a null: nothing added); h = rmsnorm(x, eps) * w
// in the output's type; out = h + conv over time with the earlier inputs from tail [slots, taps - 1, E],
// which is moved on (conv_w null: out = h; the convolution is for steps of one row a sequence).  With
// row_idx only those rows are formed and x stays.  E floats of LDS: E <= 16384.
int illm_post_add_rmsnorm(float* x, const void* a, int a_dt, const void* post_w, int post_w_dt,
                          float post_eps, float gain, const void* w, int w_dt, void* out, int out_dt,
                          const int32_t* row_idx, int rows, int E, float eps, const float* conv_w,
                          int taps, void* tail, int tail_dt, const int32_t* row_slot, void* stream);
// gate_up [T, 2F]: out = g sigmoid(alpha g) (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit).
int illm_clamped_swish_mul(const void* gate_up, void* out, int dt, int T, int F, float limit,
                           float alpha, void* stream);

// ---- attention over a window of tokens and pooled blocks before it (attention_pooled.hip)
// In place on packed rows [q (nh dk) | .. k at k_off (nkv dk) | v at v_off (nkv dv)]: q and k heads
// turned by their positions (cos_sin float32 [n_positions, rot / 2, 2]; pairing 0: i with i + rot / 2,
// 1: 2i with 2i + 1; null: none), then, with `unit_norm`, divided by their root mean square, query head
// h then times q_scale[h] (float32 [nh]; null: none); k and v
// stored in the paged cache (kcache null: not stored; nkv 0: queries alone).
int illm_qk_rotate_store(void* rows, int dt, int row_len, int k_off, int v_off, const float* cos_sin,
                         int rot, int pairing, int n_positions, int unit_norm, float eps,
                         const float* q_scale, const int32_t* row_pos, const int32_t* row_slot, void* kcache, void* vcache,
                         const int32_t* page_table, int table_stride, int page_size, int ring, int T,
                         int nh, int nkv, int dk, int dv, void* stream);
// For every row whose position ends a block of `pool` tokens: the block's mean key and value, from
// the cache, into row (position / pool) of the sequence in kpool, vpool (same layout and page table).
int illm_pool_store(const int32_t* row_pos, const int32_t* row_slot, const void* kcache,
                    const void* vcache, void* kpool, void* vpool, int dt, const int32_t* page_table,
                    int table_stride, int page_size, int T, int nkv, int dk, int dv, int pool,
                    void* stream);
// Rows of a step over the cache: position i sees tokens j with 0 <= i - j < window and pooled block b
// if b pool + pool - 1 <= i - window (pool 0: none).  score = q . k scale head_scale[h] (null: 1).
int illm_attn_pooled_rows(const void* q, int q_stride, void* out, int dt, const int32_t* cu,
                          const int32_t* seq_slot, const int32_t* seq_start, const void* kcache,
                          const void* vcache, const void* kpool, const void* vpool,
                          const int32_t* page_table, int table_stride, int page_size, int n_seqs,
                          int max_rows, int nh, int nkv, int dk, int dv, float scale,
                          const float* head_scale, int window, int pool, const float* lse, void* stream);
// With `lse` (float32 [rows, nh]) the tokens of the window are done already: `out` holds their
// normalised sums and `lse` max + log(sum) of their softmax, and the pooled rows are merged in place.
// The same for one new token a sequence, at position seq_len - 1.
int illm_attn_pooled_decode(const void* q, int q_stride, void* out, int dt, const void* kcache,
                            const void* vcache, const void* kpool, const void* vpool,
                            const int32_t* page_table, int table_stride, int page_size,
                            const int32_t* seq_slot, const int32_t* seq_len, int B, int nh, int nkv,
                            int dk, int dv, float scale, const float* head_scale, int window, int pool,
                            const float* lse, void* stream);

// ---- gated linear attention and a gated linear recurrent unit (linear_scan.hip)
// Inputs of the plain gated rule with a decay per key channel: q dk^-1/2, k, v from U; decay =
// sigmoid(Z + zb)^(1 / tau); weight 1.
int illm_gla_prepare(const void* U, int dt, int u_stride, int q_off, int k_off, int v_off,
                     const void* Z, int z_dt, int z_stride, const float* zb, float tau, float* qn,
                     float* kn, float* vv, float* beta, float* dec, int T, int H, int dk, int dv,
                     void* stream);
// a = exp(-rate sigmoid(Wr u + br) softplus(lam)), x = sqrt(1 - a^2) sigmoid(Wi u + bi) u, the maps
// block-diagonal in nb blocks: Wt float32 [2, nb, C / nb (in), C / nb (out)].
int illm_lru_gates(const float* u, const float* Wt, const float* br, const float* bi, const float* lam,
                   float rate, float* a_out, float* x_out, int T, int C, int nb, void* stream);
// S <- a S + x per channel over every sequence's rows from state [slots, C] and back into it;
// out = S gelu_tanh(Y[:, y_off + c] + yb[c]).  `scratch` (may be null): 2 n_seqs ceil(max_rows / 32) C
// floats, with which steps of 64 rows a sequence or more run chunk by chunk in parallel.
int illm_lru_scan(const float* a, const float* x, float* state, const void* Y, int y_dt, int y_stride,
                  int y_off, const float* yb, void* out, int out_dt, const int32_t* cu,
                  const int32_t* seq_slot, int n_seqs, int max_rows, int C, float* scratch, void* stream);

#ifdef __cplusplus
}
#endif
