// C launch entry points of the HIP kernel library. The kernels are compiled without any
// PyTorch headers; bindings.cpp wraps these in torch custom ops.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

// ---- norm.hip -------------------------------------------------------------------------
// out[r,:] = norm(x[row_idx ? row_idx[r] : r,:] (+ addend, written back into x)) * w (+ b).
// addend: `delta` (bf16 rows) or the fp32 split-K partials [splits][pM][H] of the preceding GEMM
// (+ pbias). mode: 0 RMSNorm, 1 LayerNorm, 2 only fold the addend into x.
void dlia_norm(void* out, void* x, const void* delta, const float* partial, int splits, long pM,
               const void* pbias, const void* w, const void* b, const int* row_idx, int rows, int H,
               long ldx, long ldo, float eps, int mode, float* qscale, hipStream_t stream);
// qscale != null: `out` receives e4m3 bytes (row stride ldo BYTES) and qscale[r] the row's scale

// ---- embed.hip ------------------------------------------------------------------------
// out[t,:] = wte[ids[t],:] (+ wpe[pos[t],:])
void dlia_embed(void* out, const int* ids, const int* pos, const void* wte, const void* wpe,
                int T, int H, int vocab, int max_pos, hipStream_t stream);

// ---- rope_kv.hip ----------------------------------------------------------------------
// RoPE on the q and k slices of a fused qkv activation (in place on q), and scatter of the
// (rotated) k and v rows into the paged, MFMA-fragment-ordered KV cache.
// The q/k/v values come from `qkv` itself, or (partial != null) from the fp32 split-K partials
// [splits][T][(Hq+2Hkv)*D] (+ pbias) of the QKV GEMM; the rotated q is written to `qkv` either way.
void dlia_rope_kvwrite(void* qkv, const float* partial, int splits, const void* pbias, void* kv_cache,
                       float* kv_scale, const float* cos_t, const float* sin_t,
                       const int* tok_pos, const int* tok_seq, const int* block_table,
                       int T, int Hq, int Hkv, int D, int max_blocks, int num_blocks,
                       int rope_len, int use_rope, hipStream_t stream);

// ---- gemm_skinny.hip ------------------------------------------------------------------
// out[M,N] = epilogue(x[M,K] @ Wp^T), M <= 128 per call (weight-streaming regime).
// epi: 0 none, 1 +bias, 2 +residual, 3 +bias+residual, 4 swiglu (interleaved gate/up tiles,
// N = 2*N_out), 5 +bias then gelu_tanh, 6 fp32 partials [splitk][M][N] only (summed by the
// consumer kernel). out_f32: write fp32 instead of bf16.
void dlia_gemm_skinny_head(void* logits, const void* x, const void* wp, int M, int N, int K, long ldx, long ldo,
                           float* chunk_max, long ldc, int n_valid, hipStream_t stream);
void dlia_gemm_skinny(void* out, const void* x, const void* wp, const void* bias,
                      const void* residual, float* workspace, const float* wscale,
                      int M, int N, int K, long ldx, long ldo, long ldr, int epi, int out_f32,
                      int splitk, int ntw, hipStream_t stream);
// the decomposition the launcher would choose: n-tiles per wave and split-K factor
void dlia_gemm_skinny_config(int M, int N, int K, int epi, int allow_split, int* ntw_out, int* splitk_out);
int dlia_gemm_skinny_splitk(int M, int N, int K);

// ---- gemm_a8w8.hip --------------------------------------------------------------------
// fp8 x fp8 streaming GEMM on the block-scaled MFMA (M <= 256): xq = e4m3 bytes [M,K] with per-row
// scales, wp = pack_weight_a8w8 image with per-column scales. Epilogues as dlia_gemm_skinny.
void dlia_gemm_a8w8(void* out, const void* xq, const float* xscale, const void* wp, const float* wscale,
                    const void* bias, const void* residual, float* workspace, int M, int N, int K,
                    long ldx, long ldo, long ldr, int epi, int out_f32, int splitk, int ntw, hipStream_t stream);
// per-row dynamic e4m3 quantisation of bf16 activations: q[M,K] bytes (row stride ldq), scale[M]
void dlia_quant_rows(void* q, float* scale, const void* x, int M, int K, long ldx, long ldq, hipStream_t stream);

// ---- gemm_rows.hip / gemm_pingpong.hip (more than 128 / 256 rows; reached through dlia_gemm_skinny) ----
// 1: the streaming GEMM picks 128- / 64-row blocks on shapes with few column blocks (off by default); returns the old value
int dlia_gemm_rows_set_narrow(int on);
// bf16 GEMM of more than 256 rows, same epilogues as dlia_gemm_skinny (0..5). workspace / ws_floats (optional):
// room for the in-launch split-K of thin shapes; its LAST 4096 words are arrival counters, zero between launches.
// chunk_max (optional, the ping-pong kernel only): per row the maximum of every 32-column chunk of the output
// (columns >= n_valid excluded), chunk_max[m * ldc + n / 32].
void dlia_gemm_large(void* out, const void* x, const void* wp, const void* bias, const void* residual,
                     float* workspace, long ws_floats, int M, int N, int K, long ldx, long ldo, long ldr,
                     int epi, int out_f32, int wg_target, hipStream_t stream, float* chunk_max = nullptr, long ldc = 0,
                     int n_valid = 0);
extern "C" void dlia_gemm_a8w8_large(void* out, const void* xq, const float* xscale, const void* wp, const float* wscale,
                                     const void* bias, const void* residual, float* workspace, long ws_floats, int M,
                                     int N, int K, long ldx, long ldo, long ldr, int epi, int out_f32, int wg_target,
                                     hipStream_t stream);
// kernel for bf16 GEMMs of more than 256 rows: 0 = 256 x 256 ping-pong tiles (default), 2 = the loader-wave
// kernel of gemm_rows.hip; which < 0 only reads; returns the previous choice
int dlia_gemm_large_choice(int which);
// the large-M kernel's in-launch split-K: factor for a shape, and the workspace floats it needs (slabs + counters)
int dlia_gemm_pingpong_splitk(int M, int N, int K);
long dlia_gemm_pingpong_ws_floats(int M, int N, int K);

// ---- attention.hip --------------------------------------------------------------------
// Causal GQA attention of ragged query chunks against the paged KV cache (prefill chunks and
// single-token decode are the same kernel). kv_scale != null: e4m3 cache + per-(token, head) scales. Work items are (sequence, kv head, query tile,
// kv split); `partial` holds split-KV partials when splits > 1.
void dlia_paged_attention(void* out, const void* qkv, const void* kv_cache, const float* kv_scale,
                          const int* q_start, const int* ctx_lens, const int* block_table,
                          const int* slots, float* partial, int B, int max_q_len, int Hq,
                          int Hkv, int D, int table_rows, int max_blocks, int num_blocks,
                          long ldq, long ldo, float scale, int splits, hipStream_t stream, int window = 0, int sink = 0,
                          const float* temp = nullptr, const float* bias = nullptr, int bias_rows = 0, const float* sinkv = nullptr,
                          const float* gate = nullptr, long ldg = 0);
// temp / bias / sinkv / gate (bf16 cache, sink set): a learned factor per head on the scores, a bias per (distance, head) and
// the sink's score, both divided by `scale` by the caller, and a sigmoid gate logit per (token, head) on the head's output
// (window > 0: a query at i sees the keys j with 0 <= i - j < window; sink: one more softmax term exp(0) without a value;
// both for the bf16 cache only)
long dlia_paged_attention_ws_floats(int B, int max_q_len, int Hq, int Hkv, int D, int splits);

// ---- sampler.hip ----------------------------------------------------------------------
// One token per row from fp32 logits [R, ldl] with temperature / top-k / top-p and a
// counter-based RNG keyed by (seed[r], step[r]); temperature <= 0 -> argmax.
// chunk_max (optional): per row the maximum of every 32-column chunk of its logits (row stride ldc, at most
// 8192 chunks), as the lm_head GEMM writes them; the row is then read only where a candidate can be.
void dlia_sample(int* out_tokens, const float* logits, const float* temperature,
                 const int* top_k, const float* top_p, const uint64_t* seeds,
                 const int* steps, int R, int vocab, long ldl, float* dbg_probs,
                 int* dbg_ids, int dbg_cap, hipStream_t stream, const float* chunk_max = nullptr, long ldc = 0,
                 int* ids_out = nullptr, int* steps_adv = nullptr, int* ctx_adv = nullptr);

// ---- norm32.hip (fp32 residual stream) ------------------------------------------------------
void dlia_embed32(float* out, const int* ids, const void* table, int table_f32, int T, int H, int vocab, hipStream_t stream);
// y != null: x += rms(y) * (off + wb); out != null: out = rms(x[row_idx ? row_idx[r] : r]) * (off + wn)
void dlia_norm32(void* out, int out_f32, float* x, const float* y, const float* wb, const float* wn, const int* row_idx,
                 int rows, int H, long ldx, long ldy, long ldo, float eps, float off, hipStream_t stream);
void dlia_gated_headnorm(void* out, int out_f32, const float* o, const float* gate, const float* w, int T, int heads, int dv,
                         long ldo_in, long ldg, long ld_out, float eps, hipStream_t stream);

// ---- gemm_any.hip ---------------------------------------------------------------------------
// C[M,N] = A[M,K] . W[N,K]^T (+ bias), any shape, row-major W; epi 1: gated pair (interleaved gate / up tiles) ->
// gelu_tanh(gate) * up, N / 2 columns
void dlia_gemm_any(void* C, int out_f32, const void* A, const void* W, int in_f32, const float* bias, int M, int N, int K,
                   long lda, long ldw, long ldc, int epi, hipStream_t stream);
// `blocks` independent products in one launch: block b reads A + b * a_step, W + b * w_step, bias + b * N and writes
// C + b * c_step (steps in elements). epi 0 only.
void dlia_gemm_blocks(void* C, int out_f32, const void* A, const void* W, int in_f32, const float* bias, int M, int N, int K,
                      long lda, long ldw, long ldc, int blocks, long a_step, long w_step, long c_step, hipStream_t stream);

// act[m, j] = gelu_tanh(gu[m, j]) * gu[m, F + j] (bf16, F a multiple of 8, 16-byte aligned rows)
void dlia_gated_gelu(void* act, const void* gu, int M, int F, long ldg, long lda, hipStream_t stream);

// ---- window_attention.hip -------------------------------------------------------------------
void dlia_kv_store(const float* qkv, float* vfirst, const float* lam, int mix, void* kcache, void* vcache, int cache_f32,
                   const int* tok_pos, const int* tok_seq, const int* block_table, int T, int max_blocks, int num_blocks,
                   int table_rows, int G, int d, int dv, int q_cols, long ld, hipStream_t stream);
void dlia_window_attention(void* out, const float* qkv, const void* kcache, const void* vcache, int f32, const int* tok_pos,
                           const int* tok_seq, const int* block_table, int T, int max_blocks, int num_blocks, int table_rows,
                           int H, int G, int d, int dv, long ldq, long ldo, float scale, int window, int sink,
                           const float* temp, const float* bias, int bias_rows, const float* sinkv, const float* gate, long ldg,
                           hipStream_t stream);

// v <- (1 - lam) v + lam v_first on the v columns of a bf16 fused qkv activation (mix 2), or v_first <- v (mix 1)
void dlia_value_mix(void* qkv, float* vfirst, const float* lam, int mix, int T, int v_off, int v_cols, long ld, hipStream_t stream);

// ---- delta_rule.hip -------------------------------------------------------------------------
void dlia_short_conv(float* y, const float* z, float* carry, const float* taps, const int* q_start, const int* ctx,
                     const int* slots, int B, int max_q, int C, int K, long ldz, int state_rows, const float* bias, int silu,
                     hipStream_t stream);
void dlia_unit_heads(float* x, int T, int heads, int d, long ld, int scaled_heads, float mult, float eps, hipStream_t stream);
int dlia_delta_rule(float* o, const float* y, const float* z, float* state, const float* A_log, const float* dt_bias,
                    const int* q_start, const int* ctx, const int* slots, int B, int G, int Hv, int d, int dv, int C, long ldz,
                    int col_beta, int col_a, int state_rows, int max_q, hipStream_t stream);

// ---- gated_ops.hip --------------------------------------------------------------------------
void dlia_embed_pos32(float* out, const int* ids, const int* pos, const void* table, const void* ptable, int f32, int T, int H,
                      int vocab, int max_pos, hipStream_t stream);
void dlia_dyt_gate(void* out, int out_f32, float* x, const float* ya, const float* yb, const float* wa, const float* wb,
                   const float* gl, const float* gb, const float* step, const float* nw, const float* nb, const int* row_idx,
                   int rows, int H, long ldx, long ldy, long ldg, long ldo, float alpha, float eps, hipStream_t stream);
void dlia_headnorm_gate(void* out, int out_f32, const float* o, const float* gate, const float* w, int T, int heads, int dv,
                        int extra, long ldo_in, long ldg, long ld_out, float eps, hipStream_t stream);
void dlia_unary_act(void* act, int out_f32, const float* z, int M, int F, long ldz, long lda, int kind, hipStream_t stream);
void dlia_softcap(float* z, int M, int V, long ld, float cap, hipStream_t stream);

// ---- state_scan.hip -------------------------------------------------------------------------
int dlia_state_scan_blocks(int d, int ncols);
int dlia_state_scan(int rule, float* o, long ldo, const float* z, long ldz, const float* wz, long ldw, float* state, float* mstate,
                    const float* b0, const float* b1, const int* q_start, const int* ctx, const int* slots, int B, int H, int d,
                    int dv, int state_rows, int col_q, int col_k, int col_v, int col_a, int col_i, int col_f, float cap,
                    float qscale, int max_q, int quick, hipStream_t stream);

// ---- moe.hip --------------------------------------------------------------------------------
void dlia_moe_route(int* sel, float* wts, const float* logits, long ld, int T, int E, int top, int groups, int keep, float scale,
                    const float* corr, int softmax, int group_rank, int renorm, hipStream_t stream);
void dlia_moe_plan(int* tiles, int* row_tok, int* pair_row, const int* sel, int pairs, int top, int E, int max_rows, int tile_rows,
                   hipStream_t stream);
// tile_rows: 32 (register-tiled expert kernels, any type and shape) or 128 (LDS-tiled, bf16, K a multiple of 32, aligned rows)
void dlia_moe_up(void* act, const void* x, const void* wg, const void* wu, int f32, const int* tiles, const int* row_tok,
                 int max_tiles, int wide, int F, int K, long ldx, long lda, float limit, int tile_rows, hipStream_t stream);
void dlia_moe_down(float* y, const void* act, const void* wd, int f32, const int* tiles, const int* row_tok, int max_tiles, int wide,
                   int H, int F, long lda, int tile_rows, hipStream_t stream);
// (wide: 128 / 256 output columns per workgroup, for steps with many rows; else 64)
void dlia_moe_combine(float* out, const float* y, const int* pair_row, const float* wts, int T, int H, int top, long ldo,
                      const float* x, long ldx, hipStream_t stream);



// ---- parallel_ops.hip (parallel layers on one norm, token shift, rotation + cache write, attention over score maps, RG-LRU) ----
void dlia_par_norm(void* out, int out_f32, float* out32, float* x, const float* ya, const float* yb, const float* ls1,
                   const float* ls2, const float* w, float* carry, const int* tok_seq, int T, int state_rows, int H, long ldx,
                   long ldya, long ldyb, long ldo, float eps, hipStream_t stream);
void dlia_token_shift(void* out, int out_f32, const float* n32, const float* carry, const float* mu, const int* tok_pos,
                      const int* tok_seq, int T, int state_rows, int H, long ldo, hipStream_t stream);
void dlia_rope_cache_write(float* q, long ldq, int q_vecs, int q_stride, int q_off, void* q_out, long ldqo, int q_cols, float* kv,
                           long ldkv, int k_cols, int k_vecs, int k_stride, int k_off, int v_src, int v_cols, int v_t, void* kcache,
                           void* vcache, int f32, int G, int dims, int interleaved, const float* cos_t, const float* sin_t, int table_pos,
                           const int* tok_pos, const int* tok_seq, const int* block_table, int T, int max_blocks, int num_blocks,
                           int table_rows, hipStream_t stream);
void dlia_multi_attention(void* out, long ldo, const float* q, long ldq, int q_head, const void* kcache, int k_row,
                          const void* vcache, int v_row, int v_off, int f32, const int* tok_pos, const int* tok_seq,
                          const int* block_table, int T, int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv,
                          int maps, float scale, int window, int keep_first, float softcap, float lam, float post, float eps,
                          const float* gate, long ldg, int Gk, int chunk, const float* sink, hipStream_t stream);
// bf16 on the matrix cores; values key-contiguous in `vt` [blocks, G, dv, 32]. Returns 1 (nothing launched) for sizes it does not take.
int dlia_tile_attention(void* out, long ldo, const void* q, long ldq, int q_head, const void* kcache, int k_row, const void* vt,
                        const int* q_start, const int* ctx, const int* slots, const int* block_table, int B, int max_q,
                        int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv, int maps, float scale,
                        int window, int keep_first, float softcap, float lam, float post, float eps, const float* gate, long ldg,
                        float* part, long part_floats, int Gk, int chunk, const float* sink, hipStream_t stream);
// key splits of a single-token step of B rows (the workspace `part` holds B * H * maps * splits * (dv + 2) floats)
int dlia_tile_attention_splits(int B, int H, int G);
// what to pass as G there: the value heads, or 1 when the tiles of a single-token step span all heads (a key cache of Gk = 1 head)
int dlia_tile_attention_tile_groups(int G, int Gk);
void dlia_rglru_scan(void* out, int out_f32, long ldo, const float* u, long ldu, const float* gates, long ldg, const float* ypre,
                     long ldy, const float* clam, float* state, const int* q_start, const int* ctx, const int* slots, int B,
                     int max_q, int W, int bw, int state_rows, float* ws, long ws_floats, int rows, hipStream_t stream);
long dlia_rglru_scan_ws_floats(int rows, int B, int W);
void dlia_xielu(void* act, int out_f32, const float* z, int M, int F, long ldz, long lda, const float* pq, hipStream_t stream);
void dlia_scale_rows(float* x, int M, int N, long ld, float s, hipStream_t stream);
// ---- postnorm_ops.hip (norms on the sublayers' outputs only; q / k / v preparation of an attention mixer) ----
void dlia_post_norm_add(void* out, int out_f32, long ldo, float* x, long ldx, const float* ya, long ldya, const float* yb, long ldyb,
                        float a, float b, const float* w, int T, int H, float eps, hipStream_t stream);
// Returns 1 (nothing launched) when a token's q and k do not fit a workgroup's LDS.
int dlia_mix_prep(const float* z, long ldz, int T, int H, int G, int d, int dv, const float* qw, const float* kw, float eps, int dims,
                  const float* cos_t, const float* sin_t, int table_pos, int v_unit, const float* mix, void* q_out, int q_f32, long ldqo,
                  void* kcache, int Gk, void* vcache, int v_t, int cache_f32, const int* tok_pos, const int* tok_seq,
                  const int* block_table, int max_blocks, int num_blocks, int table_rows, hipStream_t stream);
// ---- mixed_attention.hip (scores mixed across heads before the softmax; prompt portions, bf16, matrix cores) ----
void dlia_tile_merge(void* out, long ldo, const float* part, int items, int H, int dv, int nz, const float* gate, long ldg,
                     const float* sink, hipStream_t stream);
int dlia_mixed_attention_fits(int H, int G, int d, int dv);
// floats of the workspace with which a step of T rows may deal a tile's key blocks out to several workgroups
long dlia_mixed_attention_part_floats(int T, int H, int dv);
// keys [blocks][32][G d] (one row of all key heads per token), values [blocks][G][dv][32]; returns 1 (nothing launched) for sizes it does not take
int dlia_mixed_attention(void* out, long ldo, const void* q, long ldq, const void* kcache, int k_row, const void* vt, const float* mix,
                         const int* q_start, const int* ctx, const int* slots, const int* block_table, int B, int max_q, int max_blocks,
                         int num_blocks, int table_rows, int H, int G, int d, int dv, int chunk, const float* sink, const float* gate,
                         long ldg, float* part, long part_floats, int T, hipStream_t stream);
// ---- misc.hip -------------------------------------------------------------------------
void dlia_advance_i32(int* x, int n, int delta, hipStream_t stream);
void dlia_scatter_rows_i32(int* dst, const int* rows, const int* src, int nrows, int ncols, int dst_rows, hipStream_t stream);
void dlia_scatter_i32(int* dst, const int* idx, const int* val, int n, long limit, hipStream_t stream);

}  // extern "C"
