// torch custom-op bindings (namespace `dlia`) of the kernels for stacks with parallel layers on one norm, token shift,
// partial rotations, attention over one or two score maps (also through a cached latent), real-gated linear recurrences and
// block-diagonal products. As everywhere in this library, shapes, types and devices are checked on the host before anything
// is launched.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/util/Optional.h>

#include "launch.h"

namespace {

using at::Tensor;
using OptTensor = const std::optional<Tensor>&;

inline hipStream_t cur_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

#define DLIA_CHECK(cond, ...) TORCH_CHECK(cond, "dlia: ", __VA_ARGS__)
#define DLIA_ON_DEVICE_OF(t) \
  DLIA_CHECK((t).is_cuda(), #t " must be a GPU tensor"); \
  const c10::hip::HIPGuardMasqueradingAsCUDA dlia_device_guard_((t).device())

inline bool is_f32(const Tensor& t) { return t.scalar_type() == at::kFloat; }
inline void check_f32(const Tensor& t, const char* name) {
  DLIA_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, " must be contiguous float32 on the GPU");
}
inline void check_i32(const Tensor& t, const char* name) {
  DLIA_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be contiguous int32 on the GPU");
}
inline void check_act(const Tensor& t, const char* name) {
  DLIA_CHECK(t.is_cuda() && (t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16), name, " must be float32 or bfloat16 on the GPU");
}
inline void check_mat(const Tensor& t, const char* name) {
  DLIA_CHECK(t.dim() == 2 && (t.size(1) == 1 || t.stride(1) == 1), name, " must be 2-D with unit inner stride");
}
inline void check_fmat(const Tensor& t, const char* name) {
  check_mat(t, name);
  DLIA_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat, name, " must be float32 on the GPU");
}
inline const float* opt_f32(OptTensor t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  check_f32(*t, name);
  DLIA_CHECK(t->numel() >= n, name, " has too few elements");
  return t->data_ptr<float>();
}

// x += ls1 * ya + ls2 * yb; the closing layer's carried rows are saved; out / out32 = rms(x) w.
void par_norm(const std::optional<Tensor>& out, Tensor out32, Tensor x, OptTensor ya, OptTensor yb, OptTensor ls1, OptTensor ls2,
              OptTensor w, const std::optional<Tensor>& carry, const Tensor& tok_seq, double eps) {
  DLIA_ON_DEVICE_OF(x);
  check_fmat(x, "x"); check_f32(out32, "out32"); check_i32(tok_seq, "tok_seq");
  const int64_t T = x.size(0), H = x.size(1);
  DLIA_CHECK(out32.dim() == 2 && out32.size(0) >= T && out32.size(1) == H && tok_seq.numel() >= T, "par_norm: out32 [T, H], tok_seq [T]");
  const float *yap = nullptr, *ybp = nullptr;
  long ldya = 0, ldyb = 0;
  if (ya.has_value()) {
    check_fmat(*ya, "ya");
    DLIA_CHECK(ya->size(0) >= T && ya->size(1) == H && ls1.has_value(), "par_norm: ya [T, H] with its scale");
    yap = ya->data_ptr<float>(); ldya = ya->stride(0);
    if (yb.has_value()) {
      check_fmat(*yb, "yb");
      DLIA_CHECK(yb->size(0) >= T && yb->size(1) == H && ls2.has_value(), "par_norm: yb [T, H] with its scale");
      ybp = yb->data_ptr<float>(); ldyb = yb->stride(0);
    }
  }
  void* op = nullptr; long ldo = 0; int of32 = 1;
  if (out.has_value()) {
    check_act(*out, "out"); check_mat(*out, "out");
    DLIA_CHECK(out->size(0) >= T && out->size(1) == H && w.has_value(), "par_norm: out [T, H] with the norm's weight");
    op = out->data_ptr(); ldo = out->stride(0); of32 = is_f32(*out);
  }
  float* cp = nullptr; int state_rows = 0;
  if (carry.has_value()) {
    check_f32(*carry, "carry");
    DLIA_CHECK(carry->dim() == 2 && carry->size(1) == H, "par_norm: carry [slots, H]");
    cp = carry->data_ptr<float>(); state_rows = (int)carry->size(0);
  }
  DLIA_CHECK(op || yap || cp, "par_norm: nothing to do");
  dlia_par_norm(op, of32, out32.data_ptr<float>(), x.data_ptr<float>(), yap, ybp, opt_f32(ls1, H, "ls1"), opt_f32(ls2, H, "ls2"),
                opt_f32(w, H, "w"), cp, tok_seq.data_ptr<int>(), (int)T, state_rows, (int)H, x.stride(0), ldya, ldyb, ldo, (float)eps,
                cur_stream());
}

void token_shift(Tensor out, const Tensor& n32, const Tensor& carry, const Tensor& mu, const Tensor& tok_pos, const Tensor& tok_seq) {
  DLIA_ON_DEVICE_OF(out);
  check_act(out, "out"); check_mat(out, "out"); check_f32(n32, "n32"); check_f32(carry, "carry"); check_f32(mu, "mu");
  check_i32(tok_pos, "tok_pos"); check_i32(tok_seq, "tok_seq");
  const int64_t T = out.size(0), H = out.size(1);
  DLIA_CHECK(n32.dim() == 2 && n32.size(0) >= T && n32.size(1) == H && carry.dim() == 2 && carry.size(1) == H && mu.numel() == H &&
             tok_pos.numel() >= T && tok_seq.numel() >= T, "token_shift: out / n32 [T, H], carry [slots, H], mu [H]");
  dlia_token_shift(out.data_ptr(), is_f32(out), n32.data_ptr<float>(), carry.data_ptr<float>(), mu.data_ptr<float>(),
                   tok_pos.data_ptr<int>(), tok_seq.data_ptr<int>(), (int)T, (int)carry.size(0), (int)H, out.stride(0), cur_stream());
}

// q [T, >= q_cols] fp32 (rotated in place: q_vecs vectors `q_stride` apart, entries [q_off, q_off + dims) of each); kv [T, k_cols + v_cols]
// fp32 (k rotated in place the same way, then k and v rows written to the caches [blocks, G, 32, k_cols / G] and [blocks, G, 32, v_cols / G]).
void rope_cache_write(Tensor q, int64_t q_vecs, int64_t q_stride, int64_t q_off, const std::optional<Tensor>& q_out, int64_t q_cols,
                      Tensor kv, int64_t k_cols, int64_t k_vecs, int64_t k_stride, int64_t k_off, int64_t v_src, int64_t v_cols,
                      bool v_t, Tensor kcache, const std::optional<Tensor>& vcache, int64_t dims, bool interleaved, OptTensor cos_t, OptTensor sin_t,
                      const Tensor& tok_pos, const Tensor& tok_seq, const Tensor& block_table) {
  DLIA_ON_DEVICE_OF(kcache);
  check_fmat(q, "q"); check_fmat(kv, "kv"); check_act(kcache, "kcache");
  check_i32(tok_pos, "tok_pos"); check_i32(tok_seq, "tok_seq"); check_i32(block_table, "block_table");
  const int64_t T = kv.size(0);
  DLIA_CHECK(q.size(0) >= T && tok_pos.numel() >= T && tok_seq.numel() >= T && block_table.dim() == 2, "rope_cache_write: rows");
  DLIA_CHECK(dims >= 0 && dims % 2 == 0 && q_vecs >= 0 && k_vecs >= 0 && q_stride >= 1 && k_stride >= 1, "rope_cache_write: rotation geometry");
  DLIA_CHECK(q_cols <= q.size(1) && (q_vecs == 0 || (q_vecs - 1) * q_stride + q_off + dims <= q.size(1)) && q_off >= 0,
             "rope_cache_write: rotated q entries beyond the row");
  DLIA_CHECK(k_cols >= 1 && v_cols >= 0 && k_cols <= kv.size(1) && v_src >= 0 && v_src + v_cols <= kv.size(1) && k_off >= 0 &&
             (k_vecs == 0 || (k_vecs - 1) * k_stride + k_off + dims <= k_cols), "rope_cache_write: rotated k entries beyond the row");
  DLIA_CHECK(kcache.dim() == 4 && kcache.is_contiguous() && kcache.size(2) == 32, "rope_cache_write: kcache [blocks, G, 32, dk]");
  const int64_t G = kcache.size(1);
  DLIA_CHECK(G * kcache.size(3) == k_cols, "rope_cache_write: k row does not fill the cache row");
  void* vp = nullptr;
  if (vcache.has_value()) {
    check_act(*vcache, "vcache");
    DLIA_CHECK(vcache->dim() == 4 && vcache->is_contiguous() && vcache->size(0) == kcache.size(0) && vcache->size(1) == G &&
               vcache->size(v_t ? 3 : 2) == 32 && G * vcache->size(v_t ? 2 : 3) == v_cols && vcache->scalar_type() == kcache.scalar_type(),
               "rope_cache_write: vcache [blocks, G, 32, dv] (or [blocks, G, dv, 32]) of the k cache's type");
    vp = vcache->data_ptr();
  } else {
    DLIA_CHECK(v_cols == 0, "rope_cache_write: values without a cache");
  }
  void* qo = nullptr; long ldqo = 0;
  if (q_out.has_value()) {
    check_act(*q_out, "q_out"); check_mat(*q_out, "q_out");
    DLIA_CHECK(q_out->size(0) >= T && q_out->size(1) >= q_cols && q_out->scalar_type() == kcache.scalar_type(), "rope_cache_write: q_out [T, q_cols] of the cache's type");
    qo = q_out->data_ptr(); ldqo = q_out->stride(0);
  }
  const float *cp = nullptr, *sp = nullptr; int table_pos = 0;
  if (dims > 0) {
    DLIA_CHECK(cos_t.has_value() && sin_t.has_value(), "rope_cache_write: rotation needs its tables");
    check_f32(*cos_t, "cos"); check_f32(*sin_t, "sin");
    DLIA_CHECK(cos_t->dim() == 2 && cos_t->size(1) == dims / 2 && sin_t->sizes() == cos_t->sizes(), "rope_cache_write: tables [positions, dims / 2]");
    cp = cos_t->data_ptr<float>(); sp = sin_t->data_ptr<float>(); table_pos = (int)cos_t->size(0);
  }
  dlia_rope_cache_write(q.data_ptr<float>(), q.stride(0), (int)q_vecs, (int)q_stride, (int)q_off, qo, ldqo, (int)q_cols,
                        kv.data_ptr<float>(), kv.stride(0), (int)k_cols, (int)k_vecs, (int)k_stride, (int)k_off, (int)v_src, (int)v_cols,
                        v_t ? 1 : 0, kcache.data_ptr(), vp, is_f32(kcache), (int)G, (int)dims, interleaved ? 1 : 0, cp, sp, table_pos,
                        tok_pos.data_ptr<int>(), tok_seq.data_ptr<int>(), block_table.data_ptr<int>(), (int)T, (int)block_table.size(1),
                        (int)kcache.size(0), (int)block_table.size(0), cur_stream());
}

// out [T, H * dv]; q [T, .] fp32, head h at columns h * q_head (maps * d entries); keys: rows of kcache [blocks, G, 32, k_row], map a
// at entries [a * d, (a + 1) * d); values: entries [v_off, v_off + dv) of the rows of vcache [blocks, G, 32, v_row] (may be kcache).
void multi_attention(Tensor out, const Tensor& q, int64_t q_head, const Tensor& kcache, const Tensor& vcache, int64_t v_off,
                     const Tensor& tok_pos, const Tensor& tok_seq, const Tensor& block_table, int64_t H, int64_t d, int64_t dv,
                     int64_t maps, double scale, int64_t window, int64_t keep_first, double softcap, double lam, double post, double eps,
                     OptTensor gate, int64_t chunk, OptTensor sink) {
  DLIA_ON_DEVICE_OF(out);
  check_act(out, "out"); check_mat(out, "out"); check_fmat(q, "q"); check_act(kcache, "kcache"); check_act(vcache, "vcache");
  check_i32(tok_pos, "tok_pos"); check_i32(tok_seq, "tok_seq"); check_i32(block_table, "block_table");
  const int64_t T = out.size(0);
  DLIA_CHECK(kcache.dim() == 4 && vcache.dim() == 4 && kcache.is_contiguous() && vcache.is_contiguous() && kcache.size(2) == 32 &&
             vcache.size(2) == 32 && kcache.size(0) == vcache.size(0) &&
             kcache.scalar_type() == vcache.scalar_type() && out.scalar_type() == kcache.scalar_type(), "multi_attention: caches [blocks, G, 32, row], output in their type");
  // (the key cache may hold fewer heads than the value cache: one row of all key heads for queries that carry a mix of heads)
  const int64_t G = vcache.size(1), Gk = kcache.size(1), k_row = kcache.size(3), v_row = vcache.size(3);
  DLIA_CHECK(Gk >= 1 && H % Gk == 0 && chunk >= 0 && (chunk == 0 || keep_first == 0), "multi_attention: key heads divide the heads; a chunked mask keeps no first tokens");
  DLIA_CHECK((maps == 1 || maps == 2) && d >= 1 && maps * d <= 1024 && maps * d <= k_row && dv >= 1 && dv <= 512 && v_off >= 0 &&
             v_off + dv <= v_row, "multi_attention: 1 or 2 maps, maps * d <= 1024 inside the key row, dv <= 512 inside the value row");
  DLIA_CHECK(H >= 1 && G >= 1 && H % G == 0 && out.size(1) == H * dv && q.size(0) >= T && q_head >= maps * d &&
             (H - 1) * q_head + maps * d <= q.size(1), "multi_attention: head geometry");
  DLIA_CHECK(tok_pos.numel() >= T && tok_seq.numel() >= T && block_table.dim() == 2 && window >= 0 && keep_first >= 0, "multi_attention: metadata");
  const float* gp = nullptr; long ldg = 0;
  if (gate.has_value()) {
    check_fmat(*gate, "gate");
    DLIA_CHECK(gate->size(0) >= T && gate->size(1) == H * dv, "multi_attention: gate [T, H * dv]");
    gp = gate->data_ptr<float>(); ldg = gate->stride(0);
  }
  dlia_multi_attention(out.data_ptr(), out.stride(0), q.data_ptr<float>(), q.stride(0), (int)q_head, kcache.data_ptr(), (int)k_row,
                       vcache.data_ptr(), (int)v_row, (int)v_off, is_f32(kcache), tok_pos.data_ptr<int>(), tok_seq.data_ptr<int>(),
                       block_table.data_ptr<int>(), (int)T, (int)block_table.size(1), (int)kcache.size(0), (int)block_table.size(0),
                       (int)H, (int)G, (int)d, (int)dv, (int)maps, (float)scale, (int)window, (int)keep_first, (float)softcap,
                       (float)lam, (float)post, (float)eps, gp, ldg, (int)Gk, (int)chunk, opt_f32(sink, H, "sink"), cur_stream());
}

// The same attention on the matrix cores: bf16, q [T, .] bf16, values key-contiguous in vt [blocks, G, dv, 32]; per sequence
// (q_start, ctx, slots) in tiles of 16 tokens.
void tile_attention(Tensor out, const Tensor& q, int64_t q_head, const Tensor& kcache, const Tensor& vt, const Tensor& q_start,
                    const Tensor& ctx, const Tensor& slots, const Tensor& block_table, int64_t max_q, int64_t H, int64_t d, int64_t dv,
                    int64_t maps, double scale, int64_t window, int64_t keep_first, double softcap, double lam, double post, double eps,
                    OptTensor gate, const std::optional<Tensor>& part, int64_t chunk, OptTensor sink) {
  DLIA_ON_DEVICE_OF(out);
  check_mat(out, "out"); check_mat(q, "q");
  check_i32(q_start, "q_start"); check_i32(ctx, "ctx"); check_i32(slots, "slots"); check_i32(block_table, "block_table");
  DLIA_CHECK(out.is_cuda() && q.is_cuda() && kcache.is_cuda() && vt.is_cuda() && out.scalar_type() == at::kBFloat16 &&
             q.scalar_type() == at::kBFloat16 && kcache.scalar_type() == at::kBFloat16 && vt.scalar_type() == at::kBFloat16,
             "tile_attention: bfloat16 on the GPU");
  const int64_t T = out.size(0), B = ctx.numel();
  DLIA_CHECK(kcache.dim() == 4 && vt.dim() == 4 && kcache.is_contiguous() && vt.is_contiguous() && kcache.size(2) == 32 && vt.size(3) == 32 &&
             kcache.size(0) == vt.size(0) && (kcache.size(1) == vt.size(1) || kcache.size(1) == 1) && vt.size(2) == dv,
             "tile_attention: kcache [blocks, G or 1, 32, row], vt [blocks, G, dv, 32]");
  const int64_t G = vt.size(1), Gk = kcache.size(1), k_row = kcache.size(3);
  DLIA_CHECK(chunk >= 0 && (chunk == 0 || keep_first == 0), "tile_attention: a chunked mask keeps no first tokens");
  DLIA_CHECK((maps == 1 || maps == 2) && d >= 8 && maps * d <= k_row && H >= 1 && H % G == 0 && out.size(1) == H * dv && q.size(0) >= T &&
             q_head >= maps * d && (H - 1) * q_head + maps * d <= q.size(1), "tile_attention: head geometry");
  DLIA_CHECK(q_start.numel() >= B + 1 && slots.numel() >= B && block_table.dim() == 2 && max_q >= 0 && max_q <= T && window >= 0 && keep_first >= 0,
             "tile_attention: metadata");
  const float* gp = nullptr; long ldg = 0;
  if (gate.has_value()) {
    check_fmat(*gate, "gate");
    DLIA_CHECK(gate->size(0) >= T && gate->size(1) == H * dv, "tile_attention: gate [T, H * dv]");
    gp = gate->data_ptr<float>(); ldg = gate->stride(0);
  }
  float* pp = nullptr; long pn = 0;
  if (part.has_value()) { check_f32(*part, "part"); pp = part->data_ptr<float>(); pn = part->numel(); }
  DLIA_CHECK(max_q != 1 || T == B, "tile_attention: a single-token step has one row per sequence");
  const int rc = dlia_tile_attention(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), (int)q_head, kcache.data_ptr(), (int)k_row,
                                     vt.data_ptr(), q_start.data_ptr<int>(), ctx.data_ptr<int>(), slots.data_ptr<int>(), block_table.data_ptr<int>(),
                                     (int)B, (int)max_q, (int)block_table.size(1), (int)kcache.size(0), (int)block_table.size(0), (int)H, (int)G,
                                     (int)d, (int)dv, (int)maps, (float)scale, (int)window, (int)keep_first, (float)softcap, (float)lam,
                                     (float)post, (float)eps, gp, ldg, pp, pn, (int)Gk, (int)chunk, opt_f32(sink, H, "sink"), cur_stream());
  DLIA_CHECK(rc != 2, "tile_attention: a single-token step needs the workspace for its key splits (tile_attention_part_floats)");
  DLIA_CHECK(rc == 0, "tile_attention: sizes must be multiples of 8 (d, key row, q head stride, q row), maps * d <= 1024, dv <= 512");
}

int64_t rglru_scan_ws_floats(int64_t rows, int64_t B, int64_t W) { return dlia_rglru_scan_ws_floats((int)rows, (int)B, (int)W); }

int64_t tile_attention_part_floats(int64_t B, int64_t H, int64_t G, int64_t dv, int64_t maps, int64_t Gk) {
  // (Gk: heads of the key cache when they are fewer than the value heads G; 0: the same)
  const int g = Gk > 0 ? dlia_tile_attention_tile_groups((int)G, (int)Gk) : (int)G;
  return B * H * maps * dlia_tile_attention_splits((int)B, (int)H, g) * (dv + 2);
}

// out [T, W] = S_t * gelu_tanh(ypre); u [T, W] conv output, gates [T, blocks * 2 bw] (per block: the decay gate's bw logits, then
// the input gate's), clam [W] = c softplus(lam), state [slots, W].
void rglru_scan(Tensor out, const Tensor& u, const Tensor& gates, const Tensor& ypre, const Tensor& clam, Tensor state,
                const Tensor& q_start, const Tensor& ctx, const Tensor& slots, int64_t bw, int64_t max_q, const std::optional<Tensor>& ws) {
  DLIA_ON_DEVICE_OF(out);
  check_act(out, "out"); check_mat(out, "out"); check_fmat(u, "u"); check_fmat(gates, "gates"); check_fmat(ypre, "ypre");
  check_f32(clam, "clam"); check_f32(state, "state"); check_i32(q_start, "q_start"); check_i32(ctx, "ctx"); check_i32(slots, "slots");
  const int64_t T = out.size(0), W = out.size(1), B = ctx.numel();
  DLIA_CHECK(bw >= 1 && W % bw == 0 && u.size(0) >= T && u.size(1) == W && gates.size(0) >= T && gates.size(1) == 2 * W &&
             ypre.size(0) >= T && ypre.size(1) == W && clam.numel() == W, "rglru_scan: u, ypre [T, W], gates [T, 2 W], clam [W]");
  DLIA_CHECK(state.dim() == 2 && state.size(1) == W && q_start.numel() >= B + 1 && slots.numel() >= B && max_q <= T, "rglru_scan: state [slots, W], q_start [B + 1]");
  if (ws.has_value()) check_f32(*ws, "ws");
  dlia_rglru_scan(out.data_ptr(), is_f32(out), out.stride(0), u.data_ptr<float>(), u.stride(0), gates.data_ptr<float>(), gates.stride(0),
                  ypre.data_ptr<float>(), ypre.stride(0), clam.data_ptr<float>(), state.data_ptr<float>(), q_start.data_ptr<int>(),
                  ctx.data_ptr<int>(), slots.data_ptr<int>(), (int)B, (int)max_q, (int)W, (int)bw, (int)state.size(0),
                  ws.has_value() ? ws->data_ptr<float>() : nullptr, ws.has_value() ? (long)ws->numel() : 0, (int)T, cur_stream());
}

void xielu(Tensor act, const Tensor& z, const Tensor& pq) {
  DLIA_ON_DEVICE_OF(act);
  check_act(act, "act"); check_mat(act, "act"); check_fmat(z, "z"); check_f32(pq, "pq");
  DLIA_CHECK(z.size(0) >= act.size(0) && z.size(1) >= act.size(1) && pq.numel() == 2, "xielu: z [M, >= F], act [M, F], two numbers");
  dlia_xielu(act.data_ptr(), is_f32(act), z.data_ptr<float>(), (int)act.size(0), (int)act.size(1), z.stride(0), act.stride(0),
             pq.data_ptr<float>(), cur_stream());
}

void scale_rows(Tensor x, int64_t cols, double s) {
  DLIA_ON_DEVICE_OF(x);
  check_fmat(x, "x");
  DLIA_CHECK(cols >= 0 && cols <= x.size(1), "scale_rows: columns");
  dlia_scale_rows(x.data_ptr<float>(), (int)x.size(0), (int)cols, x.stride(0), (float)s, cur_stream());
}

// out[:, b * n_out : (b + 1) * n_out] (row stride of out) = x[:, b * x_step : b * x_step + n_in] . w[b]^T + bias[b]
void gemm_blocks(Tensor out, const Tensor& x, const Tensor& w, OptTensor bias, int64_t x_step, int64_t out_step) {
  DLIA_ON_DEVICE_OF(out);
  check_act(out, "out"); check_act(x, "x"); check_act(w, "w"); check_mat(out, "out"); check_mat(x, "x");
  DLIA_CHECK(w.dim() == 3 && w.is_contiguous() && x.scalar_type() == w.scalar_type(), "gemm_blocks: w [blocks, n_out, n_in] of x's type");
  DLIA_CHECK(is_f32(out) || !is_f32(x), "gemm_blocks: fp32 operands give fp32 output");
  const int64_t M = x.size(0), nb = w.size(0), N = w.size(1), K = w.size(2);
  DLIA_CHECK(out.size(0) >= M && x_step >= 0 && out_step >= 0 && (nb - 1) * x_step + K <= x.size(1) && (nb - 1) * out_step + N <= out.size(1) &&
             (out_step >= N || nb == 1), "gemm_blocks: blocks beyond the rows");
  dlia_gemm_blocks(out.data_ptr(), is_f32(out), x.data_ptr(), w.data_ptr(), is_f32(x), opt_f32(bias, nb * N, "bias"), (int)M, (int)N, (int)K,
                   x.stride(0), K, out.stride(0), (int)nb, x_step, N * K, out_step, cur_stream());
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(dlia, m) {
  m.def("par_norm(Tensor(a!)? out, Tensor(b!) out32, Tensor(c!) x, Tensor? ya, Tensor? yb, Tensor? ls1, Tensor? ls2, Tensor? w, Tensor(d!)? carry, Tensor tok_seq, float eps) -> ()");
  m.def("token_shift(Tensor(a!) out, Tensor n32, Tensor carry, Tensor mu, Tensor tok_pos, Tensor tok_seq) -> ()");
  m.def("rope_cache_write(Tensor(a!) q, int q_vecs, int q_stride, int q_off, Tensor(b!)? q_out, int q_cols, Tensor(c!) kv, int k_cols, int k_vecs, int k_stride, int k_off, int v_src, int v_cols, bool v_t, Tensor(d!) kcache, Tensor(e!)? vcache, int dims, bool interleaved, Tensor? cos_t, Tensor? sin_t, Tensor tok_pos, Tensor tok_seq, Tensor block_table) -> ()");
  m.def("multi_attention(Tensor(a!) out, Tensor q, int q_head, Tensor kcache, Tensor vcache, int v_off, Tensor tok_pos, Tensor tok_seq, Tensor block_table, int H, int d, int dv, int maps, float scale, int window, int keep_first, float softcap, float lam, float post, float eps, Tensor? gate, int chunk=0, Tensor? sink=None) -> ()");
  m.def("tile_attention(Tensor(a!) out, Tensor q, int q_head, Tensor kcache, Tensor vt, Tensor q_start, Tensor ctx, Tensor slots, Tensor block_table, int max_q, int H, int d, int dv, int maps, float scale, int window, int keep_first, float softcap, float lam, float post, float eps, Tensor? gate, Tensor(b!)? part, int chunk=0, Tensor? sink=None) -> ()");
  m.def("tile_attention_part_floats(int B, int H, int G, int dv, int maps, int Gk=0) -> int");
  m.def("rglru_scan(Tensor(a!) out, Tensor u, Tensor gates, Tensor ypre, Tensor clam, Tensor(b!) state, Tensor q_start, Tensor ctx, Tensor slots, int bw, int max_q, Tensor(c!)? ws) -> ()");
  m.def("rglru_scan_ws_floats(int rows, int B, int W) -> int");
  m.def("xielu(Tensor(a!) act, Tensor z, Tensor pq) -> ()");
  m.def("scale_rows(Tensor(a!) x, int cols, float s) -> ()");
  m.def("gemm_blocks(Tensor(a!) out, Tensor x, Tensor w, Tensor? bias, int x_step, int out_step) -> ()");
}

TORCH_LIBRARY_IMPL(dlia, CUDA, m) {
  m.impl("par_norm", &par_norm);
  m.impl("token_shift", &token_shift);
  m.impl("rope_cache_write", &rope_cache_write);
  m.impl("multi_attention", &multi_attention);
  m.impl("tile_attention", &tile_attention);
  m.impl("rglru_scan", &rglru_scan);
  m.impl("xielu", &xielu);
  m.impl("scale_rows", &scale_rows);
  m.impl("gemm_blocks", &gemm_blocks);
}

TORCH_LIBRARY_IMPL(dlia, CompositeExplicitAutograd, m) {
  m.impl("tile_attention_part_floats", &tile_attention_part_floats);
  m.impl("rglru_scan_ws_floats", &rglru_scan_ws_floats);
}
