// torch custom-op bindings (namespace `dlia`) of the kernels for stacks with dynamic-tanh norms, gated residuals, linear
// recurrences over a matrix state, attention with learned distance biases, and routed feed-forwards. As everywhere in this
// library, shapes, types and devices are checked on the host before anything is launched.
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

void embed_pos32(Tensor out, const Tensor& ids, const Tensor& pos, const Tensor& table, const Tensor& ptable) {
  DLIA_ON_DEVICE_OF(out);
  check_f32(out, "out"); check_i32(ids, "ids"); check_i32(pos, "pos"); check_act(table, "table"); check_act(ptable, "ptable");
  DLIA_CHECK(out.dim() == 2 && table.dim() == 2 && ptable.dim() == 2 && table.is_contiguous() && ptable.is_contiguous() &&
             table.scalar_type() == ptable.scalar_type() && table.size(1) == out.size(1) && ptable.size(1) == out.size(1),
             "embed_pos32: out [T, H], table [V, H], ptable [P, H] of one type");
  const int64_t T = out.size(0);
  DLIA_CHECK(ids.numel() >= T && pos.numel() >= T, "embed_pos32: ids / pos shorter than the rows");
  dlia_embed_pos32(out.data_ptr<float>(), ids.data_ptr<int>(), pos.data_ptr<int>(), table.data_ptr(), ptable.data_ptr(), is_f32(table),
                   (int)T, (int)out.size(1), (int)table.size(0), (int)ptable.size(0), cur_stream());
}

void dyt_gate(const std::optional<Tensor>& out, Tensor x, OptTensor ya, OptTensor yb, OptTensor wa, OptTensor wb, OptTensor gl,
              OptTensor gb, OptTensor step, OptTensor nw, OptTensor nb, OptTensor row_idx, double alpha, double eps) {
  DLIA_ON_DEVICE_OF(x);
  check_fmat(x, "x");
  const int64_t H = x.size(1);
  int64_t rows = x.size(0);
  const int* ridx = nullptr;
  if (row_idx.has_value()) {
    check_i32(*row_idx, "row_idx");
    DLIA_CHECK(!ya.has_value() && !step.has_value() && out.has_value(), "dyt_gate: gathered rows are only normalised");
    rows = out->size(0);
    DLIA_CHECK(row_idx->numel() >= rows, "dyt_gate: row_idx shorter than the output");
    ridx = row_idx->data_ptr<int>();
  }
  const float *yap = nullptr, *ybp = nullptr, *glp = nullptr;
  long ldy = 0, ldg = 0;
  if (ya.has_value()) {
    check_fmat(*ya, "ya");
    DLIA_CHECK(ya->size(0) >= rows && ya->size(1) == H, "dyt_gate: ya [rows, H]");
    yap = ya->data_ptr<float>(); ldy = ya->stride(0);
    if (yb.has_value()) {
      check_fmat(*yb, "yb");
      DLIA_CHECK(yb->size(0) >= rows && yb->size(1) == H && yb->stride(0) == ldy && wa.has_value() && wb.has_value(),
                 "dyt_gate: yb like ya, with both weights");
      ybp = yb->data_ptr<float>();
    }
    if (gl.has_value()) {
      check_fmat(*gl, "gl");
      DLIA_CHECK(gl->size(0) >= rows && gl->size(1) == H && gb.has_value(), "dyt_gate: gate logits [rows, H] with their bias");
      glp = gl->data_ptr<float>(); ldg = gl->stride(0);
    }
  }
  void* op = nullptr; long ldo = 0; int of32 = 1;
  if (out.has_value()) {
    check_act(*out, "out"); check_mat(*out, "out");
    DLIA_CHECK(out->size(0) >= rows && out->size(1) == H && nw.has_value() && nb.has_value(), "dyt_gate: out [rows, H] with weight and bias");
    op = out->data_ptr(); ldo = out->stride(0); of32 = is_f32(*out);
  }
  DLIA_CHECK(op || yap || step.has_value(), "dyt_gate: nothing to do");
  dlia_dyt_gate(op, of32, x.data_ptr<float>(), yap, ybp, opt_f32(wa, H, "wa"), opt_f32(wb, H, "wb"), glp, opt_f32(gb, H, "gb"),
                opt_f32(step, H, "step"), opt_f32(nw, H, "nw"), opt_f32(nb, H, "nb"), ridx, (int)rows, (int)H, x.stride(0), ldy, ldg,
                ldo, (float)alpha, (float)eps, cur_stream());
}

void headnorm_gate(Tensor out, const Tensor& o, const Tensor& gate, const Tensor& w, int64_t heads, int64_t dv, int64_t extra, double eps) {
  DLIA_ON_DEVICE_OF(out);
  check_act(out, "out"); check_mat(out, "out"); check_fmat(o, "o"); check_fmat(gate, "gate"); check_f32(w, "w");
  const int64_t T = out.size(0);
  DLIA_CHECK(extra == 0 || extra == 2, "headnorm_gate: 0 or 2 normaliser columns per head");
  DLIA_CHECK(o.size(0) >= T && gate.size(0) >= T && out.size(1) == heads * dv && o.size(1) == heads * (dv + extra) &&
             gate.size(1) == heads * dv && w.numel() == heads * dv, "headnorm_gate: shapes");
  dlia_headnorm_gate(out.data_ptr(), is_f32(out), o.data_ptr<float>(), gate.data_ptr<float>(), w.data_ptr<float>(), (int)T, (int)heads,
                     (int)dv, (int)extra, o.stride(0), gate.stride(0), out.stride(0), (float)eps, cur_stream());
}

void unary_act(Tensor act, const Tensor& z, int64_t kind) {
  DLIA_ON_DEVICE_OF(act);
  check_act(act, "act"); check_mat(act, "act"); check_fmat(z, "z");
  DLIA_CHECK(kind >= 0 && kind <= 3 && z.size(0) >= act.size(0) && z.size(1) == (kind == 3 ? 2 : 1) * act.size(1),
             "unary_act: act [M, F] from z [M, F] (kinds 0 to 2) or from gate | up in z [M, 2 F] (kind 3)");
  dlia_unary_act(act.data_ptr(), is_f32(act), z.data_ptr<float>(), (int)act.size(0), (int)act.size(1), z.stride(0), act.stride(0), (int)kind,
                 cur_stream());
}

void softcap(Tensor logits, int64_t vocab, double cap) {
  DLIA_ON_DEVICE_OF(logits);
  check_fmat(logits, "logits");
  DLIA_CHECK(vocab >= 1 && vocab <= logits.size(1) && cap > 0, "softcap: vocab within the row, cap > 0");
  dlia_softcap(logits.data_ptr<float>(), (int)logits.size(0), (int)vocab, logits.stride(0), (float)cap, cur_stream());
}

void biased_attention(Tensor out, const Tensor& qkv, const Tensor& kcache, const Tensor& vcache, const Tensor& tok_pos,
                      const Tensor& tok_seq, const Tensor& block_table, int64_t H, int64_t G, int64_t d, int64_t dv, double scale,
                      OptTensor temp, OptTensor bias, OptTensor sink, OptTensor gate) {
  DLIA_ON_DEVICE_OF(out);
  check_act(out, "out"); check_mat(out, "out"); check_fmat(qkv, "qkv");
  const int64_t T = out.size(0);
  DLIA_CHECK(G >= 1 && H % G == 0 && qkv.size(0) >= T && qkv.size(1) >= H * d && out.size(1) == H * dv, "biased_attention: shapes");
  check_act(kcache, "kcache"); check_act(vcache, "vcache");
  DLIA_CHECK(kcache.scalar_type() == vcache.scalar_type() && kcache.is_contiguous() && vcache.is_contiguous() &&
             out.scalar_type() == kcache.scalar_type(), "caches and output: one type, contiguous");
  DLIA_CHECK(kcache.dim() == 4 && vcache.dim() == 4 && kcache.size(0) == vcache.size(0) && kcache.size(1) == G && vcache.size(1) == G &&
             kcache.size(2) == 32 && vcache.size(2) == 32 && kcache.size(3) == d && vcache.size(3) == dv, "caches: [blocks, G, 32, d | dv]");
  check_i32(tok_pos, "tok_pos"); check_i32(tok_seq, "tok_seq"); check_i32(block_table, "block_table");
  DLIA_CHECK(tok_pos.numel() >= T && tok_seq.numel() >= T && block_table.dim() == 2, "per-token metadata / block table shape");
  DLIA_CHECK(d >= 1 && d <= 512 && dv >= 1 && dv <= 512, "head sizes 1..512");
  int bias_rows = 0;
  const float* bp = nullptr;
  if (bias.has_value()) {
    check_f32(*bias, "bias");
    DLIA_CHECK(bias->dim() == 2 && bias->size(1) == H && bias->size(0) >= 1, "biased_attention: bias [distances, H]");
    bp = bias->data_ptr<float>(); bias_rows = (int)bias->size(0);
  }
  const float* gp = nullptr; long ldg = 0;
  if (gate.has_value()) {
    check_fmat(*gate, "gate");
    DLIA_CHECK(gate->size(0) >= T && gate->size(1) == H, "biased_attention: gate logits [T, H]");
    gp = gate->data_ptr<float>(); ldg = gate->stride(0);
  }
  dlia_window_attention(out.data_ptr(), qkv.data_ptr<float>(), kcache.data_ptr(), vcache.data_ptr(), is_f32(kcache),
                        tok_pos.data_ptr<int>(), tok_seq.data_ptr<int>(), block_table.data_ptr<int>(), (int)T, (int)block_table.size(1),
                        (int)kcache.size(0), (int)block_table.size(0), (int)H, (int)G, (int)d, (int)dv, qkv.stride(0), out.stride(0),
                        (float)scale, 0, sink.has_value() ? 1 : 0, opt_f32(temp, H, "temp"), bp, bias_rows, opt_f32(sink, H, "sink"),
                        gp, ldg, cur_stream());
}

int64_t state_scan_blocks(int64_t d, int64_t ncols) { return dlia_state_scan_blocks((int)d, (int)ncols); }

void state_scan(int64_t rule, Tensor o, const Tensor& z, OptTensor wz, Tensor state, const std::optional<Tensor>& mstate,
                const Tensor& b0, OptTensor b1, const Tensor& q_start, const Tensor& ctx, const Tensor& slots, int64_t H, int64_t d,
                int64_t dv, int64_t col_q, int64_t col_k, int64_t col_v, int64_t col_a, int64_t col_i, int64_t col_f, double cap,
                double qscale, int64_t max_q, bool quick) {
  DLIA_ON_DEVICE_OF(o);
  check_fmat(o, "o"); check_fmat(z, "z"); check_f32(state, "state"); check_f32(b0, "b0");
  check_i32(q_start, "q_start"); check_i32(ctx, "ctx"); check_i32(slots, "slots");
  DLIA_CHECK(rule == 0 || rule == 1, "state_scan: rule 0 or 1");
  const int64_t B = ctx.numel(), T = o.size(0), ZC = z.size(1);
  DLIA_CHECK(q_start.numel() >= B + 1 && slots.numel() >= B && z.size(0) >= T, "state_scan: q_start [B + 1], ctx [B], slots [B], z [T, .]");
  DLIA_CHECK(H >= 1 && d >= 1 && dv >= 1 && dv <= 4096, "state_scan: sizes");
  auto span = [&](int64_t col, int64_t n) { return col >= 0 && col + n <= ZC; };
  const float* wzp = nullptr; long ldw = 0;
  const float* mp = nullptr;
  if (rule == 0) {
    DLIA_CHECK(d == dv && state.dim() == 4 && state.size(1) == H && state.size(2) == d && state.size(3) == d, "state_scan: state [slots, H, d, d]");
    DLIA_CHECK(o.size(1) == H * d && span(col_q, H * d) && span(col_k, H * d) && span(col_v, H * d) && span(col_a, H * d), "state_scan: columns");
    DLIA_CHECK(wz.has_value() && b1.has_value() && b0.numel() == H * d && b1->numel() == H * d, "state_scan: decay logits and the two bias vectors");
    check_fmat(*wz, "wz"); check_f32(*b1, "b1");
    DLIA_CHECK(wz->size(0) >= T && wz->size(1) == H * d, "state_scan: wz [T, H d]");
    wzp = wz->data_ptr<float>(); ldw = wz->stride(0);
  } else {
    DLIA_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == d && state.size(3) == dv + 1, "state_scan: state [slots, H, d, dv + 1]");
    DLIA_CHECK(o.size(1) == H * (dv + 2) && span(col_q, H * d) && span(col_k, H * d) && span(col_v, H * dv) && span(col_i, H) && span(col_f, H),
               "state_scan: columns");
    DLIA_CHECK(mstate.has_value() && b0.numel() == 2 * H && cap > 0, "state_scan: running maxima, gate biases [2 H], cap > 0");
    check_f32(*mstate, "mstate");
    DLIA_CHECK(mstate->dim() == 3 && mstate->size(0) == state.size(0) && mstate->size(1) == H && mstate->size(2) == 128, "state_scan: mstate [slots, H, 128]");
    mp = mstate->data_ptr<float>();
  }
  const int rc = dlia_state_scan((int)rule, o.data_ptr<float>(), o.stride(0), z.data_ptr<float>(), z.stride(0), wzp, ldw,
                                 state.data_ptr<float>(), const_cast<float*>(mp), b0.data_ptr<float>(),
                                 b1.has_value() ? b1->data_ptr<float>() : nullptr, q_start.data_ptr<int>(), ctx.data_ptr<int>(),
                                 slots.data_ptr<int>(), (int)B, (int)H, (int)d, (int)dv, (int)state.size(0), (int)col_q, (int)col_k,
                                 (int)col_v, (int)col_a, (int)col_i, (int)col_f, (float)cap, (float)qscale, (int)max_q, quick ? 1 : 0, cur_stream());
  DLIA_CHECK(rc == 0, "state_scan: key size ", d, " / value size ", dv, " beyond what the kernel splits (1024 rows, 128 column blocks)");
}

void moe_route(Tensor sel, Tensor wts, const Tensor& logits, int64_t top, int64_t groups, int64_t keep, double scale, OptTensor correction,
               bool softmax, int64_t group_rank, bool renorm) {
  DLIA_ON_DEVICE_OF(sel);
  check_i32(sel, "sel"); check_f32(wts, "wts"); check_fmat(logits, "logits");
  const int64_t T = logits.size(0), E = logits.size(1);
  DLIA_CHECK(E >= 1 && E <= 256 && groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top >= 1 && top <= keep * (E / groups),
             "moe_route: up to 256 experts in equal groups, top within the kept groups");
  DLIA_CHECK(sel.numel() >= T * top && wts.numel() >= T * top && (group_rank == 1 || group_rank == 2), "moe_route: sel / wts [T, top], groups ranked by 1 or 2 members");
  dlia_moe_route(sel.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(), logits.stride(0), (int)T, (int)E, (int)top,
                 (int)groups, (int)keep, (float)scale, opt_f32(correction, E, "correction"), softmax ? 1 : 0, (int)group_rank, renorm ? 1 : 0,
                 cur_stream());
}

void moe_plan(Tensor tiles, Tensor row_tok, Tensor pair_row, const Tensor& sel, int64_t pairs, int64_t top, int64_t E, int64_t tile_rows) {
  DLIA_ON_DEVICE_OF(tiles);
  check_i32(tiles, "tiles"); check_i32(row_tok, "row_tok"); check_i32(pair_row, "pair_row"); check_i32(sel, "sel");
  DLIA_CHECK(tile_rows == 32 || tile_rows == 128, "moe: row tiles of 32 or 128");
  const int64_t max_tiles = (pairs + tile_rows - 1) / tile_rows + E;
  DLIA_CHECK(E >= 1 && E <= 256 && top >= 1 && pairs >= 0 && sel.numel() >= pairs && pair_row.numel() >= pairs, "moe_plan: pairs");
  DLIA_CHECK(tiles.numel() >= 1 + max_tiles && row_tok.numel() >= tile_rows * max_tiles, "moe_plan: room for pairs / tile_rows + E tiles");
  dlia_moe_plan(tiles.data_ptr<int>(), row_tok.data_ptr<int>(), pair_row.data_ptr<int>(), sel.data_ptr<int>(), (int)pairs, (int)top, (int)E,
                (int)(tile_rows * max_tiles), (int)tile_rows, cur_stream());
}

static void check_big(int64_t tile_rows, const Tensor& a, int64_t K, const Tensor& w) {
  DLIA_CHECK(tile_rows == 32 || tile_rows == 128, "moe: row tiles of 32 or 128");
  if (tile_rows == 128)
    DLIA_CHECK(a.scalar_type() == at::kBFloat16 && K % 32 == 0 && a.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(a.data_ptr()) % 16 == 0 &&
               reinterpret_cast<uintptr_t>(w.data_ptr()) % 16 == 0, "moe: 128-row tiles need bf16, K a multiple of 32 and 16-byte aligned rows");
}

void moe_up(Tensor act, const Tensor& x, const Tensor& wg, const Tensor& wu, const Tensor& tiles, const Tensor& row_tok, int64_t max_tiles,
            double limit, int64_t tile_rows) {
  DLIA_ON_DEVICE_OF(act);
  check_act(act, "act"); check_mat(act, "act"); check_act(x, "x"); check_mat(x, "x"); check_act(wg, "wg"); check_act(wu, "wu");
  check_i32(tiles, "tiles"); check_i32(row_tok, "row_tok");
  DLIA_CHECK(wg.dim() == 3 && wg.is_contiguous() && wu.is_contiguous() && wu.sizes() == wg.sizes() && wg.size(2) == x.size(1) &&
             x.scalar_type() == wg.scalar_type() && wu.scalar_type() == wg.scalar_type() && act.scalar_type() == x.scalar_type(),
             "moe_up: x [T, K], wg / wu [E, F, K], one type");
  check_big(tile_rows, x, x.size(1), wg);
  DLIA_CHECK(act.size(1) == wg.size(1) && act.size(0) >= tile_rows * max_tiles && row_tok.numel() >= tile_rows * max_tiles && tiles.numel() >= 1 + max_tiles,
             "moe_up: act [tile_rows max_tiles, F]");
  dlia_moe_up(act.data_ptr(), x.data_ptr(), wg.data_ptr(), wu.data_ptr(), is_f32(x), tiles.data_ptr<int>(), row_tok.data_ptr<int>(),
              (int)max_tiles, x.size(0) > 256 ? 1 : 0, (int)wg.size(1), (int)wg.size(2), x.stride(0), act.stride(0), (float)limit, (int)tile_rows, cur_stream());
}

void moe_down(Tensor y, const Tensor& act, const Tensor& wd, const Tensor& tiles, const Tensor& row_tok, int64_t max_tiles, int64_t tile_rows) {
  DLIA_ON_DEVICE_OF(y);
  check_f32(y, "y"); check_act(act, "act"); check_mat(act, "act"); check_act(wd, "wd"); check_i32(tiles, "tiles"); check_i32(row_tok, "row_tok");
  DLIA_CHECK(wd.dim() == 3 && wd.is_contiguous() && wd.size(2) == act.size(1) && wd.scalar_type() == act.scalar_type(), "moe_down: wd [E, H, F]");
  check_big(tile_rows, act, act.size(1), wd);
  DLIA_CHECK(y.dim() == 2 && y.size(1) == wd.size(1) && y.size(0) >= tile_rows * max_tiles && act.size(0) >= tile_rows * max_tiles &&
             row_tok.numel() >= tile_rows * max_tiles && tiles.numel() >= 1 + max_tiles, "moe_down: y [tile_rows max_tiles, H]");
  dlia_moe_down(y.data_ptr<float>(), act.data_ptr(), wd.data_ptr(), is_f32(act), tiles.data_ptr<int>(), row_tok.data_ptr<int>(),
                (int)max_tiles, max_tiles > 64 ? 1 : 0, (int)wd.size(1), (int)wd.size(2), act.stride(0), (int)tile_rows, cur_stream());
}

void moe_combine(Tensor out, const Tensor& y, const Tensor& pair_row, const Tensor& wts, int64_t top, OptTensor x) {
  DLIA_ON_DEVICE_OF(out);
  check_fmat(out, "out"); check_f32(y, "y"); check_i32(pair_row, "pair_row"); check_f32(wts, "wts");
  const int64_t T = out.size(0), H = out.size(1);
  DLIA_CHECK(y.dim() == 2 && y.size(1) == H && pair_row.numel() >= T * top && wts.numel() >= T * top, "moe_combine: shapes");
  const float* xp = nullptr; long ldx = 0;
  if (x.has_value()) {      // what a choice without a row (an identity expert) returns
    check_fmat(*x, "x");
    DLIA_CHECK(x->size(0) >= T && x->size(1) == H, "moe_combine: x [T, H]");
    xp = x->data_ptr<float>(); ldx = x->stride(0);
  }
  dlia_moe_combine(out.data_ptr<float>(), y.data_ptr<float>(), pair_row.data_ptr<int>(), wts.data_ptr<float>(), (int)T, (int)H, (int)top,
                   out.stride(0), xp, ldx, cur_stream());
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(dlia, m) {
  m.def("embed_pos32(Tensor(a!) out, Tensor ids, Tensor pos, Tensor table, Tensor ptable) -> ()");
  m.def("dyt_gate(Tensor(a!)? out, Tensor(b!) x, Tensor? ya, Tensor? yb, Tensor? wa, Tensor? wb, Tensor? gl, Tensor? gb, Tensor? step, Tensor? nw, Tensor? nb, Tensor? row_idx, float alpha, float eps) -> ()");
  m.def("headnorm_gate(Tensor(a!) out, Tensor o, Tensor gate, Tensor w, int heads, int dv, int extra, float eps) -> ()");
  m.def("unary_act(Tensor(a!) act, Tensor z, int kind) -> ()");
  m.def("softcap(Tensor(a!) logits, int vocab, float cap) -> ()");
  m.def("biased_attention(Tensor(a!) out, Tensor qkv, Tensor kcache, Tensor vcache, Tensor tok_pos, Tensor tok_seq, Tensor block_table, int H, int G, int d, int dv, float scale, Tensor? temp, Tensor? bias, Tensor? sink, Tensor? gate) -> ()");
  m.def("state_scan_blocks(int d, int ncols) -> int");
  m.def("state_scan(int rule, Tensor(a!) o, Tensor z, Tensor? wz, Tensor(b!) state, Tensor(c!)? mstate, Tensor b0, Tensor? b1, Tensor q_start, Tensor ctx, Tensor slots, int H, int d, int dv, int col_q, int col_k, int col_v, int col_a, int col_i, int col_f, float cap, float qscale, int max_q, bool quick) -> ()");
  m.def("moe_route(Tensor(a!) sel, Tensor(b!) wts, Tensor logits, int top, int groups, int keep, float scale, Tensor? correction=None, bool softmax=False, int group_rank=2, bool renorm=True) -> ()");
  m.def("moe_plan(Tensor(a!) tiles, Tensor(b!) row_tok, Tensor(c!) pair_row, Tensor sel, int pairs, int top, int E, int tile_rows) -> ()");
  m.def("moe_up(Tensor(a!) act, Tensor x, Tensor wg, Tensor wu, Tensor tiles, Tensor row_tok, int max_tiles, float limit, int tile_rows) -> ()");
  m.def("moe_down(Tensor(a!) y, Tensor act, Tensor wd, Tensor tiles, Tensor row_tok, int max_tiles, int tile_rows) -> ()");
  m.def("moe_combine(Tensor(a!) out, Tensor y, Tensor pair_row, Tensor wts, int top, Tensor? x=None) -> ()");
}

TORCH_LIBRARY_IMPL(dlia, CUDA, m) {
  m.impl("embed_pos32", &embed_pos32);
  m.impl("dyt_gate", &dyt_gate);
  m.impl("headnorm_gate", &headnorm_gate);
  m.impl("unary_act", &unary_act);
  m.impl("softcap", &softcap);
  m.impl("biased_attention", &biased_attention);
  m.impl("state_scan", &state_scan);
  m.impl("moe_route", &moe_route);
  m.impl("moe_plan", &moe_plan);
  m.impl("moe_up", &moe_up);
  m.impl("moe_down", &moe_down);
  m.impl("moe_combine", &moe_combine);
}

TORCH_LIBRARY_IMPL(dlia, CompositeExplicitAutograd, m) {
  m.impl("state_scan_blocks", &state_scan_blocks);
}
