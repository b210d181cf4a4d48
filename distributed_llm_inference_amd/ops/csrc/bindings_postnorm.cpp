// torch custom-op bindings (namespace `dlia`) of the row kernels for stacks that norm their sublayers' outputs only, and of
// the q / k / v preparation of their attention mixers. As everywhere in this library, shapes, types and devices are checked
// on the host before anything is launched.
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

// x += rms(a ya + b yb) w; out = x in out's type. Without ya: only the conversion.
void post_norm_add(const std::optional<Tensor>& out, Tensor x, OptTensor ya, OptTensor yb, double a, double b, OptTensor w, double eps) {
  DLIA_ON_DEVICE_OF(x);
  check_fmat(x, "x");
  const int64_t T = x.size(0), H = x.size(1);
  const float *yap = nullptr, *ybp = nullptr;
  long ldya = 0, ldyb = 0;
  if (ya.has_value()) {
    check_fmat(*ya, "ya");
    DLIA_CHECK(ya->size(0) >= T && ya->size(1) == H && w.has_value(), "post_norm_add: ya [T, H] with the norm's weight");
    yap = ya->data_ptr<float>(); ldya = ya->stride(0);
    if (yb.has_value()) {
      check_fmat(*yb, "yb");
      DLIA_CHECK(yb->size(0) >= T && yb->size(1) == H, "post_norm_add: yb [T, H]");
      ybp = yb->data_ptr<float>(); ldyb = yb->stride(0);
    }
  } else {
    DLIA_CHECK(!yb.has_value(), "post_norm_add: yb without ya");
  }
  void* op = nullptr; long ldo = 0; int of32 = 1;
  if (out.has_value()) {
    check_act(*out, "out"); check_mat(*out, "out");
    DLIA_CHECK(out->size(0) >= T && out->size(1) == H, "post_norm_add: out [T, H]");
    op = out->data_ptr(); ldo = out->stride(0); of32 = is_f32(*out);
  }
  DLIA_CHECK(op || yap, "post_norm_add: nothing to do");
  dlia_post_norm_add(op, of32, ldo, x.data_ptr<float>(), x.stride(0), yap, ldya, ybp, ldyb, (float)a, (float)b, opt_f32(w, H, "w"),
                     (int)T, (int)H, (float)eps, cur_stream());
}

// z [T, >= (H + G) d + G dv] fp32: q | k | v of one token per row. kcache [blocks, Gk, 32, G d / Gk] (Gk = G, or 1 with a mix),
// vcache [blocks, G, 32, dv] or, v_t, [blocks, G, dv, 32]; q_out [T, H d] or, with a mix [H, H], [T, H G d].
void mix_prep(const Tensor& z, int64_t H, int64_t G, int64_t d, int64_t dv, OptTensor qw, OptTensor kw, double eps, int64_t dims,
              OptTensor cos_t, OptTensor sin_t, bool v_unit, OptTensor mix, const std::optional<Tensor>& q_out, Tensor kcache, Tensor vcache,
              bool v_t, const Tensor& tok_pos, const Tensor& tok_seq, const Tensor& block_table) {
  DLIA_ON_DEVICE_OF(kcache);
  check_fmat(z, "z"); check_act(kcache, "kcache"); check_act(vcache, "vcache");
  check_i32(tok_pos, "tok_pos"); check_i32(tok_seq, "tok_seq"); check_i32(block_table, "block_table");
  const int64_t T = z.size(0);
  DLIA_CHECK(H >= 1 && G >= 1 && H % G == 0 && d >= 1 && dv >= 1 && z.size(1) >= (H + G) * d + G * dv, "mix_prep: z holds q | k | v");
  DLIA_CHECK(tok_pos.numel() >= T && tok_seq.numel() >= T && block_table.dim() == 2, "mix_prep: metadata");
  DLIA_CHECK(qw.has_value() == kw.has_value(), "mix_prep: norm weights for q and k together");
  DLIA_CHECK(dims >= 0 && dims % 2 == 0 && dims <= d, "mix_prep: an even number of rotated entries within a head");
  const float *cp = nullptr, *sp = nullptr; int table_pos = 0;
  if (dims > 0) {
    DLIA_CHECK(cos_t.has_value() && sin_t.has_value(), "mix_prep: rotation needs its tables");
    check_f32(*cos_t, "cos"); check_f32(*sin_t, "sin");
    DLIA_CHECK(cos_t->dim() == 2 && cos_t->size(1) == dims / 2 && sin_t->sizes() == cos_t->sizes(), "mix_prep: tables [positions, dims / 2]");
    cp = cos_t->data_ptr<float>(); sp = sin_t->data_ptr<float>(); table_pos = (int)cos_t->size(0);
  }
  DLIA_CHECK(kcache.dim() == 4 && kcache.is_contiguous() && kcache.size(2) == 32, "mix_prep: kcache [blocks, Gk, 32, row]");
  const int64_t Gk = kcache.size(1);
  DLIA_CHECK((Gk == G || Gk == 1) && Gk * kcache.size(3) == G * d, "mix_prep: the k row does not fill the cache row");
  DLIA_CHECK(vcache.dim() == 4 && vcache.is_contiguous() && vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
             vcache.size(v_t ? 3 : 2) == 32 && vcache.size(v_t ? 2 : 3) == dv && vcache.scalar_type() == kcache.scalar_type(),
             "mix_prep: vcache [blocks, G, 32, dv] (or [blocks, G, dv, 32]) of the k cache's type");
  const float* mp = nullptr;
  if (mix.has_value()) {
    check_f32(*mix, "mix");
    DLIA_CHECK(mix->numel() == H * H && Gk == 1, "mix_prep: mix [H, H] goes with one key row for all heads");
    mp = mix->data_ptr<float>();
  }
  void* qo = nullptr; long ldqo = 0; int qf32 = 1;
  if (q_out.has_value()) {
    check_act(*q_out, "q_out"); check_mat(*q_out, "q_out");
    DLIA_CHECK(q_out->size(0) >= T && q_out->size(1) >= (mp ? H * G * d : H * d), "mix_prep: q_out [T, H d] (with a mix [T, H G d])");
    DLIA_CHECK(is_f32(*q_out) || !is_f32(kcache), "mix_prep: a bfloat16 q goes with a bfloat16 cache");
    qo = q_out->data_ptr(); ldqo = q_out->stride(0); qf32 = is_f32(*q_out);
  }
  const int rc = dlia_mix_prep(z.data_ptr<float>(), z.stride(0), (int)T, (int)H, (int)G, (int)d, (int)dv, opt_f32(qw, H * d, "qw"),
                               opt_f32(kw, G * d, "kw"), (float)eps, (int)dims, cp, sp, table_pos, v_unit ? 1 : 0, mp, qo, qf32, ldqo,
                               kcache.data_ptr(), (int)Gk, vcache.data_ptr(), v_t ? 1 : 0, is_f32(kcache), tok_pos.data_ptr<int>(),
                               tok_seq.data_ptr<int>(), block_table.data_ptr<int>(), (int)block_table.size(1), (int)kcache.size(0),
                               (int)block_table.size(0), cur_stream());
  DLIA_CHECK(rc == 0, "mix_prep: q and k of one token and the mix ((H + G) d + H H floats) must fit a workgroup's 64 KiB of LDS");
}

// Attention over scores mixed across heads, for steps with prompt portions: out [T, H dv] bf16, q [T, H d] bf16 (normed and rotated, not
// mixed), kcache [blocks, 1, 32, G d], vt [blocks, G, dv, 32], mix [H, H] fp32 (mix x temperatures x scale), gate [T, H dv] fp32.
int64_t mixed_attention_part_floats(int64_t T, int64_t H, int64_t dv) { return dlia_mixed_attention_part_floats((int)T, (int)H, (int)dv); }

bool mixed_attention_fits(int64_t H, int64_t G, int64_t d, int64_t dv) { return dlia_mixed_attention_fits((int)H, (int)G, (int)d, (int)dv) != 0; }

void mixed_attention(Tensor out, const Tensor& q, const Tensor& kcache, const Tensor& vt, const Tensor& mix, const Tensor& q_start,
                     const Tensor& ctx, const Tensor& slots, const Tensor& block_table, int64_t max_q, int64_t H, int64_t d, int64_t dv,
                     int64_t chunk, OptTensor sink, OptTensor gate, const std::optional<Tensor>& part) {
  DLIA_ON_DEVICE_OF(out);
  check_mat(out, "out"); check_mat(q, "q"); check_f32(mix, "mix");
  check_i32(q_start, "q_start"); check_i32(ctx, "ctx"); check_i32(slots, "slots"); check_i32(block_table, "block_table");
  DLIA_CHECK(out.is_cuda() && q.is_cuda() && kcache.is_cuda() && vt.is_cuda() && out.scalar_type() == at::kBFloat16 &&
             q.scalar_type() == at::kBFloat16 && kcache.scalar_type() == at::kBFloat16 && vt.scalar_type() == at::kBFloat16,
             "mixed_attention: bfloat16 on the GPU");
  const int64_t T = out.size(0), B = ctx.numel();
  DLIA_CHECK(kcache.dim() == 4 && vt.dim() == 4 && kcache.is_contiguous() && vt.is_contiguous() && kcache.size(1) == 1 && kcache.size(2) == 32 &&
             vt.size(3) == 32 && kcache.size(0) == vt.size(0) && vt.size(2) == dv, "mixed_attention: kcache [blocks, 1, 32, G d], vt [blocks, G, dv, 32]");
  const int64_t G = vt.size(1);
  DLIA_CHECK(H >= 1 && G >= 1 && H % G == 0 && kcache.size(3) == G * d && out.size(1) == H * dv && q.size(0) >= T && q.size(1) >= H * d &&
             mix.numel() == H * H, "mixed_attention: head geometry");
  DLIA_CHECK(q_start.numel() >= B + 1 && slots.numel() >= B && block_table.dim() == 2 && max_q >= 0 && max_q <= T && chunk >= 0, "mixed_attention: metadata");
  const float* gp = nullptr; long ldg = 0;
  if (gate.has_value()) {
    check_fmat(*gate, "gate");
    DLIA_CHECK(gate->size(0) >= T && gate->size(1) == H * dv, "mixed_attention: gate [T, H * dv]");
    gp = gate->data_ptr<float>(); ldg = gate->stride(0);
  }
  float* pp = nullptr; long pn = 0;       // (workspace for dealing a tile's key blocks out to several workgroups; without it one each)
  if (part.has_value()) { check_f32(*part, "part"); pp = part->data_ptr<float>(); pn = part->numel(); }
  const int rc = dlia_mixed_attention(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), kcache.data_ptr(), (int)kcache.size(3), vt.data_ptr(),
                                      mix.data_ptr<float>(), q_start.data_ptr<int>(), ctx.data_ptr<int>(), slots.data_ptr<int>(),
                                      block_table.data_ptr<int>(), (int)B, (int)max_q, (int)block_table.size(1), (int)kcache.size(0),
                                      (int)block_table.size(0), (int)H, (int)G, (int)d, (int)dv, (int)chunk, opt_f32(sink, H, "sink"), gp, ldg,
                                      pp, pn, (int)T, cur_stream());
  DLIA_CHECK(rc == 0, "mixed_attention: up to 32 heads, key size a multiple of 8 up to 256, value size up to 128, rows in 16-byte pieces");
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(dlia, m) {
  m.def("mixed_attention_fits(int H, int G, int d, int dv) -> bool");
  m.def("mixed_attention_part_floats(int T, int H, int dv) -> int");
  m.def("mixed_attention(Tensor(a!) out, Tensor q, Tensor kcache, Tensor vt, Tensor mix, Tensor q_start, Tensor ctx, Tensor slots, Tensor block_table, int max_q, int H, int d, int dv, int chunk, Tensor? sink, Tensor? gate, Tensor(b!)? part=None) -> ()");
  m.def("post_norm_add(Tensor(a!)? out, Tensor(b!) x, Tensor? ya, Tensor? yb, float a, float b, Tensor? w, float eps) -> ()");
  m.def("mix_prep(Tensor z, int H, int G, int d, int dv, Tensor? qw, Tensor? kw, float eps, int dims, Tensor? cos_t, Tensor? sin_t, bool v_unit, Tensor? mix, Tensor(a!)? q_out, Tensor(b!) kcache, Tensor(c!) vcache, bool v_t, Tensor tok_pos, Tensor tok_seq, Tensor block_table) -> ()");
}

TORCH_LIBRARY_IMPL(dlia, CUDA, m) {
  m.impl("post_norm_add", &post_norm_add);
  m.impl("mix_prep", &mix_prep);
  m.impl("mixed_attention", &mixed_attention);
}

TORCH_LIBRARY_IMPL(dlia, CompositeExplicitAutograd, m) {
  m.impl("mixed_attention_fits", &mixed_attention_fits);
  m.impl("mixed_attention_part_floats", &mixed_attention_part_floats);
}
