// Row kernels of stacks with dynamic-tanh norms and gated residuals; the residual stream is fp32.
//
//   embed_pos32     x[t] = table[ids[t]] + ptable[pos[t]]                          (learned positions)
//   dyt_gate        x += sigmoid(gl + gb) * y;  x += step;  out = tanh(alpha x) w + b     one workgroup per row, one launch
//                   for a sublayer's gated residual add, the vector that opens a pass of a repeated stretch of layers, and the
//                   next sublayer's norm. y is one stream, or the mean of two streams that are RMS-normed over the row first
//                   (y = (rms(ya) wa + rms(yb) wb) / 2). Every part is optional; rows can be gathered for the output.
//   headnorm_gate   per (token, head): v = o / (max(|nq|, em) + 1e-6) when the head's read-out carries its two normaliser
//                   columns [dv | nq | em], then out = v / rms(v) * w[head, :] * sigmoid(gate)
//   unary_act       act = f(x) of an fp32 GEMM output, f the exact GELU x Phi(x) (kind 0) or tanh (kind 1)
//   softcap         logits <- cap tanh(logits / cap), in place
#include "common.h"
#include "launch.h"

namespace dlia {

template <typename TT>
__global__ __launch_bounds__(128) void embed_pos32_kernel(float* __restrict__ out, const int* __restrict__ ids,
                                                          const int* __restrict__ pos, const TT* __restrict__ table,
                                                          const TT* __restrict__ ptable, int H, int vocab, int max_pos) {
  const int t = blockIdx.x;
  int id = ids[t], ps = pos[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // never fault on a bad id or position
  ps = ps < 0 ? 0 : (ps >= max_pos ? max_pos - 1 : ps);
  const TT* a = table + (long)id * H;
  const TT* b = ptable + (long)ps * H;
  float* dst = out + (long)t * H;
  for (int i = threadIdx.x; i < H; i += 128) dst[i] = (float)a[i] + (float)b[i];
}

template <typename OT>
__global__ __launch_bounds__(256) void dyt_gate_kernel(
    OT* __restrict__ out, float* __restrict__ x, const float* __restrict__ ya, const float* __restrict__ yb,
    const float* __restrict__ wa, const float* __restrict__ wb, const float* __restrict__ gl, const float* __restrict__ gb,
    const float* __restrict__ step, const float* __restrict__ nw, const float* __restrict__ nb, const int* __restrict__ row_idx,
    int H, long ldx, long ldy, long ldg, long ldo, float alpha, float eps) {
  __shared__ float scratch[16];
  const int orow = blockIdx.x;
  const long irow = row_idx ? row_idx[orow] : orow;
  float* xr = x + irow * ldx;
  if (ya) {
    const float* ar = ya + irow * ldy;
    const float* br = yb ? yb + irow * ldy : nullptr;
    float ra = 1.f, rb = 1.f;
    if (br) {
      float sa = 0.f, sb = 0.f;
      for (int i = threadIdx.x; i < H; i += 256) { const float a = ar[i], b = br[i]; sa += a * a; sb += b * b; }
      sa = block_sum(sa, scratch);
      sb = block_sum(sb, scratch);
      ra = rsqrtf(sa / H + eps); rb = rsqrtf(sb / H + eps);
    }
    const float* gr = gl ? gl + irow * ldg : nullptr;
    for (int i = threadIdx.x; i < H; i += 256) {
      float y = br ? 0.5f * (ar[i] * ra * wa[i] + br[i] * rb * wb[i]) : ar[i];
      if (gr) y *= 1.f / (1.f + expf(-(gr[i] + gb[i])));
      xr[i] += y;
    }
  }
  if (step)
    for (int i = threadIdx.x; i < H; i += 256) xr[i] += step[i];
  if (!out) return;
  // (each thread reads back only the elements it wrote itself)
  OT* outr = out + (long)orow * ldo;
  for (int i = threadIdx.x; i < H; i += 256) outr[i] = (OT)(tanhf(alpha * xr[i]) * nw[i] + nb[i]);
}

template <typename OT>
__global__ __launch_bounds__(256) void headnorm_gate_kernel(OT* __restrict__ out, const float* __restrict__ o,
                                                            const float* __restrict__ gate, const float* __restrict__ w,
                                                            int items, int heads, int dv, int extra, long ldo_in, long ldg,
                                                            long ld_out, float eps) {
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int t = item / heads, h = item % heads, lane = lane_id();
  const float* orow = o + (long)t * ldo_in + (long)h * (dv + extra);
  const float* grow = gate + (long)t * ldg + (long)h * dv;
  const float den = extra ? 1.f / (fmaxf(fabsf(orow[dv]), orow[dv + 1]) + 1e-6f) : 1.f;
  float s = 0.f;
  for (int i = lane; i < dv; i += 64) { const float v = orow[i] * den; s += v * v; }
  s = wave_sum(s);
  const float r = rsqrtf(s / dv + eps) * den;
  OT* dst = out + (long)t * ld_out + (long)h * dv;
  for (int i = lane; i < dv; i += 64) dst[i] = (OT)(orow[i] * r * w[h * dv + i] / (1.f + expf(-grow[i])));
}

template <typename OT>
__global__ __launch_bounds__(256) void unary_act_kernel(OT* __restrict__ act, const float* __restrict__ z, long n, int F, long ldz,
                                                        long lda, int kind) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const long m = i / F; const int c = (int)(i % F);
  const float x = z[m * ldz + c];
  // 0: exact GELU, 1: tanh, 2: the square of relu, 3: silu(x) times the entry F columns further (gate | up side by side)
  float y;
  if (kind == 0) y = 0.5f * x * (1.f + erff(x * 0.7071067811865476f));
  else if (kind == 1) y = tanhf(x);
  else if (kind == 2) { const float r = fmaxf(x, 0.f); y = r * r; }
  else y = x / (1.f + expf(-x)) * z[m * ldz + c + F];
  act[m * lda + c] = (OT)y;
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ z, long n, int V, long ld, float cap) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float* p = z + (i / V) * ld + (i % V);
  *p = cap * tanhf(*p / cap);
}

}  // namespace dlia

extern "C" void dlia_embed_pos32(float* out, const int* ids, const int* pos, const void* table, const void* ptable, int f32, int T,
                                 int H, int vocab, int max_pos, hipStream_t stream) {
  if (T <= 0) return;
  if (f32)
    hipLaunchKernelGGL(dlia::embed_pos32_kernel<float>, dim3(T), dim3(128), 0, stream, out, ids, pos, (const float*)table,
                       (const float*)ptable, H, vocab, max_pos);
  else
    hipLaunchKernelGGL(dlia::embed_pos32_kernel<dlia::bf16>, dim3(T), dim3(128), 0, stream, out, ids, pos, (const dlia::bf16*)table,
                       (const dlia::bf16*)ptable, H, vocab, max_pos);
}

extern "C" void dlia_dyt_gate(void* out, int out_f32, float* x, const float* ya, const float* yb, const float* wa, const float* wb,
                              const float* gl, const float* gb, const float* step, const float* nw, const float* nb,
                              const int* row_idx, int rows, int H, long ldx, long ldy, long ldg, long ldo, float alpha, float eps,
                              hipStream_t stream) {
  if (rows <= 0) return;
  if (out_f32 || !out)
    hipLaunchKernelGGL(dlia::dyt_gate_kernel<float>, dim3(rows), dim3(256), 0, stream, (float*)out, x, ya, yb, wa, wb, gl, gb, step,
                       nw, nb, row_idx, H, ldx, ldy, ldg, ldo, alpha, eps);
  else
    hipLaunchKernelGGL(dlia::dyt_gate_kernel<dlia::bf16>, dim3(rows), dim3(256), 0, stream, (dlia::bf16*)out, x, ya, yb, wa, wb, gl,
                       gb, step, nw, nb, row_idx, H, ldx, ldy, ldg, ldo, alpha, eps);
}

extern "C" void dlia_headnorm_gate(void* out, int out_f32, const float* o, const float* gate, const float* w, int T, int heads,
                                   int dv, int extra, long ldo_in, long ldg, long ld_out, float eps, hipStream_t stream) {
  const int items = T * heads;
  if (items <= 0) return;
  if (out_f32)
    hipLaunchKernelGGL(dlia::headnorm_gate_kernel<float>, dim3((items + 3) / 4), dim3(256), 0, stream, (float*)out, o, gate, w, items,
                       heads, dv, extra, ldo_in, ldg, ld_out, eps);
  else
    hipLaunchKernelGGL(dlia::headnorm_gate_kernel<dlia::bf16>, dim3((items + 3) / 4), dim3(256), 0, stream, (dlia::bf16*)out, o, gate,
                       w, items, heads, dv, extra, ldo_in, ldg, ld_out, eps);
}

extern "C" void dlia_unary_act(void* act, int out_f32, const float* z, int M, int F, long ldz, long lda, int kind, hipStream_t stream) {
  const long n = (long)M * F;
  if (n <= 0) return;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (out_f32)
    hipLaunchKernelGGL(dlia::unary_act_kernel<float>, grid, dim3(256), 0, stream, (float*)act, z, n, F, ldz, lda, kind);
  else
    hipLaunchKernelGGL(dlia::unary_act_kernel<dlia::bf16>, grid, dim3(256), 0, stream, (dlia::bf16*)act, z, n, F, ldz, lda, kind);
}

extern "C" void dlia_softcap(float* z, int M, int V, long ld, float cap, hipStream_t stream) {
  const long n = (long)M * V;
  if (n <= 0) return;
  hipLaunchKernelGGL(dlia::softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, z, n, V, ld, cap);
}
