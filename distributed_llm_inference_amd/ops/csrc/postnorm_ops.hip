// Row kernels of stacks whose sublayers read the fp32 residual stream itself and are normed on their OUTPUT only,
//     x <- x + rms(a * ya + b * yb) w,
// and the preparation of an attention mixer's q, k, v between its input projection and the cache.
//
//   post_norm_add   one launch per sublayer boundary: the weighted sum of one or two sublayer outputs is RMS-normed over the
//                   row, scaled by the norm's weight and added to the stream; the stream leaves in the GEMMs' input type
//                   for the next sublayer (the role residual + RMSNorm has for the Llama path). Without outputs it only
//                   converts the stream (the embedding ahead of the first layer).
//   mix_prep        per token, on the fp32 output q | k | v of the input projection: RMS norm of q and of k over the WHOLE
//                   projection (all heads at once, a weight per entry), rotation of the first `dims` entries of every head by
//                   the token's position (pairs (i, i + dims / 2), angles from a table), every value head divided by its root
//                   mean square; k and v rows go to the paged cache, q leaves for the attention kernel. With a head-mixing
//                   matrix M [H, H] (scores of head h are sum_g M[h, g] q_g . k) the mix is carried by the query: q leaves
//                   as H rows of G * d entries, row h holding for every key head c the sum over the heads g of c's group of
//                   M[h, g] q_g, and the keys of all G heads are ONE cache row of G * d entries that every head reads.
// Norm statistics, rotation and the mix are fp32; outputs take the GEMMs' / the cache's type (bf16 or fp32).
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kPostBlock = 32;       // tokens per cache block
constexpr int kPostThreads = 256;

template <typename OT>
__global__ __launch_bounds__(kPostThreads) void post_norm_add_kernel(
    OT* __restrict__ out, long ldo, float* __restrict__ x, long ldx, const float* __restrict__ ya, long ldya,
    const float* __restrict__ yb, long ldyb, float a, float b, const float* __restrict__ w, int H, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (long)t * ldx;
  if (ya) {
    const float* ar = ya + (long)t * ldya;
    const float* br = yb ? yb + (long)t * ldyb : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += kPostThreads) {
      const float y = br ? a * ar[i] + b * br[i] : a * ar[i];
      ss += y * y;
    }
    ss = block_sum(ss, scratch);
    const float r = 1.f / sqrtf(ss / H + eps);
    for (int i = threadIdx.x; i < H; i += kPostThreads) {
      const float y = br ? a * ar[i] + b * br[i] : a * ar[i];
      xr[i] += y * r * w[i];
    }
  }
  if (!out) return;
  OT* orow = out + (long)t * ldo;       // (each thread re-reads what it wrote itself)
  for (int i = threadIdx.x; i < H; i += kPostThreads) orow[i] = (OT)xr[i];
}

template <typename T, typename QT>
__global__ __launch_bounds__(kPostThreads) void mix_prep_kernel(
    const float* __restrict__ z, long ldz, int H, int G, int d, int dv, const float* __restrict__ qw, const float* __restrict__ kw,
    float eps, int dims, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int table_pos, int v_unit,
    const float* __restrict__ mix, QT* __restrict__ q_out, long ldqo, T* __restrict__ kcache, int Gk, T* __restrict__ vcache, int v_t,
    const int* __restrict__ tok_pos, const int* __restrict__ tok_seq, const int* __restrict__ block_table, int max_blocks,
    int num_blocks, int table_rows) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int qn = H * d, kn = G * d, vn = G * dv;
  float* qs = sm;
  float* ks = sm + qn;
  float* scratch = ks + kn;
  float* ms = scratch + 16;             // the head mix [H, H]
  if (mix)
    for (int i = threadIdx.x; i < H * H; i += kPostThreads) ms[i] = mix[i];
  const int t = blockIdx.x;
  const int pos = tok_pos[t], slot = tok_seq[t];
  const float* zr = z + (long)t * ldz;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < qn; i += kPostThreads) { const float v = zr[i]; qs[i] = v; sq += v * v; }
  for (int i = threadIdx.x; i < kn; i += kPostThreads) { const float v = zr[qn + i]; ks[i] = v; sk += v * v; }
  if (qw) {
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    const float rq = 1.f / sqrtf(sq / qn + eps), rk = 1.f / sqrtf(sk / kn + eps);
    for (int i = threadIdx.x; i < qn; i += kPostThreads) qs[i] *= rq * qw[i];      // (a thread's own entries)
    for (int i = threadIdx.x; i < kn; i += kPostThreads) ks[i] *= rk * kw[i];
  }
  __syncthreads();
  if (dims > 0 && pos >= 0 && pos < table_pos) {
    const int half = dims >> 1;
    const float* cs = cos_t + (long)pos * half;
    const float* sn = sin_t + (long)pos * half;
    for (int p = threadIdx.x; p < (H + G) * half; p += kPostThreads) {
      const int vec = p / half, pi = p % half;
      float* v = vec < H ? qs + (long)vec * d : ks + (long)(vec - H) * d;
      const float u = v[pi], w2 = v[pi + half], c = cs[pi], s = sn[pi];
      v[pi] = u * c - w2 * s;
      v[pi + half] = w2 * c + u * s;
    }
  }
  __syncthreads();
  if (q_out) {
    QT* qo = q_out + (long)t * ldqo;
    if (mix) {
      // A thread takes one entry (key head c, place i) of the query rows of ALL heads: the group's queries at that place are
      // read once, the mix comes from LDS (every lane of a wave reads the same address: a broadcast), and a wave's stores
      // cover consecutive entries of one head's row.
      const int group = H / G, row = G * d;
      for (int e = threadIdx.x; e < row; e += kPostThreads) {
        const int c = e / d, i = e % d;
        for (int h0 = 0; h0 < H; h0 += 8) {
          float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          for (int j = 0; j < group; ++j) {
            const float qv = qs[(c * group + j) * d + i];
#pragma unroll
            for (int u = 0; u < 8; ++u)
              if (h0 + u < H) acc[u] += ms[(h0 + u) * H + c * group + j] * qv;
          }
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (h0 + u < H) qo[(long)(h0 + u) * row + e] = (QT)acc[u];
        }
      }
    } else {
      for (int i = threadIdx.x; i < qn; i += kPostThreads) qo[i] = (QT)qs[i];
    }
  }
  int blk = -1;
  if (slot >= 0 && slot < table_rows && pos >= 0 && pos / kPostBlock < max_blocks) blk = block_table[(long)slot * max_blocks + pos / kPostBlock];
  if (blk < 0 || blk >= num_blocks) return;
  const int off = pos % kPostBlock, dk = kn / Gk;
  for (int i = threadIdx.x; i < kn; i += kPostThreads) {
    const int g = i / dk, c = i % dk;
    kcache[(((long)blk * Gk + g) * kPostBlock + off) * dk + c] = (T)ks[i];
  }
  // values: a wave per head; v_t: a block holds them key-contiguous, [head][entry][32 tokens]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* vr = zr + qn + kn;
  for (int g = wave; g < G; g += kPostThreads / 64) {
    float r = 1.f;
    if (v_unit) {
      float ss = 0.f;
      for (int c = lane; c < dv; c += 64) { const float v = vr[g * dv + c]; ss += v * v; }
      ss = wave_sum(ss);
      r = 1.f / sqrtf(ss / dv + eps);
    }
    for (int c = lane; c < dv; c += 64) {
      const float v = vr[g * dv + c] * r;
      if (v_t) vcache[(((long)blk * G + g) * dv + c) * kPostBlock + off] = (T)v;
      else vcache[(((long)blk * G + g) * kPostBlock + off) * dv + c] = (T)v;
    }
  }
  (void)vn;
}

}  // namespace dlia

extern "C" void dlia_post_norm_add(void* out, int out_f32, long ldo, float* x, long ldx, const float* ya, long ldya, const float* yb,
                                   long ldyb, float a, float b, const float* w, int T, int H, float eps, hipStream_t stream) {
  if (T <= 0) return;
  if (out_f32 || !out)
    hipLaunchKernelGGL(dlia::post_norm_add_kernel<float>, dim3(T), dim3(dlia::kPostThreads), 0, stream, (float*)out, ldo, x, ldx, ya,
                       ldya, yb, ldyb, a, b, w, H, eps);
  else
    hipLaunchKernelGGL(dlia::post_norm_add_kernel<dlia::bf16>, dim3(T), dim3(dlia::kPostThreads), 0, stream, (dlia::bf16*)out, ldo, x,
                       ldx, ya, ldya, yb, ldyb, a, b, w, H, eps);
}

extern "C" int dlia_mix_prep(const float* z, long ldz, int T, int H, int G, int d, int dv, const float* qw, const float* kw, float eps,
                             int dims, const float* cos_t, const float* sin_t, int table_pos, int v_unit, const float* mix, void* q_out,
                             int q_f32, long ldqo, void* kcache, int Gk, void* vcache, int v_t, int cache_f32, const int* tok_pos,
                             const int* tok_seq, const int* block_table, int max_blocks, int num_blocks, int table_rows,
                             hipStream_t stream) {
  if (T <= 0) return 0;
  const size_t lds = ((size_t)(H + G) * d + 16 + (mix ? (size_t)H * H : 0)) * sizeof(float);
  if (lds > 65536) return 1;
#define DLIA_PREP(CT, QT)                                                                                                      \
  hipLaunchKernelGGL((dlia::mix_prep_kernel<CT, QT>), dim3(T), dim3(dlia::kPostThreads), lds, stream, z, ldz, H, G, d, dv, qw, kw, eps, \
                     dims, cos_t, sin_t, table_pos, v_unit, mix, (QT*)q_out, ldqo, (CT*)kcache, Gk, (CT*)vcache, v_t, tok_pos, tok_seq, \
                     block_table, max_blocks, num_blocks, table_rows)
  if (cache_f32) {
    if (q_f32) DLIA_PREP(float, float); else return 1;
  } else {
    if (q_f32) DLIA_PREP(dlia::bf16, float); else DLIA_PREP(dlia::bf16, dlia::bf16);
  }
#undef DLIA_PREP
  return 0;
}
