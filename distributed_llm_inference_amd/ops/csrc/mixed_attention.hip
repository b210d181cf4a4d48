// Attention whose heads' scores are mixed before the softmax, s_h <- sum_g M[h, g] (q_g . k), for prompt portions on the
// matrix cores (bf16), with the mix applied to the finished score tiles.
//
// One workgroup per 16 consecutive tokens of a sequence sees ALL heads. Per cache block of 32 keys wave w forms the raw score
// tiles S_g^T = K_c(g) . Q_g^T of the heads g = w, w + waves, ... (K fragments straight from the cache rows, Q fragments held in
// registers for the whole kernel) and leaves them in LDS in the lanes' own order; after a barrier it reads every head's tile
// back and accumulates sum_g M[h, g] S_g in fp32 for the ONE head h whose output it owns (M carries the mix, the heads'
// temperatures and the scale). With more than 16 heads a wave forms two raw tiles per block and gridDim.y workgroups share the
// output heads (each repeats the raw tiles: they are the cheap part). From there a head runs as in tile_attention: a lane holds
// 8 scores of ONE query, mask (causal, chunk) and the running softmax are lane-local up to two shuffles, the 8 weights are the
// lane's B fragment of O^T += V^T . P^T over key-contiguous values, the sink enters once where a row is normalised, an
// element-wise sigmoid gate multiplies the output.
//
// Against carrying the mix in the query (a query row of kv_heads * d entries per head, see mix_prep) the score products are
// those of plain attention (d per key and head instead of kv_heads * d) and the keys are read in rows of d; the price is the
// exchange: heads x 32 bytes per lane and block through LDS, read by every wave. Keys are ONE cache row of all key heads per
// token, [blocks][32][G * d], as mix_prep writes them; values [blocks][G][dv][32].
//
// A tile's key blocks are walked one after the other with two barriers each, and a prompt has few tiles (one per 16 tokens) of
// very unequal length, so with a workspace the blocks of a tile are dealt out to gridDim.z workgroups, each of which leaves its
// (maximum, sum, weighted values) per (token, head) there; tile_attention's merge kernel folds them, adds the sink and gates.
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kMixBlock = 32;

// (A variant in which a wave of a 32-head model owned two output heads, reading every tile once for both, needed more
// registers than a wave of a 16-wave workgroup gets and spilled: 1.02 ms against 0.80 ms per 2048-token layer. So every wave
// owns one output head and two workgroups share a tile's 32 heads.)
template <int DVT, int HPW, int DK>
__global__ __launch_bounds__(1024) void mixed_attention_kernel(
    bf16* __restrict__ out, long ldo, const bf16* __restrict__ q, long ldq, const bf16* __restrict__ kcache, int k_row,
    const bf16* __restrict__ vt, const float* __restrict__ mix, const int* __restrict__ q_start, const int* __restrict__ ctx,
    const int* __restrict__ slots, const int* __restrict__ block_table, int tiles_per_seq, int max_blocks, int num_blocks,
    int table_rows, int H, int G, int d, int dv, int chunk, const float* __restrict__ sink, const float* __restrict__ gate,
    long ldg, float* __restrict__ part) {
  extern __shared__ __attribute__((aligned(16))) float lds[];       // score tiles [H][64 lanes][8], then the mix [H][H]
  float* S = lds;                        // (a head's tile: the lanes' first four scores, then their second four: 16-byte rows)
  float* Ms = lds + (long)H * 512;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int nw = blockDim.x >> 6, group = H / G;
  const int b = blockIdx.x / tiles_per_seq, ti = blockIdx.x % tiles_per_seq;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  const int r0 = ti * 16, nrows = min(16, n - r0);
  if (nrows <= 0 || slot < 0 || slot >= table_rows) return;            // (the whole workgroup: nobody waits at a barrier)
  for (int i = threadIdx.x; i < H * H; i += blockDim.x) Ms[i] = mix[i];
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const bool qvalid = r16 < nrows;
  const int ho = blockIdx.y * nw + wave;          // the head whose output this wave owns (none when >= H)
  int hh[HPW];
  u32x4 qf[HPW][DK];
#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    hh[j] = wave + j * nw;
#pragma unroll
    for (int u = 0; u < DK; ++u) {
      const int k = u * 32 + kq * 8;
      qf[j][u] = (hh[j] < H && qvalid && k < d) ? ld16(q + (long)(t0 + r0 + r16) * ldq + (long)hh[j] * d + k) : zero;
    }
  }
  const int pos_first = c0 + r0, pos_last = pos_first + nrows - 1, qpos = pos_first + r16;
  const int lo_first = chunk > 0 ? pos_first / chunk * chunk : 0;       // (the first row's chunk starts lowest)
  const int chunk_lo = chunk > 0 ? qpos / chunk * chunk : 0;
  const int kb_lo = lo_first / kMixBlock, kb_hi = min(pos_last / kMixBlock, max_blocks - 1);
  const int* table = block_table + (long)slot * max_blocks;
  float m = -INFINITY, lsum = 0.f;
  f32x4 o[DVT];
#pragma unroll
  for (int c = 0; c < DVT; ++c) o[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float* mrow = Ms + (long)min(ho, H - 1) * H;
  __syncthreads();
  for (int kb = kb_lo; kb <= kb_hi; ++kb) {
    if ((kb - kb_lo) % (int)gridDim.z != (int)blockIdx.z) continue;     // (another workgroup's block)
    const int blk = table[kb];
    if (blk < 0 || blk >= num_blocks) continue;                        // (uniform over the workgroup)
    // the raw score tiles of this wave's heads
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      if (hh[j] >= H) continue;
      const bf16* kbase = kcache + (long)blk * kMixBlock * k_row + (long)(hh[j] / group) * d;
      u32x4 ak[DK][2];
#pragma unroll
      for (int u = 0; u < DK; ++u)
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
          const int k = u * 32 + kq * 8;
          ak[u][tl] = k < d ? ld16(kbase + (long)(tl * 16 + r16) * k_row + k) : zero;
        }
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < DK; ++u) {
        s0 = mfma16(ak[u][0], qf[j][u], s0);
        s1 = mfma16(ak[u][1], qf[j][u], s1);
      }
      float* dst = S + ((long)hh[j] * 128 + lane) * 4;
      *reinterpret_cast<f32x4*>(dst) = s0;
      *reinterpret_cast<f32x4*>(dst + 256) = s1;
    }
    __syncthreads();
    // the mix: every head's tile weighted by this wave's row of M
    f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
    for (int g = 0; g < H; ++g) {
      const float* src = S + ((long)g * 128 + lane) * 4;
      const f32x4 x0 = *reinterpret_cast<const f32x4*>(src), x1 = *reinterpret_cast<const f32x4*>(src + 256);
      const float w = mrow[g];
      a0 += w * x0;
      a1 += w * x1;
    }
    __syncthreads();                                                    // (all tiles are read before the next block's are written)
    if (ho < H) {
      float sv[8], bm = -INFINITY;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int key = kb * kMixBlock + (i >> 2) * 16 + kq * 4 + (i & 3);
        const bool vis = qvalid && key <= qpos && key >= chunk_lo;
        sv[i] = vis ? (i < 4 ? a0[i & 3] : a1[i & 3]) : -INFINITY;
        bm = fmaxf(bm, sv[i]);
      }
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(m, bm);
      float p[8], corr = 1.f, add = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int i = 0; i < 8; ++i) p[i] = 0.f;
      } else {
        corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
#pragma unroll
        for (int i = 0; i < 8; ++i) { p[i] = sv[i] == -INFINITY ? 0.f : expf(sv[i] - m_new); add += p[i]; }
      }
      lsum = lsum * corr + add;
      m = m_new;
      const u32x4 pf = pack8(p);
      const bf16* vbase = vt + ((long)blk * G + ho / group) * dv * kMixBlock + (long)r16 * kMixBlock + kq * 4;
#pragma unroll
      for (int c = 0; c < DVT; ++c) {
        o[c] *= corr;
        if (c * 16 >= dv) continue;
        u32x4 v1 = zero;
        if (c * 16 + r16 < dv) {
          const u32x2 lo = *reinterpret_cast<const u32x2*>(vbase + (long)c * 16 * kMixBlock);
          const u32x2 hi = *reinterpret_cast<const u32x2*>(vbase + (long)c * 16 * kMixBlock + 16);
          v1 = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
        o[c] = mfma16(v1, pf, o[c]);
      }
    }
  }
  if (ho < H) {
    const int h = ho;
    float l = lsum;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (part) {                          // one of several workgroups of this tile: the merge finishes the row
      if (!qvalid) return;
      float* pr = part + ((((long)t0 + r0 + r16) * H + h) * gridDim.z + blockIdx.z) * (dv + 2);
      if (kq == 0) { pr[dv] = m; pr[dv + 1] = l; }
#pragma unroll
      for (int c = 0; c < DVT; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int col = c * 16 + kq * 4 + r;
          if (col < dv) pr[col] = o[c][r];
        }
      return;
    }
    if (sink) l = m == -INFINITY ? 1.f : l + expf(sink[h] - m);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (!qvalid) return;
    const long t = t0 + r0 + r16;
    bf16* orow = out + t * ldo + (long)h * dv;
    const float* grow = gate ? gate + t * ldg + (long)h * dv : nullptr;
#pragma unroll
    for (int c = 0; c < DVT; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = c * 16 + kq * 4 + r;
        if (col < dv) {
          float v = o[c][r] * inv;
          if (grow) v *= 1.f / (1.f + expf(-grow[col]));
          orow[col] = (bf16)v;
        }
      }
  }
}

template <int DVT, int HPW, int DK>
static void launch_mixed(dim3 grid, int threads, size_t lds, hipStream_t stream, void* out, long ldo, const void* q, long ldq,
                         const void* kcache, int k_row, const void* vt, const float* mix, const int* q_start, const int* ctx,
                         const int* slots, const int* block_table, int tiles, int max_blocks, int num_blocks, int table_rows, int H,
                         int G, int d, int dv, int chunk, const float* sink, const float* gate, long ldg, float* part) {
  static const bool once = [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&mixed_attention_kernel<DVT, HPW, DK>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
    return true;
  }();
  (void)once;
  hipLaunchKernelGGL((mixed_attention_kernel<DVT, HPW, DK>), grid, dim3(threads), lds, stream, (bf16*)out, ldo, (const bf16*)q, ldq,
                     (const bf16*)kcache, k_row, (const bf16*)vt, mix, q_start, ctx, slots, block_table, tiles, max_blocks, num_blocks,
                     table_rows, H, G, d, dv, chunk, sink, gate, ldg, part);
}

}  // namespace dlia

// 1: sizes this kernel does not take (up to 32 heads, key size a multiple of 8 up to 256, value size up to 128); nothing launched.
extern "C" int dlia_mixed_attention_fits(int H, int G, int d, int dv) {
  return H >= 1 && H <= 32 && G >= 1 && H % G == 0 && d % 8 == 0 && d >= 8 && d <= 256 && dv >= 1 && dv <= 128;
}

constexpr int kMixMaxSplits = 4;
extern "C" long dlia_mixed_attention_part_floats(int T, int H, int dv) { return (long)T * H * kMixMaxSplits * (dv + 2); }

extern "C" int dlia_mixed_attention(void* out, long ldo, const void* q, long ldq, const void* kcache, int k_row, const void* vt,
                                    const float* mix, const int* q_start, const int* ctx, const int* slots, const int* block_table,
                                    int B, int max_q, int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv,
                                    int chunk, const float* sink, const float* gate, long ldg, float* part, long part_floats, int T,
                                    hipStream_t stream) {
  using namespace dlia;
  if (B <= 0 || max_q <= 0) return 0;
  if (!dlia_mixed_attention_fits(H, G, d, dv) || k_row % 8 || ldq % 8) return 1;
  const int tiles = (max_q + 15) / 16;
  const int hpw = H <= 16 ? 1 : 2, nw = H <= 16 ? H : 16;       // (raw tiles per wave; the waves' output heads: one each)
  const int dk = d <= 64 ? 2 : d <= 128 ? 4 : 8, dvt = dv <= 64 ? 4 : 8;
  const size_t lds = ((size_t)H * 512 + (size_t)H * H) * sizeof(float);
  // enough workgroups for the chip: a tile's key blocks over up to kMixMaxSplits of them when the workspace is there
  const int ny = (H + nw - 1) / nw;
  int nz = 1;
  while (nz < kMixMaxSplits && B * tiles * ny * nz < 1024 && max_q > 16) nz <<= 1;
  if (!part || part_floats < (long)T * H * nz * (dv + 2)) nz = 1;
  if (nz == 1) part = nullptr;
  const dim3 grid(B * tiles, ny, nz);
#define DLIA_MIXED(DVT, HPW, DK)                                                                                          \
  launch_mixed<DVT, HPW, DK>(grid, 64 * nw, lds, stream, out, ldo, q, ldq, kcache, k_row, vt, mix, q_start, ctx, slots,   \
                             block_table, tiles, max_blocks, num_blocks, table_rows, H, G, d, dv, chunk, sink, gate, ldg, part)
#define DLIA_MIXED_DK(DVT, HPW)                                                              \
  do {                                                                                       \
    if (dk == 2) DLIA_MIXED(DVT, HPW, 2); else if (dk == 4) DLIA_MIXED(DVT, HPW, 4); else DLIA_MIXED(DVT, HPW, 8); \
  } while (0)
  if (dvt == 4) { if (hpw == 1) DLIA_MIXED_DK(4, 1); else DLIA_MIXED_DK(4, 2); }
  else { if (hpw == 1) DLIA_MIXED_DK(8, 1); else DLIA_MIXED_DK(8, 2); }
#undef DLIA_MIXED_DK
#undef DLIA_MIXED
  if (nz > 1) dlia_tile_merge(out, ldo, part, T * H, H, dv, nz, gate, ldg, sink, stream);
  return 0;
}
