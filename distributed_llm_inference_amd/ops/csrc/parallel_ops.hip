// Kernels for stacks whose layers run their two sublayers side by side on ONE norm of an fp32 residual stream,
//     n = rms(x) w;   x <- x + ls1 * mixer(shifted(n)) + ls2 * ff(n),
// whose mixers read a blend of n with the previous token's n, and whose mixers are a real-gated linear recurrence,
// attention over one or two score maps per head with partial rotation, or attention through a cached latent.
//
//   par_norm        one launch per layer boundary: the carried n of the closing layer is saved for its sequences' next
//                   step, x += ls1 * ya + ls2 * yb, and the next layer's n leaves in fp32 (for the blend) and in the
//                   GEMMs' input type (for the feed-forward)
//   token_shift     n + (previous n - n) * mu per token; the previous n is the row above, the slot's carried n at the
//                   start of a portion, zeros at position 0
//   rope_cache_write per token: rotates the first `dims` entries of a set of q vectors and of the k vectors (pairs
//                   (2i, 2i + 1) or (i, i + dims / 2), angles from a table by position), optionally leaves q in the
//                   GEMMs' input type, and writes the k row (and the v row) into the paged cache
//   multi_attention one wave per (token, head): softmax attention over the paged cache with a window that also keeps
//                   the sequence's first tokens, scores through cap tanh(s / cap); with two maps per head both are
//                   walked at once over the shared values and combined as rms(a1 - lam a2) (1 - diff) sigmoid(gate).
//                   Keys are rows of any length (a map is a slice of the row), values may be a slice of the key rows.
//                   The key cache may have fewer heads than the value cache (one row of all key heads for queries that carry
//                   a mix of heads); `chunk` > 0 hides the keys of other chunks of that many positions; `sink` [H] adds
//                   exp(sink[h]) to the softmax's denominator.
//   rglru_scan      S <- a S + sqrt(1 - a^2) i u per channel with a = exp(-c r), r and i sigmoids of the block gates;
//                   read-out S * gelu_tanh(y). Long portions are cut into stretches that are scanned side by side and
//                   joined through the stretches' (decay product, end value) pairs: inside a workgroup through LDS, or,
//                   given a workspace, over workgroups through memory in two launches.
//   xielu, scale_rows   the feed-forward's activation; logits times a constant
// Everything is fp32 except what feeds a GEMM or sits in the cache (the compute type, bf16 or fp32).
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kParBlock = 32;        // tokens per cache block
constexpr int kParThreads = 256;

// ---- norm / residual / carried rows -------------------------------------------------------------------------------
template <typename OT>
__global__ __launch_bounds__(kParThreads) void par_norm_kernel(
    OT* __restrict__ out, float* __restrict__ out32, float* __restrict__ x, const float* __restrict__ ya,
    const float* __restrict__ yb, const float* __restrict__ ls1, const float* __restrict__ ls2, const float* __restrict__ w,
    float* __restrict__ carry, const int* __restrict__ tok_seq, int T, int state_rows, int H, long ldx, long ldya, long ldyb,
    long ldo, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (long)t * ldx;
  float* nr = out32 + (long)t * H;
  if (carry) {
    const int slot = tok_seq[t];
    const bool last = t + 1 == T || tok_seq[t + 1] != slot;
    if (last && slot >= 0 && slot < state_rows)
      for (int i = threadIdx.x; i < H; i += kParThreads) carry[(long)slot * H + i] = nr[i];
  }
  if (ya) {
    const float* ar = ya + (long)t * ldya;
    const float* br = yb ? yb + (long)t * ldyb : nullptr;
    for (int i = threadIdx.x; i < H; i += kParThreads) {
      float add = ls1[i] * ar[i];
      if (br) add += ls2[i] * br[i];
      xr[i] += add;
    }
  }
  if (!out) return;
  float s = 0.f;
  for (int i = threadIdx.x; i < H; i += kParThreads) { const float v = xr[i]; s += v * v; }   // (each thread re-reads what it wrote itself)
  s = block_sum(s, scratch);
  const float r = 1.f / sqrtf(s / H + eps);
  OT* orow = out + (long)t * ldo;
  for (int i = threadIdx.x; i < H; i += kParThreads) {
    const float v = xr[i] * r * w[i];
    nr[i] = v;
    orow[i] = (OT)v;
  }
}

template <typename OT>
__global__ __launch_bounds__(kParThreads) void token_shift_kernel(
    OT* __restrict__ out, const float* __restrict__ n32, const float* __restrict__ carry, const float* __restrict__ mu,
    const int* __restrict__ tok_pos, const int* __restrict__ tok_seq, int state_rows, int H, long ldo) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t], slot = tok_seq[t];
  const float* cur = n32 + (long)t * H;
  const float* prev = nullptr;
  if (pos > 0) {
    if (t > 0 && tok_seq[t - 1] == slot && tok_pos[t - 1] == pos - 1) prev = cur - H;
    else if (slot >= 0 && slot < state_rows) prev = carry + (long)slot * H;
  }
  OT* orow = out + (long)t * ldo;
  for (int i = threadIdx.x; i < H; i += kParThreads) {
    const float h = cur[i], p = prev ? prev[i] : 0.f;
    orow[i] = (OT)(h + (p - h) * mu[i]);
  }
}

// ---- rotation + cache write ----------------------------------------------------------------------------------------
// A set of vectors inside a row: entries [off, off + dims) of every `stride` entries are rotated.
__device__ __forceinline__ void rotate_row(float* row, int n_vec, int stride, int off, int dims, int interleaved,
                                           const float* cs, const float* sn) {
  const int half = dims >> 1;
  for (int p = threadIdx.x; p < n_vec * half; p += kParThreads) {
    const int vi = p / half, pi = p % half;
    float* v = row + (long)vi * stride + off;
    const int i0 = interleaved ? 2 * pi : pi, i1 = interleaved ? 2 * pi + 1 : pi + half;
    const float a = v[i0], b = v[i1], c = cs[pi], s = sn[pi];
    v[i0] = a * c - b * s;
    v[i1] = b * c + a * s;
  }
}

template <typename T>
__global__ __launch_bounds__(kParThreads) void rope_cache_write_kernel(
    float* __restrict__ q, long ldq, int q_vecs, int q_stride, int q_off, T* __restrict__ q_out, long ldqo, int q_cols,
    float* __restrict__ kv, long ldkv, int k_cols, int k_vecs, int k_stride, int k_off, int v_src, int v_cols, int v_t,
    T* __restrict__ kcache, T* __restrict__ vcache, int G, int dims, int interleaved, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t,
    int table_pos, const int* __restrict__ tok_pos, const int* __restrict__ tok_seq, const int* __restrict__ block_table,
    int max_blocks, int num_blocks, int table_rows) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t], slot = tok_seq[t];
  float* qrow = q + (long)t * ldq;
  float* krow = kv + (long)t * ldkv;
  if (dims > 0 && pos >= 0 && pos < table_pos) {
    const float* cs = cos_t + (long)pos * (dims >> 1);
    const float* sn = sin_t + (long)pos * (dims >> 1);
    rotate_row(qrow, q_vecs, q_stride, q_off, dims, interleaved, cs, sn);
    rotate_row(krow, k_vecs, k_stride, k_off, dims, interleaved, cs, sn);
  }
  __syncthreads();
  if (q_out)
    for (int i = threadIdx.x; i < q_cols; i += kParThreads) q_out[(long)t * ldqo + i] = (T)qrow[i];
  int blk = -1;
  if (slot >= 0 && slot < table_rows && pos >= 0 && pos / kParBlock < max_blocks) blk = block_table[(long)slot * max_blocks + pos / kParBlock];
  if (blk < 0 || blk >= num_blocks) return;
  const int off = pos % kParBlock, dk = k_cols / G;
  for (int i = threadIdx.x; i < k_cols; i += kParThreads) {
    const int g = i / dk, c = i % dk;
    kcache[(((long)blk * G + g) * kParBlock + off) * dk + c] = (T)krow[i];
  }
  if (vcache) {
    // values: entries [v_src, v_src + v_cols) of the row; v_t: a block holds them key-contiguous, [head][entry][32 tokens]
    const int dv = v_cols / G;
    const float* vrow = krow + v_src;
    for (int i = threadIdx.x; i < v_cols; i += kParThreads) {
      const int g = i / dv, c = i % dv;
      if (v_t) vcache[(((long)blk * G + g) * dv + c) * kParBlock + off] = (T)vrow[i];
      else vcache[(((long)blk * G + g) * kParBlock + off) * dv + c] = (T)vrow[i];
    }
  }
}

// ---- attention ---------------------------------------------------------------------------------------------------
constexpr int kMultiMaxQ = 1024;     // MAPS * d
constexpr int kMultiMaxDV = 512;

__device__ __forceinline__ float dot_row(const float* qs, const bf16* k, int d, bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int i = 0; i < d; i += 8) {
      float f[8];
      unpack8(ld16(k + i), f);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += qs[i + j] * f[j];
    }
  } else {
    for (int i = 0; i < d; ++i) acc += qs[i] * (float)k[i];
  }
  return acc;
}
__device__ __forceinline__ float dot_row(const float* qs, const float* k, int d, bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int i = 0; i < d; i += 4) {
      const f32x4 f = *reinterpret_cast<const f32x4*>(k + i);
      acc += qs[i] * f[0] + qs[i + 1] * f[1] + qs[i + 2] * f[2] + qs[i + 3] * f[3];
    }
  } else {
    for (int i = 0; i < d; ++i) acc += qs[i] * k[i];
  }
  return acc;
}

template <typename T, typename OT, int MAPS>
__global__ __launch_bounds__(256) void multi_attention_kernel(
    OT* __restrict__ out, long ldo, const float* __restrict__ q, long ldq, int q_head, const T* __restrict__ kcache, int k_row,
    const T* __restrict__ vcache, int v_row, int v_off, const int* __restrict__ tok_pos, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int items, int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv,
    float scale, int window, int keep_first, float softcap, float lam, float post, float eps, const float* __restrict__ gate,
    long ldg, int vec, int Gk, int chunk, const float* __restrict__ sink) {
  __shared__ float qs[4][kMultiMaxQ];
  const int wave = threadIdx.x >> 6, lane = lane_id();
  const int item = blockIdx.x * 4 + wave;
  if (item >= items) return;
  const int t = item / H, h = item % H, g = h / (H / G), gk = h / (H / Gk);
  const int pos = tok_pos[t], slot = tok_seq[t];
  OT* orow = out + (long)t * ldo + (long)h * dv;
  const bool live = slot >= 0 && slot < table_rows && pos >= 0 && pos / kParBlock < max_blocks;
  if (!live) {                                   // padding row of a fixed-shape step
    for (int c = lane; c < dv; c += 64) orow[c] = (OT)0.f;
    return;
  }
  const float* qrow = q + (long)t * ldq + (long)h * q_head;
  for (int i = lane; i < MAPS * d; i += 64) qs[wave][i] = qrow[i] * scale;
  __builtin_amdgcn_wave_barrier();
  const int* table = block_table + (long)slot * max_blocks;
  int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  if (chunk > 0) lo = max(lo, pos / chunk * chunk);                             // the query's own chunk only
  const int kept = (window > 0 && keep_first > 0) ? min(keep_first, lo) : 0;    // keys [0, kept) in front of the window
  float m[MAPS], l[MAPS], acc[MAPS][kMultiMaxDV / 64];
#pragma unroll
  for (int a = 0; a < MAPS; ++a) {
    m[a] = -INFINITY; l[a] = 0.f;
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) acc[a][c] = 0.f;
  }
  const int ncol = (dv + 63) / 64;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;
  for (int seg = kept > 0 ? 0 : 1; seg < 2; ++seg) {
    const int j_lo = seg == 0 ? 0 : lo, j_hi = seg == 0 ? kept - 1 : pos;
    for (int j0 = j_lo; j0 <= j_hi; j0 += 64) {
      const int j = j0 + lane;
      int blk = -1;
      if (j <= j_hi) blk = table[j / kParBlock];
      const bool valid = blk >= 0 && blk < num_blocks;
      float s[MAPS], p[MAPS];
      bool any = false;
#pragma unroll
      for (int a = 0; a < MAPS; ++a) {
        s[a] = -INFINITY;
        if (valid) {
          const T* krow = kcache + (((long)blk * Gk + gk) * kParBlock + (j % kParBlock)) * k_row + a * d;
          float dot = dot_row(qs[wave] + a * d, krow, d, vec != 0);
          if (softcap > 0.f) dot = softcap * tanhf(dot * inv_cap);
          s[a] = dot;
        }
        const float m_new = fmaxf(m[a], wave_max(s[a]));
        if (m_new == -INFINITY) { p[a] = 0.f; continue; }      // (uniform over the wave)
        p[a] = valid ? expf(s[a] - m_new) : 0.f;
        const float corr = (m[a] == -INFINITY) ? 0.f : expf(m[a] - m_new);
        l[a] = l[a] * corr + wave_sum(p[a]);
        m[a] = m_new;
#pragma unroll
        for (int c = 0; c < kMultiMaxDV / 64; ++c) acc[a][c] *= corr;
        any = true;
      }
      if (!any) continue;
      const int nk = (j_hi - j0 + 1) < 64 ? (j_hi - j0 + 1) : 64;
      for (int jj = 0; jj < nk; ++jj) {
        float pj[MAPS];
        bool zero = true;
#pragma unroll
        for (int a = 0; a < MAPS; ++a) { pj[a] = __shfl(p[a], jj, 64); zero = zero && pj[a] == 0.f; }
        const int bj = __shfl(blk, jj, 64);
        if (zero) continue;                       // (uniform: an unreadable key, or weights that underflowed)
        const T* vrow = vcache + (((long)bj * G + g) * kParBlock + ((j0 + jj) % kParBlock)) * v_row + v_off;
#pragma unroll
        for (int c = 0; c < kMultiMaxDV / 64; ++c)
          if (c < ncol) {
            const int col = c * 64 + lane;
            if (col < dv) {
              const float v = (float)vrow[col];
#pragma unroll
              for (int a = 0; a < MAPS; ++a) acc[a][c] += pj[a] * v;
            }
          }
      }
    }
  }
  if (sink) {
    // one more term in the denominator: a key of score sink[h] that has no value
#pragma unroll
    for (int a = 0; a < MAPS; ++a) l[a] = m[a] == -INFINITY ? 1.f : l[a] + expf(sink[h] - m[a]);
  }
  float o[kMultiMaxDV / 64];
  const float i0 = l[0] > 0.f ? 1.f / l[0] : 0.f;
  if constexpr (MAPS == 1) {
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) o[c] = acc[0][c] * i0;
  } else {
    // the two maps combined, normalised over the head's values, and gated
    const float i1 = l[1] > 0.f ? 1.f / l[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) {
      o[c] = 0.f;
      if (c < ncol && c * 64 + lane < dv) { o[c] = acc[0][c] * i0 - lam * acc[1][c] * i1; ss += o[c] * o[c]; }
    }
    ss = wave_sum(ss);
    const float r = post / sqrtf(ss / dv + eps);
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) o[c] *= r;
  }
#pragma unroll
  for (int c = 0; c < kMultiMaxDV / 64; ++c)
    if (c < ncol) {
      const int col = c * 64 + lane;
      if (col < dv) {
        float v = o[c];
        if (gate) v *= 1.f / (1.f + expf(-gate[(long)t * ldg + (long)h * dv + col]));
        orow[col] = (OT)v;
      }
    }
}


// ---- attention on the matrix cores (bf16) ---------------------------------------------------------------------------
// One wave per (16 consecutive tokens of a sequence, head). Per cache block of 32 keys: S^T = K . Q^T as two 16-key MFMA tiles
// per score map (K fragments straight from the cache rows, Q fragments from LDS), so that a lane holds 8 scores of ONE query:
// scale, cap, mask and the running softmax are lane-local up to two shuffles over the four lanes that share a query. The
// weights of those 8 keys ARE the lane's B fragment of O^T += V^T . P^T when the A fragment takes the same keys in the same
// order, which it can because values sit key-contiguous in the cache: two 8-byte loads per 16 value entries. Both maps of a
// head use the same value fragments. Blocks in front of the window are skipped except those that hold kept first tokens.
// Single-token steps over ONE key row for all heads (Gk == 1 < G): with many key / value heads a tile takes 16 consecutive heads
// whatever their value head, so that the long key rows are read once per 16 heads instead of once per value head; the value
// product then runs once per value head of the tile, one after the other. With few value heads a tile per value head is
// faster (64 sequences at 1024 tokens, key rows of 4 x 128: 17 against 30 us per layer; key rows of 8 x 128: a step of four
// layers 2.47 against 2.12 ms).
__host__ __device__ inline bool tile_all_heads(int G, int Gk) { return Gk == 1 && G > 4; }

template <int MAPS, int DVT, bool HEADROWS, int KS>
__global__ __launch_bounds__(256) void tile_attention_kernel(
    bf16* __restrict__ out, long ldo, const bf16* __restrict__ q, long ldq, int q_head, const bf16* __restrict__ kcache, int k_row,
    const bf16* __restrict__ vt, const int* __restrict__ q_start, const int* __restrict__ ctx, const int* __restrict__ slots,
    const int* __restrict__ block_table, int tiles_per_seq, int max_blocks, int num_blocks, int table_rows, int H, int G, int d,
    int dv, float scale, int window, int keep_first, float softcap, float lam, float post, float eps,
    const float* __restrict__ gate, long ldg, float* __restrict__ part, int Gk, int chunk, const float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) bf16 qs_all[];        // per wave [16][MAPS * d + 8]
  // Rows of a wave's tile. Prompt portions: 16 consecutive tokens of one head; the waves of a workgroup take neighbouring heads
  // (those of one key / value head first), so the key and value fragments they all read come from L1 after the first.
  // HEADROWS (steps of single tokens): the rows are the heads that share a key / value head, for ONE token: its keys and
  // values are read once for all of them. The token's key blocks are dealt out to gridDim.z workgroups, each of which leaves
  // its (maximum, sum, weighted values) in `part`; tile_merge_kernel folds them and finishes the heads.
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int group = H / G;
  const int b = blockIdx.x / tiles_per_seq, ti = blockIdx.x % tiles_per_seq;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  const bool all_heads = HEADROWS && tile_all_heads(G, Gk);      // (rows: 16 consecutive heads, see above)
  int h, g, r0, nrows;
  if constexpr (HEADROWS) {
    const int gt = (group + 15) / 16;
    g = all_heads ? 0 : blockIdx.y / gt;
    h = all_heads ? blockIdx.y * 16 : g * group + (blockIdx.y % gt) * 16;   // head of row 0
    r0 = 0;
    nrows = n <= 0 ? 0 : all_heads ? min(16, H - h) : min(16, group - (blockIdx.y % gt) * 16);
  } else {
    h = blockIdx.y * (blockDim.x >> 6) + wave;
    g = h < H ? h / group : 0;
    r0 = ti * 16;
    nrows = h < H ? min(16, n - r0) : 0;
  }
  if (nrows <= 0 || slot < 0 || slot >= table_rows) return;             // (whole wave; nothing below synchronises across waves)
  const int qp = MAPS * d + 8, per_row = MAPS * d / 8;
  bf16* qs = qs_all + (long)wave * 16 * qp;
  for (int i = lane; i < 16 * per_row; i += 64) {
    const int r = i / per_row, c8 = i % per_row;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (r < nrows) v = ld16(q + (long)(HEADROWS ? t0 : t0 + r0 + r) * ldq + (long)(HEADROWS ? h + r : h) * q_head + c8 * 8);
    st16(qs + r * qp + c8 * 8, v);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int pos_first = c0 + r0, pos_last = HEADROWS ? pos_first : pos_first + nrows - 1;
  const int qpos = HEADROWS ? pos_first : pos_first + r16;
  const bool qvalid = r16 < nrows;
  const int* table = block_table + (long)slot * max_blocks;
  float m[MAPS], lsum[MAPS];
  f32x4 o[MAPS][DVT];
#pragma unroll
  for (int a = 0; a < MAPS; ++a) {
    m[a] = -INFINITY; lsum[a] = 0.f;
#pragma unroll
    for (int c = 0; c < DVT; ++c) o[a][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;
  int lo_first = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  if (chunk > 0) lo_first = max(lo_first, pos_first / chunk * chunk);     // (the first row's chunk starts lowest)
  const int chunk_lo = chunk > 0 ? qpos / chunk * chunk : 0;
  const int gk = Gk == G ? g : 0;                                         // (the key cache has G heads or one)
  const int g_lo = all_heads ? h / group : g, g_hi = all_heads ? (h + nrows - 1) / group : g;
  const int my_g = all_heads ? min(h + r16, H - 1) / group : g;
  const int kb_lo = lo_first / kParBlock, kb_hi = min(pos_last / kParBlock, max_blocks - 1);
  const int kept = (window > 0 && keep_first > 0) ? min(keep_first, lo_first) : 0;
  const int kb_kept = kept > 0 ? min((kept - 1) / kParBlock, kb_lo - 1) : -1;      // blocks [0, kb_kept] hold kept tokens only
  const u32x4 zero = {0u, 0u, 0u, 0u};
  int turn = 0;
  for (int kb = kb_kept >= 0 ? 0 : kb_lo; kb <= kb_hi; kb = (kb == kb_kept ? kb_lo : kb + 1)) {
    if constexpr (HEADROWS) {
      if ((turn++) % (int)gridDim.z != (int)blockIdx.z) continue;
    }
    const int blk = table[kb];
    if (blk < 0 || blk >= num_blocks) continue;                        // (uniform)
    f32x4 s[MAPS][2];
#pragma unroll
    for (int a = 0; a < MAPS; ++a) s[a][0] = s[a][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    const bf16* kbase = kcache + ((long)blk * Gk + gk) * kParBlock * k_row;
    for (int k0 = 0; k0 < d; k0 += 32 * KS) {
      u32x4 ak[MAPS][KS][2];          // KS k-steps of key fragments in flight at once
#pragma unroll
      for (int a = 0; a < MAPS; ++a)
#pragma unroll
        for (int u = 0; u < KS; ++u)
#pragma unroll
          for (int tl = 0; tl < 2; ++tl) {
            const int k = k0 + u * 32 + kq * 8;
            ak[a][u][tl] = k < d ? ld16(kbase + (long)(tl * 16 + r16) * k_row + a * d + k) : zero;
          }
#pragma unroll
      for (int a = 0; a < MAPS; ++a)
#pragma unroll
        for (int u = 0; u < KS; ++u) {
          const int k = k0 + u * 32 + kq * 8;
          const u32x4 bq = k < d ? ld16(qs + r16 * qp + a * d + k) : zero;
          s[a][0] = mfma16(ak[a][u][0], bq, s[a][0]);
          s[a][1] = mfma16(ak[a][u][1], bq, s[a][1]);
        }
    }
    // Up to 16 accumulator tiles: the value fragments of the block's first VB tiles are asked for now, so that their way from
    // memory overlaps the softmax. (With more accumulators the registers do not hold them as well: fragment by fragment then.)
    constexpr bool AHEAD = MAPS * DVT <= 16;
    constexpr int VB = DVT > 8 ? 8 : DVT;
    const bf16* vbase = vt + ((long)blk * G + g_lo) * dv * kParBlock + (long)r16 * kParBlock + kq * 4;
    u32x4 av[VB];
    auto load_values = [&](int c0) {
#pragma unroll
      for (int j = 0; j < VB; ++j) {
        av[j] = zero;
        if ((c0 + j) * 16 + r16 < dv) {
          const u32x2 lo = *reinterpret_cast<const u32x2*>(vbase + (long)(c0 + j) * 16 * kParBlock);
          const u32x2 hi = *reinterpret_cast<const u32x2*>(vbase + (long)(c0 + j) * 16 * kParBlock + 16);
          av[j] = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
      }
    };
    if constexpr (AHEAD) load_values(0);
    u32x4 pf[MAPS];
#pragma unroll
    for (int a = 0; a < MAPS; ++a) {
      float sv[8];
      float bm = -INFINITY;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int j = kb * kParBlock + (i >> 2) * 16 + kq * 4 + (i & 3);
        const bool vis = qvalid && j <= qpos && j >= chunk_lo && (window <= 0 || qpos - j < window || j < keep_first);
        float x = s[a][i >> 2][i & 3] * scale;
        if (softcap > 0.f) x = softcap * tanhf(x * inv_cap);
        sv[i] = vis ? x : -INFINITY;
        bm = fmaxf(bm, sv[i]);
      }
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(m[a], bm);
      float p[8], corr = 1.f, add = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int i = 0; i < 8; ++i) p[i] = 0.f;
      } else {
        corr = (m[a] == -INFINITY) ? 0.f : expf(m[a] - m_new);
#pragma unroll
        for (int i = 0; i < 8; ++i) { p[i] = sv[i] == -INFINITY ? 0.f : expf(sv[i] - m_new); add += p[i]; }
      }
      lsum[a] = lsum[a] * corr + add;
      m[a] = m_new;
#pragma unroll
      for (int c = 0; c < DVT; ++c) o[a][c] *= corr;
      pf[a] = pack8(p);
    }
    for (int gv = g_lo; gv <= g_hi; ++gv) {
      u32x4 pm[MAPS];                   // the weights of the rows whose values are head gv's
#pragma unroll
      for (int a = 0; a < MAPS; ++a) pm[a] = my_g == gv ? pf[a] : zero;
      if (gv > g_lo) {
        vbase += (long)dv * kParBlock;
        if constexpr (AHEAD) load_values(0);
      }
      if constexpr (AHEAD) {
#pragma unroll
        for (int c0 = 0; c0 < DVT; c0 += VB) {
          if (c0 * 16 >= dv) break;
          if (c0 > 0) load_values(c0);
#pragma unroll
          for (int j = 0; j < VB; ++j) {
            if ((c0 + j) * 16 >= dv) break;
#pragma unroll
            for (int a = 0; a < MAPS; ++a) o[a][c0 + j] = mfma16(av[j], pm[a], o[a][c0 + j]);
          }
        }
      } else {
#pragma unroll
        for (int c = 0; c < DVT; ++c) {
          if (c * 16 >= dv) break;
          u32x4 v1 = zero;
          if (c * 16 + r16 < dv) {
            const u32x2 lo = *reinterpret_cast<const u32x2*>(vbase + (long)c * 16 * kParBlock);
            const u32x2 hi = *reinterpret_cast<const u32x2*>(vbase + (long)c * 16 * kParBlock + 16);
            v1 = u32x4{lo.x, lo.y, hi.x, hi.y};
          }
#pragma unroll
          for (int a = 0; a < MAPS; ++a) o[a][c] = mfma16(v1, pm[a], o[a][c]);
        }
      }
    }
  }
  float inv[MAPS];
#pragma unroll
  for (int a = 0; a < MAPS; ++a) {
    float l = lsum[a];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    lsum[a] = l;
  }
  if constexpr (HEADROWS) {
    if (!qvalid) return;
    const int nz = gridDim.z;
#pragma unroll
    for (int a = 0; a < MAPS; ++a) {
      float* pr = part + ((((long)t0 * H + h + r16) * MAPS + a) * nz + blockIdx.z) * (dv + 2);
      if (kq == 0) { pr[dv] = m[a]; pr[dv + 1] = lsum[a]; }
#pragma unroll
      for (int c = 0; c < DVT; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int col = c * 16 + kq * 4 + r;
          if (col < dv) pr[col] = o[a][c][r];
        }
    }
    return;
  }
  if (sink && qvalid) {
    const float sk = sink[h];
#pragma unroll
    for (int a = 0; a < MAPS; ++a) lsum[a] = m[a] == -INFINITY ? 1.f : lsum[a] + expf(sk - m[a]);
  }
#pragma unroll
  for (int a = 0; a < MAPS; ++a) inv[a] = lsum[a] > 0.f ? 1.f / lsum[a] : 0.f;
  float mul = inv[0];
  if constexpr (MAPS == 2) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < DVT; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float v = o[0][c][r] * inv[0] - lam * o[1][c][r] * inv[1];
        o[0][c][r] = v;
        ss += v * v;
      }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    mul = post / sqrtf(ss / dv + eps);
  }
  if (!qvalid) return;
  const long t = HEADROWS ? t0 : t0 + r0 + r16;
  const int hr = HEADROWS ? h + r16 : h;
  bf16* orow = out + t * ldo + (long)hr * dv;
  const float* grow = gate ? gate + t * ldg + (long)hr * dv : nullptr;
#pragma unroll
  for (int c = 0; c < DVT; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int col = c * 16 + kq * 4 + r;
      if (col < dv) {
        float v = o[0][c][r] * mul;
        if (grow) v *= 1.f / (1.f + expf(-grow[col]));
        orow[col] = (bf16)v;
      }
    }
}


// Folds the partial results of tile_attention_kernel's key splits for the heads of single-token rows and finishes them:
// normalisation, the two maps combined and RMS-normed, the gate. One wave per (token, head).
template <int MAPS>
__global__ __launch_bounds__(256) void tile_merge_kernel(bf16* __restrict__ out, long ldo, const float* __restrict__ part, int items,
                                                         int H, int dv, int nz, float lam, float post, float eps,
                                                         const float* __restrict__ gate, long ldg, const float* __restrict__ sink) {
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6), lane = lane_id();
  if (item >= items) return;
  const int t = item / H, h = item % H;
  float o[MAPS][kMultiMaxDV / 64];
#pragma unroll
  for (int a = 0; a < MAPS; ++a) {
    const float* pr = part + (((long)t * H + h) * MAPS + a) * nz * (dv + 2);
    float M = -INFINITY;
    for (int z = 0; z < nz; ++z) M = fmaxf(M, pr[(long)z * (dv + 2) + dv]);
    float L = 0.f;
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) o[a][c] = 0.f;
    for (int z = 0; z < nz; ++z) {
      const float* pz = pr + (long)z * (dv + 2);
      const float mz = pz[dv];
      if (mz == -INFINITY) continue;                  // (uniform: a split that saw no key)
      const float w = expf(mz - M);
      L += pz[dv + 1] * w;
#pragma unroll
      for (int c = 0; c < kMultiMaxDV / 64; ++c) { const int col = c * 64 + lane; if (col < dv) o[a][c] += pz[col] * w; }
    }
    if (sink) L = M == -INFINITY ? 1.f : L + expf(sink[h] - M);
    const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) o[a][c] *= inv;
  }
  float mul = 1.f;
  if constexpr (MAPS == 2) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kMultiMaxDV / 64; ++c) { o[0][c] -= lam * o[1][c]; ss += o[0][c] * o[0][c]; }
    ss = wave_sum(ss);
    mul = post / sqrtf(ss / dv + eps);
  }
  bf16* orow = out + (long)t * ldo + (long)h * dv;
#pragma unroll
  for (int c = 0; c < kMultiMaxDV / 64; ++c) {
    const int col = c * 64 + lane;
    if (col < dv) {
      float v = o[0][c] * mul;
      if (gate) v *= 1.f / (1.f + expf(-gate[(long)t * ldg + (long)h * dv + col]));
      orow[col] = (bf16)v;
    }
  }
}

// ---- real-gated linear recurrence ----------------------------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh32(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.f + tanhf(u));
}

// One token of one channel: (decay a, input b) of S <- a S + b.
__device__ __forceinline__ void rglru_terms(float u, float gr, float gi, float cl, float& a, float& b) {
  const float r = 1.f / (1.f + expf(-gr)), i = 1.f / (1.f + expf(-gi));
  const float la = -cl * r;
  a = expf(la);
  b = sqrtf(-expm1f(2.f * la)) * i * u;
}

// grid (sequences, channel blocks of 64), SEGS waves per workgroup: wave s scans the s-th stretch of the step's tokens for
// 64 channels. First pass: every stretch from zero, keeping only its (decay product, end value); the stretches are joined
// in order; second pass: every stretch again from its true start, writing the read-outs. A step with few tokens per
// sequence runs with one stretch and one pass.
template <typename OT, int SEGS>
__global__ __launch_bounds__(64 * SEGS) void rglru_scan_kernel(
    OT* __restrict__ out, long ldo, const float* __restrict__ u, long ldu, const float* __restrict__ gates, long ldg,
    const float* __restrict__ ypre, long ldy, const float* __restrict__ clam, float* __restrict__ state,
    const int* __restrict__ q_start, const int* __restrict__ ctx, const int* __restrict__ slots, int W, int bw, int state_rows) {
  __shared__ float seg_a[SEGS][64], seg_b[SEGS][64];
  const int b = blockIdx.x;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  if (n <= 0 || slot < 0 || slot >= state_rows) return;              // (whole workgroup)
  const int lane = threadIdx.x & 63, sg = SEGS == 1 ? 0 : (int)(threadIdx.x >> 6);
  const int c = blockIdx.y * 64 + lane;
  const bool on = c < W;
  const int cc = on ? c : 0;
  const int gcol = (cc / bw) * 2 * bw + cc % bw;
  const float cl = clam[cc];
  const int per = (n + SEGS - 1) / SEGS;
  const int r0 = min(n, sg * per), r1 = min(n, r0 + per);
  float S = 0.f;
  if constexpr (SEGS > 1) {
    float A = 1.f, Bv = 0.f;
    for (int r = r0; r < r1; ++r) {
      const long t = t0 + r;
      float a, bb;
      rglru_terms(u[t * ldu + cc], gates[t * ldg + gcol], gates[t * ldg + gcol + bw], cl, a, bb);
      A *= a; Bv = a * Bv + bb;
    }
    seg_a[sg][lane] = A; seg_b[sg][lane] = Bv;
    __syncthreads();
    S = c0 > 0 ? state[(long)slot * W + cc] : 0.f;
    for (int k = 0; k < sg; ++k) S = seg_a[k][lane] * S + seg_b[k][lane];
  } else {
    S = c0 > 0 ? state[(long)slot * W + cc] : 0.f;
  }
  for (int r = r0; r < r1; ++r) {
    const long t = t0 + r;
    float a, bb;
    rglru_terms(u[t * ldu + cc], gates[t * ldg + gcol], gates[t * ldg + gcol + bw], cl, a, bb);
    S = a * S + bb;
    if (on) out[t * ldo + c] = (OT)(S * gelu_tanh32(ypre[t * ldy + c]));
  }
  // (a short step may leave the last stretches empty: the one that holds the step's last token has the end state)
  if (on && r1 == n && r1 > r0) state[(long)slot * W + c] = S;
}

// Long portions over the whole chip: the step's tokens are cut into stretches of 64 per sequence, one single-wave workgroup per
// (sequence, 64 channels, stretch). First launch: every stretch scanned from zero, its (decay product, end value) left in `ws`
// (row: the stretch's place among all stretches of the step). Second launch: a stretch folds those of the stretches before it
// onto the slot's state, scans again from there and writes; the stretch with the step's last token leaves the new state.
constexpr int kScanStretch = 64;

template <typename OT, bool APPLY>
__global__ __launch_bounds__(64) void rglru_stretch_kernel(
    OT* __restrict__ out, long ldo, const float* __restrict__ u, long ldu, const float* __restrict__ gates, long ldg,
    const float* __restrict__ ypre, long ldy, const float* __restrict__ clam, float* __restrict__ state, float* __restrict__ ws,
    const int* __restrict__ q_start, const int* __restrict__ ctx, const int* __restrict__ slots, int W, int bw, int state_rows) {
  const int b = blockIdx.x, sg = blockIdx.z;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  const int r0 = sg * kScanStretch;
  if (r0 >= n || slot < 0 || slot >= state_rows) return;
  const int r1 = min(n, r0 + kScanStretch);
  const int c = blockIdx.y * 64 + threadIdx.x;
  const bool on = c < W;
  const int cc = on ? c : 0;
  const int gcol = (cc / bw) * 2 * bw + cc % bw;
  const float cl = clam[cc];
  // this sequence's rows of ws (rows of different sequences never meet): the slot's state as the step found it, then a row per
  // stretch. The second launch reads the old state from there: by then the slot may already hold the new one.
  const long row0 = t0 / kScanStretch + 2 * b;
  if constexpr (!APPLY) {
    if (sg == 0 && on) ws[(row0 * W + c) * 2 + 1] = c0 > 0 ? state[(long)slot * W + c] : 0.f;
    float A = 1.f, Bv = 0.f;
    for (int r = r0; r < r1; ++r) {
      const long t = t0 + r;
      float a, bb;
      rglru_terms(u[t * ldu + cc], gates[t * ldg + gcol], gates[t * ldg + gcol + bw], cl, a, bb);
      A *= a; Bv = a * Bv + bb;
    }
    if (on) { ws[((row0 + 1 + sg) * W + c) * 2] = A; ws[((row0 + 1 + sg) * W + c) * 2 + 1] = Bv; }
  } else {
    float S = ws[(row0 * W + cc) * 2 + 1];
    for (int k = 0; k < sg; ++k) S = ws[((row0 + 1 + k) * W + cc) * 2] * S + ws[((row0 + 1 + k) * W + cc) * 2 + 1];
    for (int r = r0; r < r1; ++r) {
      const long t = t0 + r;
      float a, bb;
      rglru_terms(u[t * ldu + cc], gates[t * ldg + gcol], gates[t * ldg + gcol + bw], cl, a, bb);
      S = a * S + bb;
      if (on) out[t * ldo + c] = (OT)(S * gelu_tanh32(ypre[t * ldy + c]));
    }
    if (on && r1 == n) state[(long)slot * W + c] = S;
  }
}

// ---- activation, scaling ---------------------------------------------------------------------------------------------
template <typename OT>
__global__ __launch_bounds__(256) void xielu_kernel(OT* __restrict__ act, const float* __restrict__ z, int M, int F, long ldz,
                                                    long lda, const float* __restrict__ pq) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)M * F) return;
  const int m = (int)(i / F), c = (int)(i % F);
  const float ap = pq[0], aq = pq[1];          // softplus(p), 1/2 + softplus(q)
  const float v = z[(long)m * ldz + c];
  const float r = v > 0.f ? ap * v * v + 0.5f * v : aq * (expm1f(v) - v) + 0.5f * v;
  act[(long)m * lda + c] = (OT)r;
}

__global__ __launch_bounds__(256) void scale_rows_kernel(float* __restrict__ x, int M, int N, long ld, float s) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)M * N) return;
  x[(i / N) * ld + i % N] *= s;
}

}  // namespace dlia

using namespace dlia;

extern "C" void dlia_par_norm(void* out, int out_f32, float* out32, float* x, const float* ya, const float* yb, const float* ls1,
                              const float* ls2, const float* w, float* carry, const int* tok_seq, int T, int state_rows, int H,
                              long ldx, long ldya, long ldyb, long ldo, float eps, hipStream_t stream) {
  if (T <= 0) return;
  if (out_f32 || !out)
    hipLaunchKernelGGL(par_norm_kernel<float>, dim3(T), dim3(kParThreads), 0, stream, (float*)out, out32, x, ya, yb, ls1, ls2, w,
                       carry, tok_seq, T, state_rows, H, ldx, ldya, ldyb, ldo, eps);
  else
    hipLaunchKernelGGL(par_norm_kernel<bf16>, dim3(T), dim3(kParThreads), 0, stream, (bf16*)out, out32, x, ya, yb, ls1, ls2, w,
                       carry, tok_seq, T, state_rows, H, ldx, ldya, ldyb, ldo, eps);
}

extern "C" void dlia_token_shift(void* out, int out_f32, const float* n32, const float* carry, const float* mu, const int* tok_pos,
                                 const int* tok_seq, int T, int state_rows, int H, long ldo, hipStream_t stream) {
  if (T <= 0) return;
  if (out_f32)
    hipLaunchKernelGGL(token_shift_kernel<float>, dim3(T), dim3(kParThreads), 0, stream, (float*)out, n32, carry, mu, tok_pos,
                       tok_seq, state_rows, H, ldo);
  else
    hipLaunchKernelGGL(token_shift_kernel<bf16>, dim3(T), dim3(kParThreads), 0, stream, (bf16*)out, n32, carry, mu, tok_pos,
                       tok_seq, state_rows, H, ldo);
}

extern "C" void dlia_rope_cache_write(float* q, long ldq, int q_vecs, int q_stride, int q_off, void* q_out, long ldqo, int q_cols,
                                      float* kv, long ldkv, int k_cols, int k_vecs, int k_stride, int k_off, int v_src, int v_cols,
                                      int v_t, void* kcache, void* vcache, int f32, int G, int dims, int interleaved, const float* cos_t,
                                      const float* sin_t, int table_pos, const int* tok_pos, const int* tok_seq,
                                      const int* block_table, int T, int max_blocks, int num_blocks, int table_rows,
                                      hipStream_t stream) {
  if (T <= 0) return;
  if (f32)
    hipLaunchKernelGGL(rope_cache_write_kernel<float>, dim3(T), dim3(kParThreads), 0, stream, q, ldq, q_vecs, q_stride, q_off,
                       (float*)q_out, ldqo, q_cols, kv, ldkv, k_cols, k_vecs, k_stride, k_off, v_src, v_cols, v_t, (float*)kcache,
                       (float*)vcache, G, dims, interleaved, cos_t, sin_t, table_pos, tok_pos, tok_seq, block_table, max_blocks,
                       num_blocks, table_rows);
  else
    hipLaunchKernelGGL(rope_cache_write_kernel<bf16>, dim3(T), dim3(kParThreads), 0, stream, q, ldq, q_vecs, q_stride, q_off,
                       (bf16*)q_out, ldqo, q_cols, kv, ldkv, k_cols, k_vecs, k_stride, k_off, v_src, v_cols, v_t, (bf16*)kcache,
                       (bf16*)vcache, G, dims, interleaved, cos_t, sin_t, table_pos, tok_pos, tok_seq, block_table, max_blocks,
                       num_blocks, table_rows);
}

template <typename T, typename OT>
static void launch_multi(int maps, dim3 grid, hipStream_t stream, void* out, long ldo, const float* q, long ldq, int q_head,
                         const void* kc, int k_row, const void* vc, int v_row, int v_off, const int* tok_pos, const int* tok_seq,
                         const int* table, int items, int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv,
                         float scale, int window, int keep_first, float softcap, float lam, float post, float eps,
                         const float* gate, long ldg, int vec, int Gk, int chunk, const float* sink) {
  if (maps == 2)
    hipLaunchKernelGGL((multi_attention_kernel<T, OT, 2>), grid, dim3(256), 0, stream, (OT*)out, ldo, q, ldq, q_head, (const T*)kc,
                       k_row, (const T*)vc, v_row, v_off, tok_pos, tok_seq, table, items, max_blocks, num_blocks, table_rows, H, G,
                       d, dv, scale, window, keep_first, softcap, lam, post, eps, gate, ldg, vec, Gk, chunk, sink);
  else
    hipLaunchKernelGGL((multi_attention_kernel<T, OT, 1>), grid, dim3(256), 0, stream, (OT*)out, ldo, q, ldq, q_head, (const T*)kc,
                       k_row, (const T*)vc, v_row, v_off, tok_pos, tok_seq, table, items, max_blocks, num_blocks, table_rows, H, G,
                       d, dv, scale, window, keep_first, softcap, lam, post, eps, gate, ldg, vec, Gk, chunk, sink);
}

extern "C" void dlia_multi_attention(void* out, long ldo, const float* q, long ldq, int q_head, const void* kcache, int k_row,
                                     const void* vcache, int v_row, int v_off, int f32, const int* tok_pos, const int* tok_seq,
                                     const int* block_table, int T, int max_blocks, int num_blocks, int table_rows, int H, int G,
                                     int d, int dv, int maps, float scale, int window, int keep_first, float softcap, float lam,
                                     float post, float eps, const float* gate, long ldg, int Gk, int chunk, const float* sink,
                                     hipStream_t stream) {
  const int items = T * H;
  if (items <= 0) return;
  const dim3 grid((items + 3) / 4);
  const int per = f32 ? 4 : 8;
  const int vec = d % per == 0 && k_row % per == 0 && (uintptr_t)kcache % 16 == 0;
  if (f32)
    launch_multi<float, float>(maps, grid, stream, out, ldo, q, ldq, q_head, kcache, k_row, vcache, v_row, v_off, tok_pos, tok_seq,
                               block_table, items, max_blocks, num_blocks, table_rows, H, G, d, dv, scale, window, keep_first,
                               softcap, lam, post, eps, gate, ldg, vec, Gk, chunk, sink);
  else
    launch_multi<bf16, bf16>(maps, grid, stream, out, ldo, q, ldq, q_head, kcache, k_row, vcache, v_row, v_off, tok_pos, tok_seq,
                             block_table, items, max_blocks, num_blocks, table_rows, H, G, d, dv, scale, window, keep_first,
                             softcap, lam, post, eps, gate, ldg, vec, Gk, chunk, sink);
}

extern "C" long dlia_rglru_scan_ws_floats(int rows, int B, int W) { return ((long)rows / kScanStretch + 2 * B + 2) * W * 2; }

extern "C" void dlia_rglru_scan(void* out, int out_f32, long ldo, const float* u, long ldu, const float* gates, long ldg,
                                const float* ypre, long ldy, const float* clam, float* state, const int* q_start, const int* ctx,
                                const int* slots, int B, int max_q, int W, int bw, int state_rows, float* ws, long ws_floats, int rows,
                                hipStream_t stream) {
  if (B <= 0 || max_q <= 0) return;
  if (max_q >= 128 && ws && ws_floats >= dlia_rglru_scan_ws_floats(rows, B, W)) {
    const dim3 grid(B, (W + 63) / 64, (max_q + kScanStretch - 1) / kScanStretch);
#define DLIA_STRETCH(OT, APPLY)                                                                                                \
  hipLaunchKernelGGL((rglru_stretch_kernel<OT, APPLY>), grid, dim3(64), 0, stream, (OT*)out, ldo, u, ldu, gates, ldg, ypre, ldy, clam, \
                     state, ws, q_start, ctx, slots, W, bw, state_rows)
    if (out_f32) { DLIA_STRETCH(float, false); DLIA_STRETCH(float, true); }
    else { DLIA_STRETCH(bf16, false); DLIA_STRETCH(bf16, true); }
#undef DLIA_STRETCH
    return;
  }
  const dim3 grid(B, (W + 63) / 64);
#define DLIA_RGLRU(OT, SEGS)                                                                                              \
  hipLaunchKernelGGL((rglru_scan_kernel<OT, SEGS>), grid, dim3(64 * SEGS), 0, stream, (OT*)out, ldo, u, ldu, gates, ldg, ypre, \
                     ldy, clam, state, q_start, ctx, slots, W, bw, state_rows)
  if (max_q >= 256) {
    if (out_f32) DLIA_RGLRU(float, 16); else DLIA_RGLRU(bf16, 16);
  } else if (max_q >= 16) {
    if (out_f32) DLIA_RGLRU(float, 4); else DLIA_RGLRU(bf16, 4);
  } else {
    if (out_f32) DLIA_RGLRU(float, 1); else DLIA_RGLRU(bf16, 1);
  }
#undef DLIA_RGLRU
}

extern "C" void dlia_xielu(void* act, int out_f32, const float* z, int M, int F, long ldz, long lda, const float* pq,
                           hipStream_t stream) {
  const long n = (long)M * F;
  if (n <= 0) return;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (out_f32) hipLaunchKernelGGL(xielu_kernel<float>, grid, dim3(256), 0, stream, (float*)act, z, M, F, ldz, lda, pq);
  else hipLaunchKernelGGL(xielu_kernel<bf16>, grid, dim3(256), 0, stream, (bf16*)act, z, M, F, ldz, lda, pq);
}

extern "C" void dlia_scale_rows(float* x, int M, int N, long ld, float s, hipStream_t stream) {
  const long n = (long)M * N;
  if (n <= 0) return;
  hipLaunchKernelGGL(scale_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, M, N, ld, s);
}

// The merge alone, for other kernels that leave (maximum, sum, weighted values) per key split in the same layout:
// part [items = tokens x heads][nz][dv + 2] with the maximum at [dv] and the sum at [dv + 1]; one score map.
extern "C" void dlia_tile_merge(void* out, long ldo, const float* part, int items, int H, int dv, int nz, const float* gate, long ldg,
                                const float* sink, hipStream_t stream) {
  if (items <= 0) return;
  hipLaunchKernelGGL(dlia::tile_merge_kernel<1>, dim3((items + 3) / 4), dim3(256), 0, stream, (dlia::bf16*)out, ldo, part, items, H, dv, nz,
                     0.f, 1.f, 0.f, gate, ldg, sink);
}

extern "C" int dlia_tile_attention_tile_groups(int G, int Gk) { return tile_all_heads(G, Gk) ? 1 : G; }

extern "C" int dlia_tile_attention_splits(int B, int H, int G) {
  // single-token steps: enough workgroups for the chip whatever the batch (a token's key blocks are dealt out to them)
  const int per = B * G * ((H / G + 15) / 16);
  int z = 1;
  while (z < 16 && per * z < 1024) z <<= 1;
  return z;
}

extern "C" int dlia_tile_attention(void* out, long ldo, const void* q, long ldq, int q_head, const void* kcache, int k_row,
                                   const void* vt, const int* q_start, const int* ctx, const int* slots, const int* block_table,
                                   int B, int max_q, int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv,
                                   int maps, float scale, int window, int keep_first, float softcap, float lam, float post,
                                   float eps, const float* gate, long ldg, float* part, long part_floats, int Gk, int chunk,
                                   const float* sink, hipStream_t stream) {
  if (B <= 0 || max_q <= 0) return 0;
  if (Gk != G && Gk != 1) return 1;
  if (d % 8 || k_row % 8 || q_head % 8 || ldq % 8 || maps * d > 1024 || dv > 512 || (maps != 1 && maps != 2)) return 1;
  const bool head_rows = max_q == 1;
  const int tiles = (max_q + 15) / 16, group = H / G;
  const int dvt = dv <= 64 ? 4 : dv <= 128 ? 8 : dv <= 256 ? 16 : 32;
  const size_t qtile = (size_t)16 * (maps * d + 8) * sizeof(bf16);
  int nw = head_rows ? 1 : (group % 4 == 0 || G == 1) && H >= 4 ? 4 : (group % 2 == 0 && H >= 2 ? 2 : 1);
  while (nw > 1 && nw * qtile > 65536) nw >>= 1;           // (a workgroup's LDS)
  const bool all_heads = head_rows && tile_all_heads(G, Gk);
  const int nz = head_rows ? dlia_tile_attention_splits(B, H, all_heads ? 1 : G) : 1;
  const dim3 grid(B * tiles, all_heads ? (H + 15) / 16 : head_rows ? G * ((group + 15) / 16) : (H + nw - 1) / nw, nz);
  const size_t lds = nw * qtile;
  if (lds > 65536) return 1;
  if (head_rows && (!part || part_floats < (long)B * H * maps * nz * (dv + 2))) return 2;
#define DLIA_TILE_KS(MAPS, DVT, KS)                                                                                                  \
  do {                                                                                                                           \
    if (head_rows)                                                                                                               \
      hipLaunchKernelGGL((tile_attention_kernel<MAPS, DVT, true, KS>), grid, dim3(64), lds, stream, (bf16*)out, ldo, (const bf16*)q, ldq, \
                         q_head, (const bf16*)kcache, k_row, (const bf16*)vt, q_start, ctx, slots, block_table, tiles, max_blocks,   \
                         num_blocks, table_rows, H, G, d, dv, scale, window, keep_first, softcap, lam, post, eps, gate, ldg, part, Gk, chunk, sink);  \
    else                                                                                                                         \
      hipLaunchKernelGGL((tile_attention_kernel<MAPS, DVT, false, KS>), grid, dim3(64 * nw), lds, stream, (bf16*)out, ldo,              \
                         (const bf16*)q, ldq, q_head, (const bf16*)kcache, k_row, (const bf16*)vt, q_start, ctx, slots, block_table, \
                         tiles, max_blocks, num_blocks, table_rows, H, G, d, dv, scale, window, keep_first, softcap, lam, post, eps,  \
                         gate, ldg, part, Gk, chunk, sink);                                                                      \
  } while (0)
  // (a map's whole key row in flight when it is long and the registers allow: one wait per block instead of four)
#define DLIA_TILE(MAPS, DVT)                                            \
  do {                                                                  \
    if (MAPS == 1 && d > 128) DLIA_TILE_KS(MAPS, DVT, (MAPS == 1 ? 16 : 4)); \
    else DLIA_TILE_KS(MAPS, DVT, 4);                                   \
  } while (0)
  if (maps == 2) {
    if (dvt == 4) DLIA_TILE(2, 4); else if (dvt == 8) DLIA_TILE(2, 8); else if (dvt == 16) DLIA_TILE(2, 16); else DLIA_TILE(2, 32);
  } else {
    if (dvt == 4) DLIA_TILE(1, 4); else if (dvt == 8) DLIA_TILE(1, 8); else if (dvt == 16) DLIA_TILE(1, 16); else DLIA_TILE(1, 32);
  }
  if (head_rows) {
    const int items = B * H;
    if (maps == 2)
      hipLaunchKernelGGL(tile_merge_kernel<2>, dim3((items + 3) / 4), dim3(256), 0, stream, (bf16*)out, ldo, part, items, H, dv, nz, lam,
                         post, eps, gate, ldg, sink);
    else
      hipLaunchKernelGGL(tile_merge_kernel<1>, dim3((items + 3) / 4), dim3(256), 0, stream, (bf16*)out, ldo, part, items, H, dv, nz, lam,
                         post, eps, gate, ldg, sink);
  }
#undef DLIA_TILE
#undef DLIA_TILE_KS
  return 0;
}
