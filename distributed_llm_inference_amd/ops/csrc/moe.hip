// Routed feed-forward (mixture of experts) without a host round trip: routing, a plan that sorts the step's (token, choice)
// pairs by expert into 32-row tiles, the experts' two GEMMs over those tiles, and the weighted sum per token.
//
//   moe_route    one thread per token. Scores are sigmoids of the fp32 router logits, or their softmax over all router outputs.
//                The choice goes by score + correction[e] when a correction is given. Experts are split into `groups`
//                contiguous blocks of equal size; a block is ranked by its best `group_rank` (1 or 2) choice scores added up;
//                the `keep` best blocks stay; the `top` best experts of those are chosen (equal scores: the lower index),
//                weighted score / (sum + 1e-20) * scale, or score * scale without the division.
//   moe_plan     one workgroup. Pairs whose choice is not a real expert (an identity expert: index >= E) get row -1 and no
//                place in a tile. Counts the pairs per expert, lays the experts' row ranges out one after the other, each
//                padded to whole 32-row tiles, and writes for every padded row its token (or -1), for every pair its row,
//                for every tile its expert; tiles[0] holds the number of tiles. Rows of one expert are in no fixed order:
//                every row is computed on its own, so the order does not reach the results.
//   moe_up       grid (column blocks, tiles): act[row, f] = g s(1.702 g) (u + 1), g = min(x . Wg[e][f], limit),
//                u = clamp(x . Wu[e][f], -limit, limit), x the row's token; with limit <= 0 the plain silu(g) * u.
//                Gate and up accumulate over the same A fragments.
//   moe_down     y[row, c] = act[row] . Wd[e][c] in fp32.
//   moe_combine  out[t, :] = sum over the token's choices of weight * y[row, :], in the order of the choices (fp32); a choice
//                without a row (an identity expert) contributes weight * x[t, :].
// Operands are bf16 (16x16x32 MFMA) or fp32 (16x16x4 MFMA, true 32-bit), fragments read straight from the K-contiguous rows.
#include "common.h"
#include "frag.h"
#include "launch.h"

namespace dlia {

constexpr int kMoeMaxExperts = 256;
constexpr int kMoeRows = 32;           // rows of a plan tile (steps with few rows), kMoeBigRows for the LDS-tiled kernel
constexpr int kMoeBigRows = 128;

// An expert's activation from its gate and up pre-activations.
__device__ __forceinline__ float expert_act(float g, float u, float limit) {
  if (limit > 0.f) {
    const float gv = fminf(g, limit), uv = fminf(fmaxf(u, -limit), limit);
    return gv / (1.f + expf(-1.702f * gv)) * (uv + 1.f);
  }
  return g / (1.f + expf(-g)) * u;
}

__global__ __launch_bounds__(64) void moe_route_kernel(int* __restrict__ sel, float* __restrict__ wts,
                                                       const float* __restrict__ logits, long ld, int T, int E, int top,
                                                       int groups, int keep, float scale, const float* __restrict__ corr,
                                                       int softmax, int group_rank, int renorm) {
  const int t = blockIdx.x * 64 + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (long)t * ld;
  const int per = E / groups;
  float zmax = 0.f, zinv = 1.f;
  if (softmax) {
    zmax = -INFINITY;
    for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, z[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf(z[e] - zmax);
    zinv = 1.f / sum;
  }
  auto score = [&](int e) { return softmax ? expf(z[e] - zmax) * zinv : 1.f / (1.f + expf(-z[e])); };
  auto choice = [&](int e) { return corr ? score(e) + corr[e] : score(e); };
  // the groups that stay: `keep` times the best group not yet taken
  unsigned long long gmask[4] = {0ull, 0ull, 0ull, 0ull};
  for (int r = 0; r < keep; ++r) {
    int best = -1; float bs = -INFINITY;
    for (int g = 0; g < groups; ++g) {
      if (gmask[g >> 6] >> (g & 63) & 1ull) continue;
      float a = -INFINITY, b = -INFINITY;             // the block's best two choice scores
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float s = choice(e);
        if (s > a) { b = a; a = s; } else if (s > b) b = s;
      }
      const float gs = a + (group_rank >= 2 && b > -INFINITY ? b : 0.f);
      if (best < 0 || gs > bs) { bs = gs; best = g; }
    }
    if (best >= 0) gmask[best >> 6] |= 1ull << (best & 63);
  }
  unsigned long long emask[4] = {0ull, 0ull, 0ull, 0ull};
  float total = 0.f;
  for (int r = 0; r < top; ++r) {
    int best = -1; float bs = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const int g = e / per;
      if (!(gmask[g >> 6] >> (g & 63) & 1ull) || (emask[e >> 6] >> (e & 63) & 1ull)) continue;
      const float s = choice(e);
      if (best < 0 || s > bs) { bs = s; best = e; }
    }
    if (best < 0) best = 0;
    emask[best >> 6] |= 1ull << (best & 63);
    const float w = score(best);
    sel[(long)t * top + r] = best;
    wts[(long)t * top + r] = w;
    total += w;
  }
  const float inv = renorm ? scale / (total + 1e-20f) : scale;
  for (int r = 0; r < top; ++r) wts[(long)t * top + r] *= inv;
}

// tiles: [0] number of tiles, [1 + i] expert of tile i. row_tok [max_rows], pair_row [T * top].
__global__ __launch_bounds__(1024) void moe_plan_kernel(int* __restrict__ tiles, int* __restrict__ row_tok,
                                                        int* __restrict__ pair_row, const int* __restrict__ sel, int pairs,
                                                        int top, int E, int max_rows, int tile_rows) {
  __shared__ int count[kMoeMaxExperts], start[kMoeMaxExperts], fill[kMoeMaxExperts];
  __shared__ int ntiles;
  for (int e = threadIdx.x; e < E; e += 1024) { count[e] = 0; fill[e] = 0; }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024)
    if (sel[i] < E) atomicAdd(&count[sel[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      const int n = (count[e] + tile_rows - 1) / tile_rows;
      for (int i = 0; i < n; ++i) tiles[1 + nt + i] = e;
      nt += n; at += n * tile_rows;
    }
    tiles[0] = nt;
    ntiles = nt;
  }
  __syncthreads();
  const int used = ntiles * tile_rows;
  for (int i = threadIdx.x; i < max_rows; i += 1024) row_tok[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024) {
    const int e = sel[i];
    if (e >= E) { pair_row[i] = -1; continue; }                      // (an identity expert: no row)
    const int r = start[e] + atomicAdd(&fill[e], 1);
    if (r < max_rows && r < used) { row_tok[r] = i / top; pair_row[i] = r; }
  }
}

// Row tiles of the plan: 32 rows. A workgroup of four waves covers one row tile by 128 (up) or 256 (down) output columns; a
// wave holds both 16-row halves of the tile against its 32 (64) columns, so every fragment it loads feeds two or more MFMAs,
// and the fragments of the next k-step are on their way while the current ones are multiplied.
constexpr int kMoeTile = kMoeRows;

template <typename T, typename OT, int NJ>
__global__ __launch_bounds__(256) void moe_up_kernel(OT* __restrict__ act, const T* __restrict__ x, const T* __restrict__ wg,
                                                     const T* __restrict__ wu, const int* __restrict__ tiles,
                                                     const int* __restrict__ row_tok, int F, int K, long ldx, long lda,
                                                     float limit, int vec_ok) {
  constexpr int VEC = 16 / sizeof(T), KS = 4 * VEC;
  const int tile = blockIdx.y;
  if (tile >= tiles[0]) return;
  const int e = tiles[1 + tile];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int f0 = (blockIdx.x * 4 + wave) * 16 * NJ;
  if (f0 >= F) return;
  const T* arow[2]; long wrow[NJ]; bool av[2], wv[NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int tok = row_tok[tile * kMoeTile + i * 16 + r16];
    av[i] = tok >= 0;
    arow[i] = x + (long)(av[i] ? tok : 0) * ldx;
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    wv[j] = f0 + j * 16 + r16 < F;
    wrow[j] = ((long)e * F + (wv[j] ? f0 + j * 16 + r16 : 0)) * K;
  }
  f32x4 ag[2][NJ], au[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) { ag[i][j] = f32x4{0.f, 0.f, 0.f, 0.f}; au[i][j] = f32x4{0.f, 0.f, 0.f, 0.f}; }
  u32x4 a[2], g[NJ], u[NJ], an[2], gn[NJ], un[NJ];
  auto load = [&](u32x4 (&fa)[2], u32x4 (&fg)[NJ], u32x4 (&fu)[NJ], int k0) {
    const int k = k0 + kq * VEC;
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[i] = load_frag<T>(arow[i], k, K, av[i], vec_ok);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      fg[j] = load_frag<T>(wg + wrow[j], k, K, wv[j], vec_ok);
      fu[j] = load_frag<T>(wu + wrow[j], k, K, wv[j], vec_ok);
    }
  };
  load(a, g, u, 0);
  for (int k0 = 0; k0 < K; k0 += KS) {
    if (k0 + KS < K) load(an, gn, un, k0 + KS);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) { ag[i][j] = mma_frag(T{}, a[i], g[j], ag[i][j]); au[i][j] = mma_frag(T{}, a[i], u[j], au[i][j]); }
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = an[i];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { g[j] = gn[j]; u[j] = un[j]; }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int col = f0 + j * 16 + r16;
      if (col >= F) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = tile * kMoeTile + i * 16 + kq * 4 + r;
        act[(long)row * lda + col] = (OT)expert_act(ag[i][j][r], au[i][j][r], limit);
      }
    }
}

template <typename T, int NJ>
__global__ __launch_bounds__(256) void moe_down_kernel(float* __restrict__ y, const T* __restrict__ act, const T* __restrict__ wd,
                                                       const int* __restrict__ tiles, const int* __restrict__ row_tok,
                                                       int H, int F, long lda, int vec_ok) {
  constexpr int VEC = 16 / sizeof(T), KS = 4 * VEC;
  const int tile = blockIdx.y;
  if (tile >= tiles[0]) return;
  const int e = tiles[1 + tile];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int c0 = (blockIdx.x * 4 + wave) * 16 * NJ;
  if (c0 >= H) return;
  const T* arow[2]; const T* wrow[NJ]; bool av[2], wv[NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    av[i] = row_tok[tile * kMoeTile + i * 16 + r16] >= 0;
    arow[i] = act + (long)(tile * kMoeTile + i * 16 + r16) * lda;
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    wv[j] = c0 + j * 16 + r16 < H;
    wrow[j] = wd + ((long)e * H + (wv[j] ? c0 + j * 16 + r16 : 0)) * F;
  }
  f32x4 acc[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  u32x4 a[2], w[NJ], an[2], wn[NJ];
  auto load = [&](u32x4 (&fa)[2], u32x4 (&fw)[NJ], int k0) {
    const int k = k0 + kq * VEC;
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[i] = load_frag<T>(arow[i], k, F, av[i], vec_ok);
#pragma unroll
    for (int j = 0; j < NJ; ++j) fw[j] = load_frag<T>(wrow[j], k, F, wv[j], vec_ok);
  };
  load(a, w, 0);
  for (int k0 = 0; k0 < F; k0 += KS) {
    if (k0 + KS < F) load(an, wn, k0 + KS);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = mma_frag(T{}, a[i], w[j], acc[i][j]);
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = an[i];
#pragma unroll
    for (int j = 0; j < NJ; ++j) w[j] = wn[j];
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int col = c0 + j * 16 + r16;
      if (col >= H) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[(long)(tile * kMoeTile + i * 16 + kq * 4 + r) * H + col] = acc[i][j][r];
    }
}

// Steps with many rows (prompts): 128-row tiles, operands staged through LDS. A workgroup owns one row tile by 128 weight rows —
// for the up projection 64 gate rows and the 64 up rows of the same columns, so the activation is formed in registers; for the
// down projection 128 output columns — and walks K in steps of 32: every thread brings four 16-byte pieces of the next step
// (two of the rows, gathered through the plan for the up projection; two of the weights) into registers while the current
// step is multiplied, then parks them in the other half of a double buffer. Rows are 80 bytes apart in LDS, which spreads the
// fragment reads of a 16-row tile over the banks. A wave multiplies 32 rows by all 128 weight rows: 10 fragment reads for 16
// MFMAs. bf16, K a multiple of 32 with 16-byte aligned rows (the caller falls back to the register-tiled kernels otherwise).
constexpr int kBigStride = 40;          // bf16 elements between rows in LDS (64 bytes of data + 16 of padding)

template <bool UP>
__global__ __launch_bounds__(256) void moe_big_kernel(bf16* __restrict__ act_out, float* __restrict__ y_out, const bf16* __restrict__ a,
                                                      const bf16* __restrict__ w0, const bf16* __restrict__ w1,
                                                      const int* __restrict__ tiles, const int* __restrict__ row_tok, int N, int K,
                                                      long lda, long ldo, float limit) {
  __shared__ __attribute__((aligned(16))) bf16 lds[2][256 * kBigStride];
  const int tile = blockIdx.y;
  if (tile >= tiles[0]) return;
  const int e = tiles[1 + tile];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r16 = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.x * (UP ? 64 : 128);                  // first output column of the workgroup
  // the four pieces this thread stages per k-step: pieces 2 tid, 2 tid + 1 of the 512 row pieces, and of the 512 weight pieces
  const bf16* src[4]; bool ok[4]; int dst[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid * 2 + i, row = c >> 2, part = c & 3;
    const int grow = tile * kMoeBigRows + row;
    if constexpr (UP) { const int tok = row_tok[grow]; ok[i] = tok >= 0; src[i] = a + (long)(ok[i] ? tok : 0) * lda + part * 8; }
    else { ok[i] = row_tok[grow] >= 0; src[i] = a + (long)grow * lda + part * 8; }
    dst[i] = row * kBigStride + part * 8;
    // weights: LDS rows 128 .. 255
    int wr; const bf16* base;
    if constexpr (UP) { wr = n0 + (row & 63); base = row < 64 ? w0 : w1; }
    else { wr = n0 + row; base = w0; }
    ok[2 + i] = wr < N;
    src[2 + i] = base + ((long)e * N + (ok[2 + i] ? wr : 0)) * K + part * 8;
    dst[2 + i] = (128 + row) * kBigStride + part * 8;
  }
  u32x4 st[4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) st[i] = ok[i] ? ld16(src[i] + k0) : u32x4{0u, 0u, 0u, 0u};
  };
  auto park = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(&lds[buf][dst[i]]) = st[i];
  };
  f32x4 acc[2][8];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  park(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool more = k0 + 32 < K;
    if (more) fetch(k0 + 32);
    u32x4 fa[2], fw[8];
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[i] = *reinterpret_cast<const u32x4*>(&lds[buf][(wave * 32 + i * 16 + r16) * kBigStride + kq * 8]);
#pragma unroll
    for (int j = 0; j < 8; ++j) fw[j] = *reinterpret_cast<const u32x4*>(&lds[buf][(128 + j * 16 + r16) * kBigStride + kq * 8]);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = mfma16(fa[i], fw[j], acc[i][j]);
    if (more) park(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const long row = (long)tile * kMoeBigRows + wave * 32 + i * 16 + kq * 4 + r;
      if constexpr (UP) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int col = n0 + j * 16 + r16;
          if (col >= N) continue;
          act_out[row * ldo + col] = (bf16)expert_act(acc[i][j][r], acc[i][j + 4][r], limit);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int col = n0 + j * 16 + r16;
          if (col < N) y_out[row * ldo + col] = acc[i][j][r];
        }
      }
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y,
                                                          const int* __restrict__ pair_row, const float* __restrict__ wts,
                                                          int H, int top, long ldo, const float* __restrict__ x, long ldx) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < H; c += 256) {
    float s = 0.f;
    for (int r = 0; r < top; ++r) {
      const int row = pair_row[(long)t * top + r];
      s += wts[(long)t * top + r] * (row >= 0 ? y[(long)row * H + c] : (x ? x[(long)t * ldx + c] : 0.f));
    }
    out[(long)t * ldo + c] = s;
  }
}

}  // namespace dlia

extern "C" void dlia_moe_route(int* sel, float* wts, const float* logits, long ld, int T, int E, int top, int groups, int keep,
                               float scale, const float* corr, int softmax, int group_rank, int renorm, hipStream_t stream) {
  if (T <= 0) return;
  hipLaunchKernelGGL(dlia::moe_route_kernel, dim3((T + 63) / 64), dim3(64), 0, stream, sel, wts, logits, ld, T, E, top, groups,
                     keep, scale, corr, softmax, group_rank, renorm);
}

extern "C" void dlia_moe_plan(int* tiles, int* row_tok, int* pair_row, const int* sel, int pairs, int top, int E, int max_rows,
                              int tile_rows, hipStream_t stream) {
  hipLaunchKernelGGL(dlia::moe_plan_kernel, dim3(1), dim3(1024), 0, stream, tiles, row_tok, pair_row, sel, pairs, top, E, max_rows,
                     tile_rows);
}

// Steps with few rows (decoding) take narrow column blocks: more workgroups stream the experts' weights at once.
template <typename T, typename OT, int NJ>
static void launch_moe_up(void* act, const void* x, const void* wg, const void* wu, const int* tiles, const int* row_tok, int max_tiles,
                          int F, int K, long ldx, long lda, float limit, int ok, hipStream_t stream) {
  const dim3 grid((F + 64 * NJ - 1) / (64 * NJ), max_tiles);
  hipLaunchKernelGGL((dlia::moe_up_kernel<T, OT, NJ>), grid, dim3(256), 0, stream, (OT*)act, (const T*)x, (const T*)wg, (const T*)wu,
                     tiles, row_tok, F, K, ldx, lda, limit, ok);
}
template <typename T, int NJ>
static void launch_moe_down(float* y, const void* act, const void* wd, const int* tiles, const int* row_tok, int max_tiles, int H, int F,
                            long lda, int ok, hipStream_t stream) {
  const dim3 grid((H + 64 * NJ - 1) / (64 * NJ), max_tiles);
  hipLaunchKernelGGL((dlia::moe_down_kernel<T, NJ>), grid, dim3(256), 0, stream, y, (const T*)act, (const T*)wd, tiles, row_tok, H, F, lda, ok);
}

extern "C" void dlia_moe_up(void* act, const void* x, const void* wg, const void* wu, int f32, const int* tiles, const int* row_tok,
                            int max_tiles, int wide, int F, int K, long ldx, long lda, float limit, int tile_rows, hipStream_t stream) {
  if (max_tiles <= 0) return;
  if (tile_rows == dlia::kMoeBigRows) {
    hipLaunchKernelGGL(dlia::moe_big_kernel<true>, dim3((F + 63) / 64, max_tiles), dim3(256), 0, stream, (dlia::bf16*)act, (float*)nullptr,
                       (const dlia::bf16*)x, (const dlia::bf16*)wg, (const dlia::bf16*)wu, tiles, row_tok, F, K, ldx, lda, limit);
    return;
  }
  const int vec = f32 ? 4 : 8;
  const int ok = K % vec == 0 && ldx % vec == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)wg % 16 == 0 && (uintptr_t)wu % 16 == 0;
  if (f32) {
    if (wide) launch_moe_up<float, float, 2>(act, x, wg, wu, tiles, row_tok, max_tiles, F, K, ldx, lda, limit, ok, stream);
    else launch_moe_up<float, float, 1>(act, x, wg, wu, tiles, row_tok, max_tiles, F, K, ldx, lda, limit, ok, stream);
  } else {
    if (wide) launch_moe_up<dlia::bf16, dlia::bf16, 2>(act, x, wg, wu, tiles, row_tok, max_tiles, F, K, ldx, lda, limit, ok, stream);
    else launch_moe_up<dlia::bf16, dlia::bf16, 1>(act, x, wg, wu, tiles, row_tok, max_tiles, F, K, ldx, lda, limit, ok, stream);
  }
}

extern "C" void dlia_moe_down(float* y, const void* act, const void* wd, int f32, const int* tiles, const int* row_tok,
                              int max_tiles, int wide, int H, int F, long lda, int tile_rows, hipStream_t stream) {
  if (max_tiles <= 0) return;
  if (tile_rows == dlia::kMoeBigRows) {
    hipLaunchKernelGGL(dlia::moe_big_kernel<false>, dim3((H + 127) / 128, max_tiles), dim3(256), 0, stream, (dlia::bf16*)nullptr, y,
                       (const dlia::bf16*)act, (const dlia::bf16*)wd, (const dlia::bf16*)nullptr, tiles, row_tok, H, F, lda, (long)H, 0.f);
    return;
  }
  const int vec = f32 ? 4 : 8;
  const int ok = F % vec == 0 && lda % vec == 0 && (uintptr_t)act % 16 == 0 && (uintptr_t)wd % 16 == 0;
  if (f32) {
    if (wide) launch_moe_down<float, 4>(y, act, wd, tiles, row_tok, max_tiles, H, F, lda, ok, stream);
    else launch_moe_down<float, 1>(y, act, wd, tiles, row_tok, max_tiles, H, F, lda, ok, stream);
  } else {
    if (wide) launch_moe_down<dlia::bf16, 4>(y, act, wd, tiles, row_tok, max_tiles, H, F, lda, ok, stream);
    else launch_moe_down<dlia::bf16, 1>(y, act, wd, tiles, row_tok, max_tiles, H, F, lda, ok, stream);
  }
}

extern "C" void dlia_moe_combine(float* out, const float* y, const int* pair_row, const float* wts, int T, int H, int top, long ldo,
                                 const float* x, long ldx, hipStream_t stream) {
  if (T <= 0) return;
  hipLaunchKernelGGL(dlia::moe_combine_kernel, dim3(T), dim3(256), 0, stream, out, y, pair_row, wts, H, top, ldo, x, ldx);
}
