// Recurrent mixer kernels: causal short convolution with carried inputs, per-head unit vectors, and the gated
// delta rule over a per-sequence fp32 state. Everything here is fp32: inputs are the fp32 output of the mixer's
// fused input projection, the state never leaves fp32.
//
// A step is ragged: sequence b brings n = q_start[b+1] - q_start[b] new tokens after ctx[b] earlier ones and
// owns state slot slots[b]. A sequence's first step (ctx = 0) starts from zeros whatever its slot held before,
// so a slot needs no clearing when it changes hands; later steps continue from the slot.
//
//   short_conv      y[t, c] = act(bias[c] + sum_j taps[c, j] * x[t - (K-1-j), c]), act = silu or none, bias optional; inputs before the step come from the
//                   slot's K-1 carried inputs, inputs before the sequence's start are zero
//   conv_carry      the slot's carried inputs become the last K-1 inputs including this step's (runs after
//                   short_conv has read the old ones)
//   unit_heads      x / sqrt(sum x^2 + eps) * mult per (token, head), in place
//   delta_rule      per (sequence, head, block of value columns), sequential over the step's tokens:
//                   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                   with g = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b). A value column's slice of
//                   S ([d] numbers) lives in the registers of R lanes (DPT rows each), the two dot products
//                   reduce over those lanes by shuffles; k, q, v, a, b of the next token are fetched while the
//                   current one is applied.
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kConvMaxTaps = 16;

__global__ __launch_bounds__(256) void short_conv_kernel(
    float* __restrict__ y, const float* __restrict__ z, const float* __restrict__ carry, const float* __restrict__ taps,
    const int* __restrict__ q_start, const int* __restrict__ ctx, const int* __restrict__ slots, int C, int K, long ldz,
    int tokb, int state_rows, const float* __restrict__ bias, int silu) {
  const int b = blockIdx.x;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  const int r0 = blockIdx.y * tokb, r1 = min(n, r0 + tokb);
  if (r0 >= r1 || slot < 0 || slot >= state_rows) return;
  const float* st = carry + (long)slot * (K - 1) * C;
  for (int c = blockIdx.z * 256 + threadIdx.x; c < C; c += 256 * gridDim.z) {
    float w[kConvMaxTaps];
#pragma unroll
    for (int j = 0; j < kConvMaxTaps; ++j) w[j] = j < K ? taps[(long)c * K + j] : 0.f;
    const float bc = bias ? bias[c] : 0.f;
    for (int r = r0; r < r1; ++r) {
      float acc = bc;
#pragma unroll
      for (int j = 0; j < kConvMaxTaps; ++j) {
        if (j >= K) break;
        const int s = r - (K - 1 - j);
        float x;
        if (s >= 0) x = z[(long)(t0 + s) * ldz + c];
        else x = (c0 + s >= 0) ? st[(long)(K - 1 + s) * C + c] : 0.f;
        acc += w[j] * x;
      }
      y[(long)(t0 + r) * C + c] = silu ? acc / (1.f + expf(-acc)) : acc;
    }
  }
}

__global__ __launch_bounds__(256) void conv_carry_kernel(
    float* __restrict__ carry, const float* __restrict__ z, const int* __restrict__ q_start, const int* __restrict__ ctx,
    const int* __restrict__ slots, int C, int K, long ldz, int state_rows) {
  const int b = blockIdx.x;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  if (n <= 0 || slot < 0 || slot >= state_rows) return;
  float* st = carry + (long)slot * (K - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y) {
    float nv[kConvMaxTaps];
#pragma unroll
    for (int k = 0; k < kConvMaxTaps; ++k) {
      nv[k] = 0.f;
      if (k < K - 1) {
        const int p = c0 + n - (K - 1) + k;            // absolute position this entry will hold
        if (p >= c0) nv[k] = z[(long)(t0 + p - c0) * ldz + c];
        else if (p >= 0) nv[k] = st[(long)(p - c0 + K - 1) * C + c];
      }
    }
#pragma unroll
    for (int k = 0; k < kConvMaxTaps; ++k)
      if (k < K - 1) st[(long)k * C + c] = nv[k];
  }
}

__global__ __launch_bounds__(256) void unit_heads_kernel(float* __restrict__ x, int items, int heads, int d, long ld,
                                                         int scaled_heads, float mult, float eps) {
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int t = item / heads, h = item % heads, lane = lane_id();
  float* row = x + (long)t * ld + (long)h * d;
  float s = 0.f;
  for (int i = lane; i < d; i += 64) { const float v = row[i]; s += v * v; }
  s = wave_sum(s);
  const float r = rsqrtf(s + eps) * (h < scaled_heads ? mult : 1.f);
  for (int i = lane; i < d; i += 64) row[i] *= r;
}

// One workgroup per (sequence, head, block of 64 / R value columns): a COMPUTE wave that owns the state slice and
// walks the tokens, and (prompt portions) a LOADER wave that stages the operands of the chunk after the current one
// in the other half of a double buffer in LDS — per token k [dpad], q [dpad], the block's v columns, the decay g
// and beta, the two gates already evaluated (exp / log1p once per token, not once per lane). The loader keeps the
// chunk after that on its way in its registers, so neither wave waits for global memory in steady state; the two
// meet at one barrier per chunk. The compute wave's loop over tokens reads at LDS latency, and a chunk's read-outs
// leave through LDS in one coalesced write. Decode steps (one token) run the single-wave form of the same code.
template <int DPT, int R, bool DECODE, bool VEC>
__global__ __launch_bounds__(DECODE ? 64 : 128) void delta_rule_kernel(
    float* __restrict__ o, const float* __restrict__ y, const float* __restrict__ z, float* __restrict__ state,
    const float* __restrict__ A_log, const float* __restrict__ dt_bias, const int* __restrict__ q_start,
    const int* __restrict__ ctx, const int* __restrict__ slots, int G, int Hv, int d, int dv, int C, long ldz, int col_beta,
    int col_a, int cols_per_block, int state_rows, int rowlen) {
  constexpr int dpad = R * DPT, SEG = (dpad + 63) / 64;
  constexpr int CH = DECODE ? 1 : (SEG <= 2 ? 16 : (SEG <= 4 ? 8 : 4));      // tokens staged at a time
  constexpr int NBUF = DECODE ? 1 : 2;
  extern __shared__ __attribute__((aligned(16))) float smem[];       // NBUF x [CH][rowlen]: k [dpad] | q [dpad] | v [cols] | g | beta
  float* ostage = smem + NBUF * CH * rowlen;                          // [CH][cols]: the chunk's read-outs
  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = q_start[b], n = q_start[b + 1] - t0, c0 = ctx[b], slot = slots[b];
  if (n <= 0 || slot < 0 || slot >= state_rows) return;              // (whole workgroup)
  const int g = h / (Hv / G);
  const int lane = threadIdx.x & 63;
  const int wave = DECODE ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const bool computes = wave == 0, loads = DECODE || wave == 1;
  const int r = lane % R, jl = lane / R;
  const int col0 = blockIdx.z * cols_per_block;
  const int j = col0 + jl;
  const bool active = jl < cols_per_block && j < dv;
  const int i0 = r * DPT;
  float* Sp = state + (((long)slot * Hv + h) * d) * dv + (active ? j : 0);
  float s[DPT];
  if (computes) {
#pragma unroll
    for (int i = 0; i < DPT; ++i) s[i] = (c0 > 0 && active && i0 + i < d) ? Sp[(long)(i0 + i) * dv] : 0.f;
  }
  const float nA = -expf(A_log[h]), dtb = dt_bias[h];
  const long koff = (long)G * d + (long)g * d, qoff = (long)g * d, voff = 2L * G * d + (long)h * dv + col0;
  const bool has_v = lane < cols_per_block && col0 + lane < dv;
  // (the state has landed before anything else is asked of memory: the loops below carry no wait for it)
  __builtin_amdgcn_s_waitcnt(0x0F70);             // vmcnt(0)
  // VEC (d and the row length of y multiples of 4): a token's k | q image, 2 dpad floats, travels as 16-byte pieces,
  // piece f = lane + 64 u covering elements 4f .. 4f + 3 of the image; otherwise element by element.
  constexpr int SEG4 = (2 * dpad / 4 + 63) / 64;
  f32x4 p4[VEC ? CH : 1][VEC ? SEG4 : 1];
  float pk[VEC ? 1 : CH][VEC ? 1 : SEG], pq[VEC ? 1 : CH][VEC ? 1 : SEG], pv[CH], pgate = 0.f;      // (gate inputs: lane tt holds token tt's decay input, lane CH + tt its beta input)
  auto prefetch = [&](int tc) {                  // chunk at token tc: global -> registers (nothing if it is past the end)
    const int nt = min(CH, n - tc);
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      if (tt < nt) {
        const long t = t0 + tc + tt;
        const float* yr = y + t * C;
        if constexpr (VEC) {
#pragma unroll
          for (int u = 0; u < SEG4; ++u) {
            const int e = 4 * (lane + 64 * u);
            const int ek = e < dpad ? e : e - dpad;               // element within k or within q
            const float* src = yr + (e < dpad ? koff : qoff) + ek;
            p4[tt][u] = (e < 2 * dpad && ek < d) ? *reinterpret_cast<const f32x4*>(src) : f32x4{0.f, 0.f, 0.f, 0.f};
          }
        } else {
#pragma unroll
          for (int u = 0; u < SEG; ++u) {
            const int e = lane + 64 * u;
            pk[tt][u] = e < d ? yr[koff + e] : 0.f;
            pq[tt][u] = e < d ? yr[qoff + e] : 0.f;
          }
        }
        pv[tt] = has_v ? yr[voff + lane] : 0.f;
      }
    }
    if (lane < 2 * CH) {
      const int tt = lane % CH;
      if (tt < nt) pgate = z[(long)(t0 + tc + tt) * ldz + (lane < CH ? col_a : col_beta) + h];
    }
  };
  auto publish = [&](float* stage, int tc) {     // registers -> LDS, gates evaluated on the way
    const int nt = min(CH, n - tc);
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      if (tt < nt) {
        float* row = stage + tt * rowlen;
        if constexpr (VEC) {
#pragma unroll
          for (int u = 0; u < SEG4; ++u) {
            const int e = 4 * (lane + 64 * u);
            if (e < 2 * dpad) *reinterpret_cast<f32x4*>(row + e) = p4[tt][u];
          }
        } else {
#pragma unroll
          for (int u = 0; u < SEG; ++u) {
            const int e = lane + 64 * u;
            if (e < dpad) { row[e] = pk[tt][u]; row[dpad + e] = pq[tt][u]; }
          }
        }
        if (lane < cols_per_block) row[2 * dpad + lane] = pv[tt];
      }
    }
    // the chunk's gates in one pass, a token per lane: decay = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b)
    if (lane < 2 * CH) {
      const int tt = lane % CH;
      if (tt < nt) {
        const float a = pgate + dtb;
        const float decay = expf(nA * (a > 20.f ? a : log1pf(expf(a))));
        const float beta = 1.f / (1.f + expf(-pgate));
        stage[tt * rowlen + 2 * dpad + cols_per_block + (lane < CH ? 0 : 1)] = lane < CH ? decay : beta;
      }
    }
  };
  auto apply = [&](const float* stage, int tc) {  // the recurrence over one staged chunk
    const int nt = min(CH, n - tc);
    for (int tt = 0; tt < nt; ++tt) {
      const float* row = stage + tt * rowlen;
      float k[DPT], q[DPT];
#pragma unroll
      for (int i = 0; i < DPT; i += 4) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(row + i0 + i), qv = *reinterpret_cast<const f32x4*>(row + dpad + i0 + i);
        k[i] = kv.x; k[i + 1] = kv.y; k[i + 2] = kv.z; k[i + 3] = kv.w;
        q[i] = qv.x; q[i + 1] = qv.y; q[i + 2] = qv.z; q[i + 3] = qv.w;
      }
      const float v = row[2 * dpad + (jl < cols_per_block ? jl : 0)];
      const float gd = row[2 * dpad + cols_per_block], beta = row[2 * dpad + cols_per_block + 1];
      // (four partial sums each: a single accumulator would make the 2 x DPT multiply-adds one dependent chain)
      float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < DPT; ++i) { s[i] *= gd; d4[i & 3] += s[i] * k[i]; }
      const float dot = group_sum<R>((d4[0] + d4[1]) + (d4[2] + d4[3]));
      const float u = beta * (v - dot);
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < DPT; ++i) { s[i] += k[i] * u; o4[i & 3] += s[i] * q[i]; }
      const float oa = group_sum<R>((o4[0] + o4[1]) + (o4[2] + o4[3]));
      if (r == 0 && jl < cols_per_block) ostage[tt * cols_per_block + jl] = oa;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int idx = lane; idx < nt * cols_per_block; idx += 64) {
      const int tt = idx / cols_per_block, c = idx - tt * cols_per_block;
      if (col0 + c < dv) o[(long)(t0 + tc + tt) * ((long)Hv * dv) + (long)h * dv + col0 + c] = ostage[idx];
    }
  };
  if constexpr (DECODE) {
    for (int tc = 0; tc < n; tc += CH) {
      prefetch(tc);
      __builtin_amdgcn_wave_barrier();
      publish(smem, tc);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      apply(smem, tc);
    }
  } else {
    // Step i: the loader publishes chunk i into buffer i & 1 (and sends for chunk i + 1) while the compute wave
    // applies chunk i - 1 from the other buffer; the barrier that ends the step hands buffers over both ways.
    const int nchunks = (n + CH - 1) / CH;
    if (loads) prefetch(0);
    for (int i = 0; i <= nchunks; ++i) {
      if (loads && i < nchunks) {
        publish(smem + (i & 1) * CH * rowlen, i * CH);
        if (i + 1 < nchunks) prefetch((i + 1) * CH);
      }
      if (computes && i > 0) apply(smem + ((i - 1) & 1) * CH * rowlen, (i - 1) * CH);
      __syncthreads();
    }
  }
  if (computes && active) {
#pragma unroll
    for (int i = 0; i < DPT; ++i)
      if (i0 + i < d) Sp[(long)(i0 + i) * dv] = s[i];
  }
}

}  // namespace dlia

extern "C" void dlia_short_conv(float* y, const float* z, float* carry, const float* taps, const int* q_start, const int* ctx,
                                const int* slots, int B, int max_q, int C, int K, long ldz, int state_rows, const float* bias,
                                int silu, hipStream_t stream) {
  if (B <= 0 || max_q <= 0) return;
  // a workgroup takes 8 tokens of a sequence and every fourth 256-channel slice (thousands of workgroups for a prompt portion)
  const int tokb = 8, cblocks = (C + 1023) / 1024 < 1 ? 1 : (C + 1023) / 1024;
  hipLaunchKernelGGL(dlia::short_conv_kernel, dim3(B, (max_q + tokb - 1) / tokb, cblocks), dim3(256), 0, stream, y, z, carry, taps,
                     q_start, ctx, slots, C, K, ldz, tokb, state_rows, bias, silu);
  if (K > 1)
    hipLaunchKernelGGL(dlia::conv_carry_kernel, dim3(B, (C + 255) / 256), dim3(256), 0, stream, carry, z, q_start, ctx, slots, C,
                       K, ldz, state_rows);
}

extern "C" void dlia_unit_heads(float* x, int T, int heads, int d, long ld, int scaled_heads, float mult, float eps,
                                hipStream_t stream) {
  const int items = T * heads;
  if (items <= 0) return;
  hipLaunchKernelGGL(dlia::unit_heads_kernel, dim3((items + 3) / 4), dim3(256), 0, stream, x, items, heads, d, ld, scaled_heads,
                     mult, eps);
}

// Launch geometry of the delta rule: R lanes share a value column (a power of two up to 64), each holding DPT of
// the d state rows (zero-padded to dpad = R * DPT); a single-wave workgroup takes 64 / R columns.
extern "C" int dlia_delta_rule(float* o, const float* y, const float* z, float* state, const float* A_log,
                               const float* dt_bias, const int* q_start, const int* ctx, const int* slots, int B, int G, int Hv,
                               int d, int dv, int C, long ldz, int col_beta, int col_a, int state_rows, int max_q, hipStream_t stream) {
  if (B <= 0) return 0;
  int dpt = d <= 16 ? 16 : (d <= 128 ? 32 : 64);
  int R = 1;
  while (R * dpt < d) R <<= 1;
  if (R > 8) return -1;                               // d up to 512
  // A prompt portion of few sequences leaves most of the chip idle at 64 / R columns per wave, and the time of a
  // token is the time of one wave's multiply-adds: spread a column over more lanes (fewer state rows each, more
  // waves) until there are some 512 waves. Decode steps keep the widest rows: their cost is the state's traffic.
  if (max_q > 1) {
    auto waves = [&](int r) { const int c = 64 / r < dv ? 64 / r : dv; return (long)B * Hv * ((dv + c - 1) / c); };
    while (waves(R) < 512 && dpt > 8 && R < 16) { dpt >>= 1; R <<= 1; }
  }
  int cols = 64 / R;
  if (cols > dv) cols = dv;
  const int dpad = R * dpt, seg = (dpad + 63) / 64;
  const int ch = max_q <= 1 ? 1 : (seg <= 2 ? 16 : (seg <= 4 ? 8 : 4));
  const int rowlen = (2 * dpad + cols + 2 + 3) / 4 * 4;
  const dim3 grid(B, Hv, (dv + cols - 1) / cols);
  const size_t smem = (size_t)ch * ((max_q <= 1 ? 1 : 2) * rowlen + cols) * sizeof(float);
  const bool vec = d % 4 == 0 && C % 4 == 0 && (uintptr_t)y % 16 == 0;
#define DLIA_DELTA(D, RR, DEC, V)                                                                                                   \
  hipLaunchKernelGGL((dlia::delta_rule_kernel<D, RR, DEC, V>), grid, dim3(DEC ? 64 : 128), smem, stream, o, y, z, state, A_log, dt_bias, \
                     q_start, ctx, slots, G, Hv, d, dv, C, ldz, col_beta, col_a, cols, state_rows, rowlen)
#define DLIA_DELTA_CASE(D, RR)                                                                        \
  if (dpt == D && R == RR) {                                                                          \
    if (max_q <= 1) { if (vec) DLIA_DELTA(D, RR, true, true); else DLIA_DELTA(D, RR, true, false); }  \
    else            { if (vec) DLIA_DELTA(D, RR, false, true); else DLIA_DELTA(D, RR, false, false); } \
    return 0;                                                                                         \
  }
  // every (rows per lane, lanes per column) the geometry above can reach
  DLIA_DELTA_CASE(16, 1) DLIA_DELTA_CASE(8, 2)
  DLIA_DELTA_CASE(32, 1) DLIA_DELTA_CASE(16, 2) DLIA_DELTA_CASE(8, 4)
  DLIA_DELTA_CASE(32, 2) DLIA_DELTA_CASE(16, 4) DLIA_DELTA_CASE(8, 8)
  DLIA_DELTA_CASE(32, 4) DLIA_DELTA_CASE(16, 8) DLIA_DELTA_CASE(8, 16)
  DLIA_DELTA_CASE(64, 4) DLIA_DELTA_CASE(32, 8) DLIA_DELTA_CASE(16, 16)
  DLIA_DELTA_CASE(64, 8) DLIA_DELTA_CASE(32, 16)
#undef DLIA_DELTA_CASE
#undef DLIA_DELTA
  return -1;
}
