// GEMM for any shape and for row-major (unpacked) weights: C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias), operands in
// bf16 (MFMA 16x16x32, fp32 accumulation) or in fp32 (MFMA 16x16x4 on fp32 operands: products and sums in true
// 32-bit), output in fp32 or in the operand type.
//
// The packed-weight kernels of this library want K in multiples of 128 and N in multiples of 16; models whose
// widths are not (a 200-wide residual stream, the few-row gate projections of a recurrent mixer) and the fp32 mode run
// here. Both operands are K-contiguous, and an MFMA fragment is 16 bytes of one row per lane, so fragments are
// loaded straight from memory: lane l of a 16-row tile reads row l % 16 at k-chunk l / 16. A workgroup of four
// waves covers a 64 x 64 tile of C (each wave 32 x 32: two row tiles by two column tiles, four MFMAs per
// k-step); the operand panels it shares are served by L1 / L2. Edges are handled by zero fragments and guarded
// stores, so M, N and K are arbitrary (rows that are not 16-byte aligned take an element-wise load).
//
// epi 0: + bias (optional). epi 1: gated pair — W's 16-row tiles alternate gate, up (`interleave_gate_up`), the
// wave holds both for the same 16 output columns and writes gelu_tanh(gate) * up, N/2 columns wide.
#include "common.h"
#include "frag.h"
#include "launch.h"

namespace dlia {

// accurate tanh-form GELU for the fp32 path (expf, IEEE division); the bf16 path's fast form is in common.h
__device__ __forceinline__ float gelu_tanh_exact(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.f + tanhf(u));
}

template <typename T, typename OT, int EPI>
__global__ __launch_bounds__(256) void gemm_any_kernel(OT* __restrict__ C, const T* __restrict__ A, const T* __restrict__ W,
                                                       const float* __restrict__ bias, int M, int N, int K, long lda,
                                                       long ldw, long ldc, int vec_ok, long a_step, long w_step, long c_step) {
  constexpr int VEC = 16 / sizeof(T), KS = 4 * VEC;
  // (blockIdx.z: one of several independent products of equal shape, e.g. the blocks of a block-diagonal matrix)
  A += blockIdx.z * a_step; W += blockIdx.z * w_step; C += blockIdx.z * c_step;
  if (bias) bias += (long)blockIdx.z * N;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int m_base = blockIdx.y * 64 + (wave >> 1) * 32, n_base = blockIdx.x * 64 + (wave & 1) * 32;
  if (m_base >= M || n_base >= N) return;
  const int r16 = lane & 15, kq = lane >> 4;
  f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const T* arow[2]; const T* wrow[2]; bool av[2], wv[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = m_base + i * 16 + r16, c = n_base + i * 16 + r16;
    av[i] = r < M; wv[i] = c < N;
    arow[i] = A + (long)(av[i] ? r : 0) * lda;
    wrow[i] = W + (long)(wv[i] ? c : 0) * ldw;
  }
  for (int k0 = 0; k0 < K; k0 += KS) {
    const int k = k0 + kq * VEC;
    u32x4 a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) { a[i] = load_frag<T>(arow[i], k, K, av[i], vec_ok); b[i] = load_frag<T>(wrow[i], k, K, wv[i], vec_ok); }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = mma_frag(T{}, a[i], b[j], acc[i][j]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = m_base + i * 16 + kq * 4 + r;
      if (row >= M) continue;
      if constexpr (EPI == 0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int col = n_base + j * 16 + r16;
          if (col < N) C[(long)row * ldc + col] = (OT)(acc[i][j][r] + (bias ? bias[col] : 0.f));
        }
      } else {
        const int cg = n_base + r16, cu = n_base + 16 + r16;
        if (cu < N) {
          const float g = acc[i][0][r] + (bias ? bias[cg] : 0.f), u = acc[i][1][r] + (bias ? bias[cu] : 0.f);
          const float act = sizeof(T) == 4 ? gelu_tanh_exact(g) : gelu_tanh(g);
          C[(long)row * ldc + (n_base >> 1) + r16] = (OT)(act * u);
        }
      }
    }
}

// The unfused form of the gated epilogue, for activations that a packed-weight GEMM left as [M, 2F] (gate columns,
// then up columns, bias already added): act[m, j] = gelu_tanh(gu[m, j]) * gu[m, F + j]. Eight columns per lane.
__global__ __launch_bounds__(256) void gated_gelu_kernel(bf16* __restrict__ act, const bf16* __restrict__ gu, int M, int F,
                                                         long ldg, long lda) {
  const int per_row = F >> 3;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)M * per_row) return;
  const int m = (int)(i / per_row), c = (int)(i % per_row) * 8;
  float g[8], u[8];
  unpack8(ld16(gu + (long)m * ldg + c), g);
  unpack8(ld16(gu + (long)m * ldg + F + c), u);
#pragma unroll
  for (int j = 0; j < 8; ++j) g[j] = gelu_tanh(g[j]) * u[j];
  st16(act + (long)m * lda + c, pack8(g));
}

template <typename T, typename OT>
static void launch_any(void* C, const void* A, const void* W, const float* bias, int M, int N, int K, long lda, long ldw,
                       long ldc, int epi, hipStream_t stream, int blocks = 1, long a_step = 0, long w_step = 0, long c_step = 0) {
  constexpr int VEC = 16 / sizeof(T);
  const int vec_ok = K % VEC == 0 && lda % VEC == 0 && ldw % VEC == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0 &&
                     a_step % VEC == 0 && w_step % VEC == 0;
  const dim3 grid((N + 63) / 64, (M + 63) / 64, blocks);
  if (epi == 0)
    hipLaunchKernelGGL((gemm_any_kernel<T, OT, 0>), grid, dim3(256), 0, stream, (OT*)C, (const T*)A, (const T*)W, bias, M, N,
                       K, lda, ldw, ldc, vec_ok, a_step, w_step, c_step);
  else
    hipLaunchKernelGGL((gemm_any_kernel<T, OT, 1>), grid, dim3(256), 0, stream, (OT*)C, (const T*)A, (const T*)W, bias, M, N,
                       K, lda, ldw, ldc, vec_ok, a_step, w_step, c_step);
}

}  // namespace dlia

extern "C" void dlia_gated_gelu(void* act, const void* gu, int M, int F, long ldg, long lda, hipStream_t stream) {
  if (M <= 0 || F <= 0) return;
  const long n = (long)M * (F >> 3);
  hipLaunchKernelGGL(dlia::gated_gelu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, (dlia::bf16*)act,
                     (const dlia::bf16*)gu, M, F, ldg, lda);
}

extern "C" void dlia_gemm_any(void* C, int out_f32, const void* A, const void* W, int in_f32, const float* bias, int M, int N,
                              int K, long lda, long ldw, long ldc, int epi, hipStream_t stream) {
  if (M <= 0 || N <= 0) return;
  if (in_f32)
    dlia::launch_any<float, float>(C, A, W, bias, M, N, K, lda, ldw, ldc, epi, stream);
  else if (out_f32)
    dlia::launch_any<dlia::bf16, float>(C, A, W, bias, M, N, K, lda, ldw, ldc, epi, stream);
  else
    dlia::launch_any<dlia::bf16, dlia::bf16>(C, A, W, bias, M, N, K, lda, ldw, ldc, epi, stream);
}

extern "C" void dlia_gemm_blocks(void* C, int out_f32, const void* A, const void* W, int in_f32, const float* bias, int M, int N,
                                 int K, long lda, long ldw, long ldc, int blocks, long a_step, long w_step, long c_step,
                                 hipStream_t stream) {
  if (M <= 0 || N <= 0 || blocks <= 0) return;
  if (in_f32)
    dlia::launch_any<float, float>(C, A, W, bias, M, N, K, lda, ldw, ldc, 0, stream, blocks, a_step, w_step, c_step);
  else if (out_f32)
    dlia::launch_any<dlia::bf16, float>(C, A, W, bias, M, N, K, lda, ldw, ldc, 0, stream, blocks, a_step, w_step, c_step);
  else
    dlia::launch_any<dlia::bf16, dlia::bf16>(C, A, W, bias, M, N, K, lda, ldw, ldc, 0, stream, blocks, a_step, w_step, c_step);
}
