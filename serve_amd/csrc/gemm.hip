// C[M, N] = A[M, K] * W[N, K]^T with fp32 multiply and fp32 accumulate on the vector ALU.
//
// This is the true 32-bit matrix product of the float32 path (no reduced-precision matrix mode
// is involved: plain v_fma_f32), and the product for any mix of storage types that the faster
// MFMA kernels do not take.  The reference leaves these products to nn.Linear
// (serve/model.py:80-82,95,97,159).
//
// Tiling: a 256-thread block owns a 64x64 tile of C; K advances in slices of 16 through LDS;
// each thread accumulates a 4x4 sub-tile.  Every edge (M, N, K not multiples of the tile) is
// guarded, so any size is accepted.
#include "common.h"

#define GT_M 64
#define GT_N 64
#define GT_K 16

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                      TC* __restrict__ C, int M, int N, int K) {
  __shared__ float As[GT_K][GT_M + 4];
  __shared__ float Ws[GT_K][GT_N + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT_M;
  const int n0 = blockIdx.x * GT_N;
  // loading: thread -> (row = tid / 4, k = (tid % 4) * 4 .. + 3)
  const int lrow = tid >> 2;
  const int lk = (tid & 3) * 4;
  // computing: thread -> rows ty*4.., cols tx*4..
  const int ty = tid >> 4;
  const int tx = tid & 15;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GT_K) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lrow;
      const int wn = n0 + lrow;
      As[lk + e][lrow] = (am < M && k < K) ? to_float(A[(size_t)am * K + k]) : 0.f;
      Ws[lk + e][lrow] = (wn < N && k < K) ? to_float(W[(size_t)wn * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GT_K; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * N + n] = from_float<TC>(acc[i][j]);
    }
  }
}

extern "C" int sa_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                          int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return SA_ERR_ARG;
  dim3 grid((N + GT_N - 1) / GT_N, (M + GT_M - 1) / GT_M), block(256);
  if (grid.y > 65535) return SA_ERR_ARG;
#define GO(TA, TW, TC)                                                                              \
  hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, TC>), grid, block, 0, stream, (const TA*)A, (const TW*)W, \
                     (TC*)C, M, N, K)
  const int code = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (code) {
    case 0: GO(float, float, float); break;
    case 1: GO(float, float, bf16_t); break;
    case 2: GO(float, bf16_t, float); break;
    case 3: GO(float, bf16_t, bf16_t); break;
    case 4: GO(bf16_t, float, float); break;
    case 5: GO(bf16_t, float, bf16_t); break;
    case 6: GO(bf16_t, bf16_t, float); break;
    case 7: GO(bf16_t, bf16_t, bf16_t); break;
    default: return SA_ERR_UNSUPPORTED;
  }
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}
