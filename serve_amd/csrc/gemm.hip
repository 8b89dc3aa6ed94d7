// C[M, N] = A[M, K] * W[N, K]^T with fp32 multiply and fp32 accumulate.
//
// This is the true 32-bit matrix product of the float32 path (no reduced-precision matrix mode
// is involved: v_fma_f32 and v_mfma_f32_32x32x2_f32, both full float32), and the product for any mix of storage types that the faster
// MFMA kernels do not take.  The reference leaves these products to nn.Linear
// (serve/model.py:80-82,95,97,159).
//
// Three kernels: gemm_nt_rows_kernel for up to 16 rows of float32 activations, gemm_nt_mfma32_kernel
// (the matrix cores' float32 instruction) for more rows whose length is a multiple of four, and
// gemm_nt_kernel for everything else: a 256-thread block owns a 64x64 tile of C; K advances in
// slices of 16 through LDS; each thread accumulates a 4x4 sub-tile with v_fma_f32.  Every edge (M,
// N, K not multiples of the tile) is guarded, so any size is accepted.
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

// The same product for few rows of activations (decode steps of the float32 path), where the work is
// reading W once: a wave owns two rows of W, its lanes split K (a float4 each, two per chunk of 512),
// the MR rows of activations of a pass lie in LDS a chunk at a time, and the lanes' partial sums are
// added across the wave at the end, always in the same order.  The stream of W never stops: the
// weights and activations of chunk c + 1 are on their way into registers while chunk c is multiplied
// (two register sets, two LDS buffers, one barrier a chunk).  Loads of W carry no conditions: a row
// beyond N is read from the last row and not stored, and beyond K the address wraps to the chunk's
// begin while the activation operand is zero.  Needs K % 4 == 0 and 16-byte aligned A and W.
template <int MR>
__global__ __launch_bounds__(256) void gemm_nt_rows_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                           float* __restrict__ C, int M, int N, int K) {
  constexpr int RW = 2;                               // rows of W per wave (four were no faster, at twice the registers)
  constexpr int KC = 512;
  constexpr int NJ = KC / 256;                        // float4 per lane, row of W and chunk
  constexpr int NA = (MR * (KC / 4) + 255) / 256;     // float4 of activations per thread and chunk
  __shared__ float4 As[2][MR][KC / 4];
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int n_base = (blockIdx.x * 4 + wave) * RW;
  const int m0 = blockIdx.y * MR;
  const float* wrow[RW];
#pragma unroll
  for (int rw = 0; rw < RW; ++rw) wrow[rw] = W + (size_t)min(n_base + rw, N - 1) * K;
  float acc[RW][MR];
#pragma unroll
  for (int rw = 0; rw < RW; ++rw)
#pragma unroll
    for (int r = 0; r < MR; ++r) acc[rw][r] = 0.f;
  const int nchunks = (K + KC - 1) / KC;

  auto fetch = [&](int c, float4 (&gw)[NJ][RW], float4 (&ga)[NA]) __attribute__((always_inline)) {
    const int k0 = min(c, nchunks - 1) * KC;          // past the last chunk: read it again, nobody uses it
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int k = k0 + (j * 64 + lane) * 4;
      const int kc = k < K ? k : k0;                  // beyond K: any valid address, the activations there are 0
#pragma unroll
      for (int rw = 0; rw < RW; ++rw) gw[j][rw] = *reinterpret_cast<const float4*>(wrow[rw] + kc);
    }
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int idx = tid + 256 * i;
      const int r = min(idx / (KC / 4), MR - 1);
      const int k = k0 + (idx % (KC / 4)) * 4;
      const int m = m0 + r;
      ga[i] = *reinterpret_cast<const float4*>(A + (size_t)min(m, M - 1) * K + (k < K ? k : k0));
    }
  };
  auto step = [&](int c, float4 (&cw)[NJ][RW], float4 (&ca)[NA], float4 (&nw)[NJ][RW], float4 (&na)[NA])
      __attribute__((always_inline)) {
    const int b = c & 1;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      // (rows beyond M and columns beyond K are zeroed here and not where the loads start: the zeroing waits for them)
      const int idx = tid + 256 * i;
      const int r = idx / (KC / 4), col = idx % (KC / 4);
      const bool inside = m0 + r < M && c * KC + col * 4 < K;
      float4 v = ca[i];
      if (!inside) v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (MR * (KC / 4) % 256 == 0 || idx < MR * (KC / 4)) As[b][r][col] = v;
    }
    __syncthreads();                                  // (the buffer was last read two chunks ago)
    fetch(c + 1, nw, na);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        const float4 a = As[b][r][j * 64 + lane];
#pragma unroll
        for (int rw = 0; rw < RW; ++rw) {
          float t = acc[rw][r];
          t = fmaf(cw[j][rw].x, a.x, t);
          t = fmaf(cw[j][rw].y, a.y, t);
          t = fmaf(cw[j][rw].z, a.z, t);
          t = fmaf(cw[j][rw].w, a.w, t);
          acc[rw][r] = t;
        }
      }
    }
  };
  float4 w0[NJ][RW], w1[NJ][RW], a0[NA], a1[NA];
  fetch(0, w0, a0);
  int c = 0;
  for (; c + 2 <= nchunks; c += 2) {
    step(c, w0, a0, w1, a1);
    step(c + 1, w1, a1, w0, a0);
  }
  if (c < nchunks) step(c, w0, a0, w1, a1);
#pragma unroll
  for (int rw = 0; rw < RW; ++rw)
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      const float v = wave_sum(acc[rw][r]);
      const int n = n_base + rw;
      const int m = m0 + r;
      if (lane == 0 && n < N && m < M) C[(size_t)m * N + n] = v;
    }
}

template <int MR>
static int launch_rows(const void* A, const void* W, void* C, int M, int N, int K, hipStream_t stream) {
  // a workgroup of four waves takes eight rows of W
  dim3 grid((N + 7) / 8, (M + MR - 1) / MR), block(256);
  hipLaunchKernelGGL((gemm_nt_rows_kernel<MR>), grid, block, 0, stream, (const float*)A, (const float*)W, (float*)C,
                     M, N, K);
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Many rows (prompt portions of the float32 path, and any mix of storage types): the matrix cores'
// float32 instruction, v_mfma_f32_32x32x2_f32, which multiplies and adds in full 32-bit precision
// (it is not the reduced "xf32" mode).  A workgroup of four waves owns a 128 x 128 tile of C, a
// wave 64 x 64 of it as 2 x 2 instruction tiles; K advances in slices of 16 through two LDS
// buffers (rows padded to 17 floats, so that the 32 lanes that read a column of a slice fall into
// 32 banks); a slice is fetched into registers while the slice before it is multiplied.
// Operands: lane l gives A[row l % 32][k l / 32] and W[row l % 32][k l / 32]; result register i of
// lane l is C[8 (i / 4) + 4 (l / 32) + i % 4][l % 32].  Needs K % 4 == 0 and 16-byte (bf16: 8-byte)
// aligned rows; rows beyond M and N are read as zeros.
// ---------------------------------------------------------------------------------------------
typedef float floatx16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float4 load4f(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4f(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_bits_to_float(u.x & 0xffffu), bf16_bits_to_float(u.x >> 16),
                     bf16_bits_to_float(u.y & 0xffffu), bf16_bits_to_float(u.y >> 16));
}

#define MF_BM 128
#define MF_BN 128
#define MF_BK 16
#define MF_FLUSH 32                // slices of K (512 terms) summed in one accumulator before they join the total

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_mfma32_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                             TC* __restrict__ C, int M, int N, int K) {
  __shared__ float As[2][MF_BM][MF_BK + 1];
  __shared__ float Ws[2][MF_BN][MF_BK + 1];
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * MF_BM;
  const int n0 = blockIdx.x * MF_BN;
  // what this thread fetches of a slice: rows lr and lr + 64 of both tiles, four floats at k4
  const int lr = tid >> 2;
  const int k4 = (tid & 3) * 4;
  const TA* arow[2];
  const TW* wrow[2];
  bool aok[2], wok[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int m = m0 + lr + 64 * j, n = n0 + lr + 64 * j;
    aok[j] = m < M;
    wok[j] = n < N;
    arow[j] = A + (size_t)(aok[j] ? m : 0) * K;
    wrow[j] = W + (size_t)(wok[j] ? n : 0) * K;
  }
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 ra[2], rw[2];
  auto fetch = [&](int k0) __attribute__((always_inline)) {
    const int k = k0 + k4;
    const bool kok = k < K;                       // K % 4 == 0: a group of four is inside or outside
    const int kc = kok ? k : 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      ra[j] = load4f(arow[j] + kc);
      rw[j] = load4f(wrow[j] + kc);
      if (!(kok && aok[j])) ra[j] = zero4;
      if (!(kok && wok[j])) rw[j] = zero4;
    }
  };
  auto stash = [&](int b) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float* a = &As[b][lr + 64 * j][k4];
      float* w = &Ws[b][lr + 64 * j][k4];
      a[0] = ra[j].x; a[1] = ra[j].y; a[2] = ra[j].z; a[3] = ra[j].w;
      w[0] = rw[j].x; w[1] = rw[j].y; w[2] = rw[j].z; w[3] = rw[j].w;
    }
  };
  // two levels of sums: `acc` takes MF_FLUSH slices of K and is then added to `total`, so that no sum
  // runs over more than a few hundred terms in one accumulator (the rounding of a float32 sum grows
  // with its length)
  floatx16_t acc[2][2], total[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = total[i][j][e] = 0.f;

  const int nslices = (K + MF_BK - 1) / MF_BK;
  fetch(0);
  stash(0);
  __syncthreads();
  const int r32 = lane & 31, kh = lane >> 5;
  for (int s = 0; s < nslices; ++s) {
    const int b = s & 1;
    if (s + 1 < nslices) fetch((s + 1) * MF_BK);
#pragma unroll
    for (int kk = 0; kk < MF_BK; kk += 2) {
      float a[2], w[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = As[b][wm * 64 + i * 32 + r32][kk + kh];
        w[i] = Ws[b][wn * 64 + i * 32 + r32][kk + kh];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], w[j], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < nslices) stash(b ^ 1);
    if ((s & (MF_FLUSH - 1)) == MF_FLUSH - 1 || s + 1 == nslices) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          total[i][j] += acc[i][j];
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + r32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * kh + (e & 3);
        if (m < M && n < N) C[(size_t)m * N + n] = from_float<TC>(total[i][j][e]);
      }
    }
}

// Which float32 product a shape takes.  gemm_nt_rows_kernel (passes of eight rows, each reading W
// again) does about 22 TFLOP/s whatever the shape; the matrix-core kernel takes about 0.078 us per
// element of K for every round of 128 x 128 tiles over the compute units, however few tiles there
// are (both measured on an MI355X).  Up to 16 rows always take the first; up to ROWS_KERNEL_MAX_M
// rows take the one with the smaller estimate (few tiles: a narrow W, decode batches of 17 to 128).
#define ROWS_KERNEL_MAX_M 128
#ifndef ROWS_KERNEL_RATE
#define ROWS_KERNEL_RATE 22e6
#endif
static bool rows_kernel_is_faster(int M, int N, int K) {
  if (M <= 16) return true;
  if (M > ROWS_KERNEL_MAX_M) return false;
  const double rows_us = 2.0 * M * N * K / ROWS_KERNEL_RATE;
  const long long tiles = (long long)((N + 127) / 128) * ((M + 127) / 128);
  const int cus = compute_units();
  const double mfma_us = 0.078 * K * (double)((tiles + cus - 1) / cus);
  return rows_us < mfma_us;
}

extern "C" int sa_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                          int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return SA_ERR_ARG;
  if (a_dtype == SA_F32 && w_dtype == SA_F32 && c_dtype == SA_F32 && (K & 3) == 0 && rows_kernel_is_faster(M, N, K) &&
      (((uintptr_t)A | (uintptr_t)W) & 15) == 0) {
    if (M == 1) return launch_rows<1>(A, W, C, M, N, K, stream);
    if (M == 2) return launch_rows<2>(A, W, C, M, N, K, stream);
    if (M <= 4) return launch_rows<4>(A, W, C, M, N, K, stream);
    return launch_rows<8>(A, W, C, M, N, K, stream);
  }
  // the matrix cores' float32 instruction where the rows can be fetched four elements at a time
  const bool mfma = (K & 3) == 0 && ((uintptr_t)A & (a_dtype == SA_F32 ? 15 : 7)) == 0 &&
                    ((uintptr_t)W & (w_dtype == SA_F32 ? 15 : 7)) == 0;
  dim3 grid((N + GT_N - 1) / GT_N, (M + GT_M - 1) / GT_M), block(256);
  if (mfma) grid = dim3((N + MF_BN - 1) / MF_BN, (M + MF_BM - 1) / MF_BM);
  if (grid.y > 65535) return SA_ERR_ARG;
#define GO(TA, TW, TC)                                                                                  \
  do {                                                                                                  \
    if (mfma)                                                                                           \
      hipLaunchKernelGGL((gemm_nt_mfma32_kernel<TA, TW, TC>), grid, block, 0, stream, (const TA*)A,     \
                         (const TW*)W, (TC*)C, M, N, K);                                                \
    else                                                                                                \
      hipLaunchKernelGGL((gemm_nt_kernel<TA, TW, TC>), grid, block, 0, stream, (const TA*)A,            \
                         (const TW*)W, (TC*)C, M, N, K);                                                \
  } while (0)
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
