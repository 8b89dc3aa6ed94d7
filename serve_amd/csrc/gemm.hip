// C[M, N] = A[M, K] * W[N, K]^T with fp32 multiply and fp32 accumulate.
//
// This is the true 32-bit matrix product of the float32 path (no reduced-precision matrix mode
// is involved: v_fma_f32 and v_mfma_f32_32x32x2_f32, both full float32), and the product for any mix of storage types that the faster
// MFMA kernels do not take.  The reference leaves these products to nn.Linear
// (serve/model.py:80-82,95,97,159).
//
// Four kernels: gemm_nt_rows_kernel for up to 8 rows of float32 activations, gemm_nt_mid32_kernel (the
// matrix cores' float32 instruction, weights streamed once per 64 rows) for 9 to 128,
// gemm_nt_mfma32_kernel (the same instruction, 128 x 128 tiles) for more rows whose length is a
// multiple of four, and gemm_nt_kernel for everything else: a 256-thread block owns a 64x64 tile of C; K advances in
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
// 9 to 128 rows of float32 activations (decode steps of the float32 path at those batch sizes): the
// weights are streamed once per 64 rows, as in the kernel above, but multiplied on the matrix cores
// (v_mfma_f32_32x32x2_f32, full float32).  A workgroup of eight waves owns 32 rows of W; the waves
// are eight slices of each 256-column stage of K (32 columns a wave), their sums are added through
// LDS at the end, in order.  The MT 32-row tiles of activations of a stage lie in LDS (rows padded
// by four floats, which spreads the 16-byte reads of the 32 lanes of a column over the banks) and
// are shared by the eight waves; weights go from global memory straight into registers, two stages
// ahead of the products, activations one stage ahead.
// Operands: lane l = (row r = l % 32, half h = l / 32) holds W[n0 + r][k .. k + 3] and
// A[m0 + r][k .. k + 3] for k = (block of eight columns) + 4 h; component c of both is one
// instruction's k index h (the order of the columns inside a block of eight does not matter as long
// as both operands follow it).  Result register e of lane l is C[m0 + l % 32][n0 + 8 (e / 4) + 4 h +
// e % 4].  Needs K % 4 == 0 and 16-byte aligned A and W; loads carry no conditions (rows beyond M
// and N are read from the last row, columns beyond K from the stage's begin, with the activation
// operand zeroed on its way into LDS).
// ---------------------------------------------------------------------------------------------
typedef float floatx16_t __attribute__((ext_vector_type(16)));
#define MD_KH 8
#define MD_KS (32 * MD_KH)                     // columns per stage
#define MD_PITCH (MD_KS + 4)

template <int MT>
__global__ __launch_bounds__(64 * MD_KH) void gemm_nt_mid32_kernel(const float* __restrict__ A,
                                                                   const float* __restrict__ W,
                                                                   float* __restrict__ C, int M, int N, int K) {
  constexpr int THREADS = 64 * MD_KH;
  constexpr int ROWS = 32 * MT;
  constexpr int NA = ROWS * (MD_KS / 4) / THREADS;            // float4 of activations per thread and stage
  static_assert(ROWS * (MD_KS / 4) % THREADS == 0, "the activation tile is spread evenly over the threads");
  static_assert((MD_KH - 1) * MT * 16 * 64 <= ROWS * MD_PITCH, "the sums of the other K slices reuse the tile");
  __shared__ __attribute__((aligned(16))) float As[ROWS * MD_PITCH];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int kh = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int m0 = blockIdx.y * ROWS;
  const float* wrow = W + (size_t)min(n0 + r, N - 1) * K;
  // this workgroup's share of the stages of K (gridDim.z parts, each with its own [M, N] of sums)
  // (spread evenly: no part is empty while there are at least as many stages as parts)
  const int all_stages = (K + MD_KS - 1) / MD_KS;
  const int s_begin = (int)((long long)blockIdx.z * all_stages / gridDim.z);
  const int nstages = (int)((long long)(blockIdx.z + 1) * all_stages / gridDim.z) - s_begin;
  C += (size_t)blockIdx.z * M * N;

  floatx16_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[mt][e] = 0.f;

  auto fetch_w = [&](int s, float4 (&w)[4]) __attribute__((always_inline)) {
    // past the part's last stage: read it again, nobody uses it (a part without stages reads the matrix's last one)
    const int k0 = min(s_begin + max(0, min(s, nstages - 1)), all_stages - 1) * MD_KS;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + kh * 32 + j * 8 + h * 4;
      w[j] = *reinterpret_cast<const float4*>(wrow + (k < K ? k : k0));
    }
  };
  auto fetch_a = [&](int s, float4 (&a)[NA]) __attribute__((always_inline)) {
    const int k0 = min(s_begin + max(0, min(s, nstages - 1)), all_stages - 1) * MD_KS;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int idx = tid + THREADS * i;
      const int row = idx / (MD_KS / 4), col = (idx % (MD_KS / 4)) * 4;
      a[i] = *reinterpret_cast<const float4*>(A + (size_t)min(m0 + row, M - 1) * K + (k0 + col < K ? k0 + col : k0));
    }
  };
  auto step = [&](int s, float4 (&w)[4], float4 (&wpre)[4], float4 (&a)[NA]) __attribute__((always_inline)) {
    const int k0 = (s_begin + s) * MD_KS;
    __syncthreads();                                          // the stage before has been multiplied
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      // (zeroed here and not where the loads start: the zeroing waits for them)
      const int idx = tid + THREADS * i;
      const int row = idx / (MD_KS / 4), col = (idx % (MD_KS / 4)) * 4;
      float4 v = a[i];
      if (m0 + row >= M || k0 + col >= K) v = make_float4(0.f, 0.f, 0.f, 0.f);
      *reinterpret_cast<float4*>(&As[row * MD_PITCH + col]) = v;
    }
    __syncthreads();
    fetch_a(s + 1, a);
    fetch_w(s + 2, wpre);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float4 b[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        b[mt] = *reinterpret_cast<const float4*>(&As[(mt * 32 + r) * MD_PITCH + kh * 32 + j * 8 + h * 4]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[j].x, b[mt].x, acc[mt], 0, 0, 0);
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[j].y, b[mt].y, acc[mt], 0, 0, 0);
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[j].z, b[mt].z, acc[mt], 0, 0, 0);
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[j].w, b[mt].w, acc[mt], 0, 0, 0);
      }
    }
  };

  float4 w0[4], w1[4], w2[4], a0[NA];
  fetch_a(0, a0);
  fetch_w(0, w0);
  fetch_w(1, w1);
  // three stages a turn so that the register sets of W take turns without copies.  Sums in two
  // levels, as in the kernel for many rows below: an accumulator takes the 480 terms of five turns and
  // is then added to the wave's total, so that a long inner dimension does not round 1,800 terms
  // into one running sum.
  floatx16_t total[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int e = 0; e < 16; ++e) total[mt][e] = 0.f;
  int s = 0, turns = 0;
  for (; s + 3 <= nstages; s += 3) {
    step(s, w0, w2, a0);
    step(s + 1, w1, w0, a0);
    step(s + 2, w2, w1, a0);
    if (++turns == 5) {
      turns = 0;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        total[mt] += acc[mt];
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[mt][e] = 0.f;
      }
    }
  }
  if (s < nstages) {
    step(s, w0, w2, a0);
    if (s + 1 < nstages) step(s + 1, w1, w0, a0);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] += total[mt];

  // add the slices of K in a fixed order: the waves of slices 1.. hand their sums over through LDS
  __syncthreads();
  if (kh > 0) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int e = 0; e < 16; ++e) As[(((kh - 1) * MT + mt) * 16 + e) * 64 + lane] = acc[mt][e];
  }
  __syncthreads();
  if (kh > 0) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 32 + r;
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      float v[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = e4 * 4 + c;
        float sum = acc[mt][e];
#pragma unroll
        for (int o = 1; o < MD_KH; ++o) sum += As[(((o - 1) * MT + mt) * 16 + e) * 64 + lane];
        v[c] = sum;
      }
      const int n = n0 + e4 * 8 + h * 4;
      if (m >= M) continue;
      float* cp = C + (size_t)m * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<float4*>(cp) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (n + c < N) cp[c] = v[c];
      }
    }
  }
}

template <int MT>
static int launch_mid32(const void* A, const void* W, void* C, int M, int N, int K, int parts, hipStream_t stream) {
  dim3 grid((N + 31) / 32, (M + 32 * MT - 1) / (32 * MT), parts), block(64 * MD_KH);
  hipLaunchKernelGGL((gemm_nt_mid32_kernel<MT>), grid, block, 0, stream, (const float*)A, (const float*)W, (float*)C,
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

// Which float32 product a shape takes (float32 throughout, K % 4 == 0, 16-byte aligned operands): up
// to ROWS_KERNEL_MAX_M rows the weight-streaming kernel on the vector ALU; from
// there to MID32_MAX_M rows the matrix-core kernel that streams the weights once per 64 rows (at 64
// rows and the 1B shape a decode step of the float32 path went from 6.97 to 3.54 ms with it, at 16 rows
// from 2.89 to 2.58); more
// rows, and every other mix of types, the tiled kernels below.
#define ROWS_KERNEL_MAX_M 8
#define MID32_MAX_M 128

// one or two 32-row tiles of activations a pass (three and four, with the weights read once for up to
// 128 rows, were no faster at 65 to 96 rows and slower beyond: the matrix cores are the bound there)
static int pick_mid32(const void* A, const void* W, void* C, int M, int N, int K, int parts, hipStream_t stream) {
  if (M <= 32) return launch_mid32<1>(A, W, C, M, N, K, parts, stream);
  return launch_mid32<2>(A, W, C, M, N, K, parts, stream);
}

// The float32 product of ROWS_KERNEL_MAX_M + 1 to MID32_MAX_M rows with K cut into `parts` (1 to 8) over the
// grid: C [parts, M, N] takes the partial sums, which the consumer adds in order (narrow matrices have
// too few rows of W to fill the chip otherwise).  Needs K % 4 == 0 and 16-byte aligned A and W.
extern "C" int sa_gemm_f32_mid_parts(const void* A, const void* W, void* C, int M, int N, int K, int parts,
                                     hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 3) || parts < 1 || parts > 8 || M <= ROWS_KERNEL_MAX_M || M > MID32_MAX_M ||
      ((((uintptr_t)A | (uintptr_t)W) & 15) != 0))
    return SA_ERR_ARG;
  return pick_mid32(A, W, C, M, N, K, parts, stream);
}

extern "C" int sa_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                          int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return SA_ERR_ARG;
  const bool f32_rows = a_dtype == SA_F32 && w_dtype == SA_F32 && c_dtype == SA_F32 && (K & 3) == 0 &&
                        (((uintptr_t)A | (uintptr_t)W) & 15) == 0;
  if (f32_rows && M > ROWS_KERNEL_MAX_M && M <= MID32_MAX_M) return pick_mid32(A, W, C, M, N, K, 1, stream);
  if (f32_rows && M <= ROWS_KERNEL_MAX_M) {
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
