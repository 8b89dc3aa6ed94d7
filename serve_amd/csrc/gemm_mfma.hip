// bf16 matrix products on the matrix cores for few rows of activations (decode steps and short
// prompt portions): C[M, N] = A[M, K] * W[N, K]^T, fp32 accumulation, weights streamed once.
//
// The work is bound by reading W.  A wave owns RT tiles of 16 rows of W and walks a slice of K in
// steps of 32; the KS waves of a workgroup split K between them and add their partial sums
// through LDS, so no atomics and a fixed summation order.  The MFMA computes the transposed
// tile: operand "A" of v_mfma_f32_16x16x32_bf16 is a 16x32 tile of W (lane l: row l%16, k-slots
// 8*(l/16)..+7), operand "B" is 32x16 of activations (lane l: activation row l%16, same k-slots),
// and the result gives lane l the four consecutive outputs C[m = l%16][n = 4*(l/16) .. +3],
// which are contiguous in C.
//
// The SWIGLU variant reads gate rows n and up rows I + n of the stacked matrix in the same wave
// and stores silu(gate) * up (serve/model.py:85), so the [M, 2I] intermediate never exists.
//
// Requirements, checked by the caller: K % 8 == 0 (16-byte rows), pointers 16-byte aligned.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
  uint4 u;
  bf16x8_t v;
};

// KU = k-chunks of 32 loaded before their products are issued (loads in flight per wave).
// gridDim.z > 1 cuts K across workgroups as well: workgroup z writes its partial sums to
// C + z * M * N (fp32), and the consumer adds the parts in order.
// STREAM: weights are loaded with the non-temporal hint (they are read once per step).
// EPI selects what is done with the sums: EPI_PLAIN stores them; EPI_SWIGLU pairs gate row n with up
// row I + n and stores silu(gate) * up; EPI_QKV_ROPE pairs row j of a head with row j + D/2 of the
// same head of the stacked q/k/v matrix, rotates the q and k pairs by position (the rotation of
// serve/model.py:234-244 on the checkpoint's row order) and stores q to its buffer and k and v
// straight into the cache pages of each token's slot (serve/kernels/cache_write.py:49-165).
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_QKV_ROPE = 2 };

struct QkvRopeArgs {
  const int* positions;     // [M]
  const float* inv_freq;    // [D / 2]
  const int* slots;         // [M] page * page_size + offset, < 0: do not store
  bf16_t* k_pages;          // [P, Hk, page_size, D]
  bf16_t* v_pages;          // [P, Hk, D, page_size]
  int Hq, Hk, D, page_size;
};

template <int RT, int MT, int KS, int KU, typename TC, int EPI, bool STREAM = false>
__global__ __launch_bounds__(64 * KS) void gemm_skinny_kernel(const bf16_t* __restrict__ A,
                                                             const bf16_t* __restrict__ W,
                                                             TC* __restrict__ C, int M, int N, int K,
                                                             int up_offset, QkvRopeArgs qa) {
  constexpr bool SWIGLU = EPI == EPI_SWIGLU;
  constexpr bool QKV = EPI == EPI_QKV_ROPE;
  static_assert(KS * RT * MT <= 64, "partial sums must fit into 64 KB of LDS");
  static_assert(EPI == EPI_PLAIN || RT == 2, "the pairing epilogues work on two row tiles");
  __shared__ float red[KS][RT * MT * 4][64];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  // first row of this workgroup's (first) tile; QKV: tile t16 of head `head`, second tile D/2 below
  const int tph = QKV ? (qa.D >> 5) : 1;
  const int head = QKV ? blockIdx.x / tph : 0;
  const int t16 = QKV ? blockIdx.x - head * tph : 0;
  const int n0 = QKV ? head * qa.D + t16 * 16 : blockIdx.x * (SWIGLU ? 16 : RT * 16);
  const int m0 = blockIdx.y * (MT * 16);

  const int nchunks = (K + 31) >> 5;
  const int per_wg = (nchunks + gridDim.z - 1) / gridDim.z;
  const int wg_begin = blockIdx.z * per_wg;
  const int wg_end = min(nchunks, wg_begin + per_wg);
  const int per = (per_wg + KS - 1) / KS;
  const int ch_begin = wg_begin + wave * per;
  const int ch_end = min(wg_end, ch_begin + per);
  C += (size_t)blockIdx.z * M * N;

  const bf16_t* wrow[RT];
  bool wok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n;
    if (SWIGLU) n = (rt == 0 ? 0 : up_offset) + n0 + c;
    else if (QKV) n = n0 + rt * (qa.D >> 1) + c;
    else n = n0 + rt * 16 + c;
    wok[rt] = SWIGLU ? (n0 + c < N) : (n < N);
    wrow[rt] = W + (size_t)(wok[rt] ? n : 0) * K;
  }
  const bf16_t* arow[MT];
  bool aok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + c;
    aok[mt] = m < M;
    arow[mt] = A + (size_t)(aok[mt] ? m : 0) * K;
  }

  floatx4_t acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int ch = ch_begin; ch < ch_end; ch += KU) {
    Frag wf[RT][KU], af[MT][KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int k = (ch + u) * 32 + g * 8;
      const bool kin = (ch + u) < ch_end && k < K;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        wf[rt][u].u = zero;
        if (kin && wok[rt]) {
          const uint4* src = reinterpret_cast<const uint4*>(wrow[rt] + k);
          if (STREAM) {
            typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
            const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
            wf[rt][u].u = make_uint4(t.x, t.y, t.z, t.w);
          } else {
            wf[rt][u].u = *src;
          }
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        af[mt][u].u = zero;
        if (kin && aok[mt]) af[mt][u].u = *reinterpret_cast<const uint4*>(arow[mt] + k);
      }
    }
#pragma unroll
    for (int u = 0; u < KU; ++u)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][u].v, af[mt][u].v, acc[rt][mt], 0, 0, 0);
  }

  // add the KS partial sums in a fixed order: every wave stores, wave 0 sums and writes
  if (KS > 1) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][(rt * MT + mt) * 4 + r][lane] = acc[rt][mt][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float s = acc[rt][mt][r];
          for (int w = 1; w < KS; ++w) s += red[w][(rt * MT + mt) * 4 + r][lane];
          acc[rt][mt][r] = s;
        }
  }

  const int ldc = N;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + c;
    if (m >= M) continue;
    if (SWIGLU) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + 4 * g + r;
        if (n < N) {
          const float gt = acc[0][mt][r];
          const float up = acc[1][mt][r];
          C[(size_t)m * ldc + n] = from_float<TC>((gt / (1.f + __expf(-gt))) * up);
        }
      }
    } else if (QKV) {
      const int D = qa.D, half = qa.D >> 1;
      const int dim0 = t16 * 16 + 4 * g;                 // this lane's four dims, and dim0 + D/2 ..
      float lo[4], hi[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        lo[r] = acc[0][mt][r];
        hi[r] = acc[1][mt][r];
      }
      if (head < qa.Hq + qa.Hk) {
        const float pos = (float)qa.positions[m];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float sn, cs;
          sincosf(pos * qa.inv_freq[dim0 + r], &sn, &cs);
          const float a = lo[r], b = hi[r];
          lo[r] = a * cs - b * sn;
          hi[r] = b * cs + a * sn;
        }
      }
      if (head < qa.Hq) {
        TC* qp = C + ((size_t)m * qa.Hq + head) * D + dim0;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          qp[r] = from_float<TC>(lo[r]);
          qp[half + r] = from_float<TC>(hi[r]);
        }
      } else {
        const int slot = qa.slots[m];
        if (slot >= 0) {
          const int page = slot / qa.page_size;
          const int off = slot - page * qa.page_size;
          if (head < qa.Hq + qa.Hk) {
            bf16_t* kp = qa.k_pages + (((size_t)page * qa.Hk + (head - qa.Hq)) * qa.page_size + off) * D + dim0;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              kp[r] = from_float<bf16_t>(lo[r]);
              kp[half + r] = from_float<bf16_t>(hi[r]);
            }
          } else {
            bf16_t* vp = qa.v_pages + (((size_t)page * qa.Hk + (head - qa.Hq - qa.Hk)) * D + dim0) * qa.page_size + off;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              vp[(size_t)r * qa.page_size] = from_float<bf16_t>(lo[r]);
              vp[(size_t)(half + r) * qa.page_size] = from_float<bf16_t>(hi[r]);
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = n0 + rt * 16 + 4 * g + r;
          if (n < N) C[(size_t)m * ldc + n] = from_float<TC>(acc[rt][mt][r]);
        }
    }
  }
}

template <int RT, int MT, int KS, int KU, typename TC, int EPI>
static int launch_skinny(const void* A, const void* W, void* C, int M, int N, int K, int up_offset,
                         int parts, const QkvRopeArgs& qa, hipStream_t stream) {
  unsigned gx;
  if (EPI == EPI_SWIGLU) gx = (N + 15) / 16;
  else if (EPI == EPI_QKV_ROPE) gx = (qa.Hq + 2 * qa.Hk) * (qa.D >> 5);
  else gx = (N + RT * 16 - 1) / (RT * 16);
  dim3 grid(gx, (M + MT * 16 - 1) / (MT * 16), parts);
  if (grid.y > 65535 || parts < 1 || parts > 64) return SA_ERR_ARG;
  hipLaunchKernelGGL((gemm_skinny_kernel<RT, MT, KS, KU, TC, EPI>), grid, dim3(64 * KS), 0, stream,
                     (const bf16_t*)A, (const bf16_t*)W, (TC*)C, M, N, K, up_offset, qa);
  SA_LAUNCH_CHECK();
  return 0;
}

template <typename TC, int EPI>
static int pick_skinny(const void* A, const void* W, void* C, int M, int N, int K, int up_offset,
                       int parts, const QkvRopeArgs& qa, hipStream_t stream) {
  // rows of activations per workgroup: 16, 32 or 64 (larger M loops over grid.y)
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  // many weight rows: 2 row tiles per wave and few waves; few rows: more waves splitting K
  const bool wide = EPI == EPI_SWIGLU || N >= 8192;
#define GO(RT, MT, KS, KU) \
  return launch_skinny<RT, MT, KS, KU, TC, EPI>(A, W, C, M, N, K, up_offset, parts, qa, stream)
  // (the choices below are the best of a sweep over RT, KS and KU at the Llama-3.2-1B sizes)
  if constexpr (EPI == EPI_QKV_ROPE) {
    if (mt == 1) GO(2, 1, 8, 8);
    if (mt == 2) GO(2, 2, 8, 4);
    GO(2, 4, 4, 4);
  }
  if (wide) {
    if (mt == 1) GO(2, 1, 2, 8);
    if (mt == 2) GO(2, 2, 4, 4);
    GO(2, 4, 4, 4);
  }
  if constexpr (EPI == EPI_PLAIN) {
    if (parts > 1) {
      // K is already cut across workgroups: 2 waves each
      if (mt == 1) GO(1, 1, 2, 8);
      if (mt == 2) GO(1, 2, 4, 4);
      GO(1, 4, 4, 4);
    }
    // 16 waves leave 128 registers a lane, enough only for one activation tile
    if (mt == 1) GO(1, 1, 16, 4);
    if (mt == 2) GO(1, 2, 8, 4);
    GO(1, 4, 8, 4);
  }
#undef GO
  return SA_ERR_ARG;
}

// C = A W^T; c_dtype SA_BF16 or SA_F32.  parts > 1 (fp32 only): C is [parts, M, N] and holds
// partial sums over `parts` slices of K, to be added by the consumer.
extern "C" int sa_gemm_bf16_skinny(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K,
                                   int parts, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || parts < 1) return SA_ERR_ARG;
  const QkvRopeArgs none = {};
  if (c_dtype == SA_BF16 && parts == 1) return pick_skinny<bf16_t, EPI_PLAIN>(A, W, C, M, N, K, 0, 1, none, stream);
  if (c_dtype == SA_F32) return pick_skinny<float, EPI_PLAIN>(A, W, C, M, N, K, 0, parts, none, stream);
  return SA_ERR_UNSUPPORTED;
}

// C[M, I] = silu(A Wg^T) * (A Wu^T) with W = [Wg; Wu] stacked as [2 I, K]
extern "C" int sa_gemm_bf16_skinny_swiglu(const void* A, const void* W, void* C, int M, int I, int K,
                                          hipStream_t stream) {
  if (M <= 0 || I <= 0) return 0;
  if (K <= 0 || (K & 7)) return SA_ERR_ARG;
  const QkvRopeArgs none = {};
  return pick_skinny<bf16_t, EPI_SWIGLU>(A, W, C, M, I, K, I, 1, none, stream);
}

// q, k, v = A [Wq; Wk; Wv]^T with W stacked as [(Hq + 2 Hk) D, K]; q and k rotated by position
// (pairs (j, j + D/2), all D dims); q goes to Q [M, Hq D], k and v into the cache pages.
// Needs D % 32 == 0.
extern "C" int sa_gemm_bf16_qkv_rope(const void* A, const void* W, void* Q, const int* positions,
                                     const float* inv_freq, const int* slots, void* k_pages, void* v_pages,
                                     int M, int K, int Hq, int Hk, int D, int page_size, hipStream_t stream) {
  if (M <= 0) return 0;
  if (K <= 0 || (K & 7) || Hq <= 0 || Hk <= 0 || D <= 0 || (D & 31) || page_size <= 0) return SA_ERR_ARG;
  const QkvRopeArgs qa = {positions, inv_freq, slots, (bf16_t*)k_pages, (bf16_t*)v_pages, Hq, Hk, D, page_size};
  return pick_skinny<bf16_t, EPI_QKV_ROPE>(A, W, Q, M, (Hq + 2 * Hk) * D, K, 0, 1, qa, stream);
}
