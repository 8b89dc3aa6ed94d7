// bf16 matrix products on the matrix cores for few rows of activations (decode steps and short
// prompt portions): C[M, N] = A[M, K] * W[N, K]^T, fp32 accumulation, weights streamed once.
// Three kernels: gemm_skinny_kernel for one or two rows, gemm_mid_kernel for up to 128 (per pass),
// and gemm_wide_kernel, which brings both operands into LDS without passing registers and takes
// the products of up to 256 rows where that is faster (see takes_wide).
//
// The work is bound by reading W.  In the first, a wave owns RT tiles of 16 rows of W and walks a
// slice of K in steps of 32; the KS waves of a workgroup split K between them and add their partial sums
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
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

union Frag {
  uint4 u;
  u32x4_t r;
  bf16x8_t v;
};

// KU = k-chunks of 32 loaded before their products are issued (loads in flight per wave).
// gridDim.z > 1 cuts K across workgroups as well: workgroup z writes its partial sums to
// C + z * M * N (fp32), and the consumer adds the parts in order.
// EPI selects what is done with the sums: EPI_PLAIN stores them; EPI_SWIGLU pairs gate row n with up
// row I + n and stores silu(gate) * up; EPI_QKV_ROPE works on one tile of 16 rows of the stacked
// q/k/v matrix that holds eight dims j.. of a head and their partners j + D/2..: the sums of a pair
// sit in lanes 32 apart and are exchanged with one row swap each, the q and k pairs are rotated by
// position (the rotation of serve/model.py:234-244 on the checkpoint's row order), q goes to its
// buffer and k and v straight into the cache pages of each token's slot
// (serve/kernels/cache_write.py:49-165).
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_QKV_ROPE = 2 };

struct QkvRopeArgs {
  const int* positions;     // [M]
  const float* inv_freq;    // [D / 2]
  const int* slots;         // [M] page * page_size + offset, < 0: do not store
  bf16_t* k_pages;          // [P, Hk, page_size, D]
  bf16_t* v_pages;          // [P, Hk, D, page_size]
  int Hq, Hk, D, page_size;
};

// What the rotating epilogue needs besides the sums: read when a kernel starts, so that the trip to
// memory for them runs beside the product and not after it.
template <int MT>
struct QkvLane {
  float pos[MT];
  int slot[MT];
  float freq[4];
};

template <int MT>
__device__ __forceinline__ QkvLane<MT> load_qkv_lane(const QkvRopeArgs& qa, int M, int m0, int head, int t8,
                                                     int g, int c) {
  QkvLane<MT> ql;
  const bool rotated = head < qa.Hq + qa.Hk;
  const bool stored = head >= qa.Hq && head < qa.Hq + 2 * qa.Hk;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = min(m0 + mt * 16 + c, M - 1);
    ql.pos[mt] = rotated ? (float)qa.positions[m] : 0.f;
    ql.slot[mt] = stored ? qa.slots[m] : -1;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) ql.freq[r] = rotated ? qa.inv_freq[t8 * 8 + 4 * (g & 1) + r] : 0.f;
  return ql;
}

__device__ __forceinline__ void store4(float* p, const float (&v)[4], bool vec) {
  if (vec) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r) p[r] = v[r];
  }
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&v)[4], bool vec) {
  if (vec) {
    uint2 u;
    u.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
    u.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = u;
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r) p[r] = from_float<bf16_t>(v[r]);
  }
}

// What is done with a wave's finished sums acc[rt][mt] (lane l: activation row m0 + 16 mt + l%16,
// outputs 4*(l/16) .. +3 of row tile rt); the row tiles start at n0 as the kernels below lay them
// out.  A lane's four outputs are consecutive in memory and go out as one store where the row
// length keeps them aligned.
template <int RT, int MT, typename TC, int EPI>
__device__ __forceinline__ void store_tiles(floatx4_t (&acc)[RT][MT], TC* __restrict__ C, int M, int N, int m0,
                                            int n0, int head, int t16, const QkvRopeArgs& qa,
                                            const QkvLane<MT>& ql, int g, int c) {
  constexpr bool SWIGLU = EPI == EPI_SWIGLU;
  constexpr bool QKV = EPI == EPI_QKV_ROPE;
  const int ldc = N;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + c;
    if (m >= M) continue;
    if (SWIGLU) {
      const int n = n0 + 4 * g;
      float o[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float gt = acc[0][mt][r];
        const float up = acc[1][mt][r];
        o[r] = (gt / (1.f + __expf(-gt))) * up;
      }
      if (n + 3 < N) {
        store4(C + (size_t)m * ldc + n, o, (N & 3) == 0);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) C[(size_t)m * ldc + n + r] = from_float<TC>(o[r]);
      }
    } else if (QKV) {
      // handled below, outside this loop's early exit: the exchange needs both partner lanes
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int n = n0 + rt * 16 + 4 * g;
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = acc[rt][mt][r];
        if (n + 3 < N) {
          store4(C + (size_t)m * ldc + n, o, (N & 3) == 0);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < N) C[(size_t)m * ldc + n + r] = from_float<TC>(o[r]);
        }
      }
    }
  }
  if (QKV) {
    // rows 0..7 of the tile are dims d0.. of the head, rows 8..15 their partners d0 + D/2..; lane
    // groups 0, 1 hold the former, 2, 3 the latter, for the same activation row: lanes 32 apart
    const int D = qa.D, half = qa.D >> 1;
    const bool upper = g >= 2;
    const int dim0 = t16 * 8 + 4 * (g & 1) + (upper ? half : 0);     // this lane's four consecutive dims
    const bool rotated = head < qa.Hq + qa.Hk;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = m0 + mt * 16 + c;
      float o[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float own = acc[0][mt][r];
        const uint32_t u = __float_as_uint(own);
        const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        const float partner = __uint_as_float(upper ? sw[0] : sw[1]);
        float sn, cs;
        sincos_reduced(ql.pos[mt] * ql.freq[r], &sn, &cs);
        // lower: a cos - b sin with a = own; upper: b cos + a sin with b = own
        o[r] = rotated ? (upper ? own * cs + partner * sn : own * cs - partner * sn) : own;
      }
      if (m >= M) continue;
      if (head < qa.Hq) {
        store4(C + ((size_t)m * qa.Hq + head) * D + dim0, o, true);      // D % 16 == 0: 8-byte aligned
      } else {
        const int slot = ql.slot[mt];
        if (slot < 0) continue;
        const int page = slot / qa.page_size;
        const int off = slot - page * qa.page_size;
        if (head < qa.Hq + qa.Hk) {
          store4(qa.k_pages + (((size_t)page * qa.Hk + (head - qa.Hq)) * qa.page_size + off) * D + dim0, o, true);
        } else {
          bf16_t* vp = qa.v_pages + (((size_t)page * qa.Hk + (head - qa.Hq - qa.Hk)) * D + dim0) * qa.page_size + off;
#pragma unroll
          for (int r = 0; r < 4; ++r) vp[(size_t)r * qa.page_size] = from_float<bf16_t>(o[r]);
        }
      }
    }
  }
}

template <int RT, int MT, int KS, int KU, typename TC, int EPI>
__global__ __launch_bounds__(64 * KS) void gemm_skinny_kernel(const bf16_t* __restrict__ A,
                                                             const bf16_t* __restrict__ W,
                                                             TC* __restrict__ C, int M, int N, int K,
                                                             int up_offset, QkvRopeArgs qa) {
  constexpr bool SWIGLU = EPI == EPI_SWIGLU;
  constexpr bool QKV = EPI == EPI_QKV_ROPE;
  static_assert(KS * RT * MT <= 64, "partial sums must fit into 64 KB of LDS");
  static_assert(EPI != EPI_SWIGLU || RT == 2, "gate and up rows are two row tiles");
  static_assert(EPI != EPI_QKV_ROPE || RT == 1, "a pair of dims sits in one row tile");
  __shared__ float red[KS][RT * MT * 4][64];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  // first row of this workgroup's (first) tile; QKV: tile t16 of head `head` = its dims 8 t16 .. + 7
  // and their partners D/2 further on
  const int tph = QKV ? (qa.D >> 4) : 1;
  const int head = QKV ? blockIdx.x / tph : 0;
  const int t16 = QKV ? blockIdx.x - head * tph : 0;
  const int n0 = QKV ? head * qa.D + t16 * 8 : blockIdx.x * (SWIGLU ? 16 : RT * 16);
  const int m0 = blockIdx.y * (MT * 16);

  QkvLane<MT> ql = {};
  if (QKV) ql = load_qkv_lane<MT>(qa, M, m0, head, t16, g, c);

  const int nchunks = (K + 31) >> 5;
  const int per_wg = (nchunks + gridDim.z - 1) / gridDim.z;
  const int wg_begin = blockIdx.z * per_wg;
  const int wg_end = min(nchunks, wg_begin + per_wg);
  const int per = (per_wg + KS - 1) / KS;
  const int ch_begin = wg_begin + wave * per;
  const int ch_end = min(wg_end, ch_begin + per);
  C += (size_t)blockIdx.z * M * N;

  // Loads carry no per-lane conditions (a branch around every load would serialize them): rows
  // beyond M or N are read from row 0 and give sums that are never stored; beyond the wave's slice
  // of K the address is clamped and the activation operand is zeroed, which zeroes the product
  // whatever finite weight stands there.
  const bf16_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n;
    if (SWIGLU) n = (rt == 0 ? 0 : up_offset) + n0 + c;
    else if (QKV) n = n0 + (c < 8 ? c : (qa.D >> 1) + c - 8);
    else n = n0 + rt * 16 + c;
    const bool ok = SWIGLU ? (n0 + c < N) : (n < N);
    wrow[rt] = W + (size_t)(ok ? n : 0) * K;
  }
  const bf16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + c;
    arow[mt] = A + (size_t)(m < M ? m : 0) * K;
  }

  floatx4_t acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  const u32x4_t zero = {0u, 0u, 0u, 0u};
  for (int ch = ch_begin; ch < ch_end; ch += KU) {
    Frag wf[RT][KU], af[MT][KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int k = min((ch + u) * 32 + g * 8, K - 8);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) wf[rt][u].r = *reinterpret_cast<const u32x4_t*>(wrow[rt] + k);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt][u].r = *reinterpret_cast<const u32x4_t*>(arow[mt] + k);
    }
    if (ch + KU > ch_end || (ch + KU) * 32 > K) {          // the last, partial round of the slice
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        const bool kin = (ch + u) < ch_end && (ch + u) * 32 + g * 8 < K;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) af[mt][u].r = kin ? af[mt][u].r : zero;
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

  store_tiles<RT, MT, TC, EPI>(acc, C, M, N, m0, n0, head, t16, qa, ql, g, c);
}

// The same products for up to 128 rows of activations a pass (decode at all but the smallest
// batches, short prompt portions).  With that many rows a workgroup reads about as many bytes of activations as of
// weights, so the activations are staged through LDS and shared.  A workgroup has NR x KH waves:
// NR groups of weight rows times KH slices of each 256-wide stage of K; the NR waves of a slice read
// the same activation fragments, and the KH slices add their sums through LDS at the end, in order.
// Weight fragments go from global memory straight into registers, two stages ahead of the products;
// activations are loaded two stages ahead into registers as well and written to the LDS buffer of
// their stage when it begins (two buffers in turn: one barrier per stage).  A row of a stage holds 32 segments of
// 16 bytes; segment s of row r is stored at slot s ^ (r % 16), which makes both the stores (16 lanes
// along a row) and the fragment reads (16 lanes along a column of segments) free of bank conflicts.
template <int RT, int MT, int NR, int KH, typename TC, int EPI>
__global__ __launch_bounds__(64 * NR * KH) void gemm_mid_kernel(const bf16_t* __restrict__ A,
                                                                const bf16_t* __restrict__ W,
                                                                TC* __restrict__ C, int M, int N, int K,
                                                                int up_offset, QkvRopeArgs qa) {
  constexpr bool SWIGLU = EPI == EPI_SWIGLU;
  constexpr bool QKV = EPI == EPI_QKV_ROPE;
  static_assert(EPI != EPI_SWIGLU || RT == 2, "gate and up rows are two row tiles");
  static_assert(EPI != EPI_QKV_ROPE || RT == 1, "a pair of dims sits in one row tile");
  static_assert(KH == 2 || KH == 4 || KH == 8, "a stage is 8 steps of 32");
  constexpr int THREADS = 64 * NR * KH;
  constexpr int ROWS = MT * 16;            // activation rows of a workgroup
  constexpr int NA = ROWS * 32 / THREADS;  // 16-byte activation segments per thread and stage
  constexpr int KU = 8 / KH;               // steps of 32 per wave and stage
  static_assert(ROWS * 32 % THREADS == 0, "the activation tile is spread evenly over the threads");
  __shared__ u32x4_t lds[2][ROWS][32];     // [buffer][row][segment slot]
  static_assert(sizeof(lds) >= (size_t)(KH - 1) * NR * RT * MT * 4 * 64 * sizeof(float),
                "the sums of the other K slices reuse it");

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int rg = wave % NR;                // row group
  const int kh = wave / NR;                // K slice
  const int tile = blockIdx.x * NR + rg;
  const int tph = QKV ? (qa.D >> 4) : 1;
  const int head = QKV ? tile / tph : 0;
  const int t16 = QKV ? tile - head * tph : 0;
  const int n0 = QKV ? head * qa.D + t16 * 8 : tile * (SWIGLU ? 16 : RT * 16);
  const int m0 = blockIdx.y * ROWS;

  QkvLane<MT> ql = {};
  if (QKV) ql = load_qkv_lane<MT>(qa, M, m0, head, t16, g, c);

  // this workgroup's slice of K, in chunks of 32
  const int nchunks = (K + 31) >> 5;
  const int per_wg = (nchunks + gridDim.z - 1) / gridDim.z;
  const int k_begin = blockIdx.z * per_wg * 32;
  const int k_end = min(K, k_begin + per_wg * 32);
  const int nstages = (k_end - k_begin + 255) >> 8;
  // Workgroups walk their stages in rotated order.  All of them read the same few activation rows,
  // whose stride is often a power of two: the same K offset of every row then lies in the same L2
  // channel, and workgroups in step would queue there.  (The order depends on the weight rows
  // only, so a row of activations gets the same sums whatever else is in the batch.)
  const int rot = nstages > 0 ? (int)(blockIdx.x % (unsigned)nstages) : 0;
  auto stage_k = [&](int s) __attribute__((always_inline)) {
    int t = s + rot;
    if (t >= nstages) t -= nstages;
    return k_begin + t * 256;
  };
  C += (size_t)blockIdx.z * M * N;

  const bf16_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n;
    if (SWIGLU) n = (rt == 0 ? 0 : up_offset) + n0 + c;
    else if (QKV) n = n0 + (c < 8 ? c : (qa.D >> 1) + c - 8);
    else n = n0 + rt * 16 + c;
    bool ok = SWIGLU ? (n0 + c < N) : (n < N);
    if (QKV) ok = head < qa.Hq + 2 * qa.Hk;
    wrow[rt] = W + (size_t)(ok ? n : 0) * K;
  }
  // the activation segments this thread moves: row idx / 32, 16-byte segment idx % 32 of the stage
  const bf16_t* asrc[NA];
  int aseg[NA];
  u32x4_t* adst[NA];
#pragma unroll
  for (int j = 0; j < NA; ++j) {
    const int idx = threadIdx.x + THREADS * j;
    const int row = idx >> 5;
    const int seg = idx & 31;
    asrc[j] = A + (size_t)(m0 + row < M ? m0 + row : 0) * K;
    aseg[j] = seg;
    adst[j] = &lds[0][row][seg ^ (row & 15)];
  }

  floatx4_t acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  // Loads carry no per-lane conditions (a branch around every load would serialize them): rows
  // beyond M or N are read from row 0 and give sums that are never stored, and beyond the end of
  // the slice of K the address is clamped and the activation operand is zeroed on its way into LDS,
  // which zeroes the product whatever finite weight stands there.
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  auto load_acts = [&](int s, u32x4_t (&areg)[NA]) __attribute__((always_inline)) {
    const int k0 = stage_k(s);
#pragma unroll
    for (int j = 0; j < NA; ++j)
      areg[j] = *reinterpret_cast<const u32x4_t*>(asrc[j] + min(k0 + aseg[j] * 8, K - 8));
  };
  auto load_weights = [&](int s, Frag (&wf)[RT][KU]) __attribute__((always_inline)) {
    const int k0 = stage_k(s) + kh * (KU * 32) + g * 8;
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int k = min(k0 + u * 32, K - 8);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) wf[rt][u].r = *reinterpret_cast<const u32x4_t*>(wrow[rt] + k);
    }
  };
  // one stage: publish its activations, start the loads of the stage after the next (both the
  // latency of L2 for the activations and of HBM for the weights take longer than a stage's
  // products), multiply
  auto stage = [&](int s, Frag (&cur)[RT][KU], Frag (&pre)[RT][KU], u32x4_t (&acur)[NA],
                   u32x4_t (&apre)[NA]) __attribute__((always_inline)) {
    constexpr int BUF = ROWS * 32;                      // 16-byte slots per buffer
    const int b = s & 1;
    const int k0 = stage_k(s);
    if (k0 + 256 > k_end) {          // the zeroing waits for the loads, so it is done here and not where they start
#pragma unroll
      for (int j = 0; j < NA; ++j) acur[j] = k0 + aseg[j] * 8 < k_end ? acur[j] : zero;
    }
#pragma unroll
    for (int j = 0; j < NA; ++j) adst[j][b * BUF] = acur[j];
    __syncthreads();
    // (unconditional, so that the number of loads in flight is known where their results are
    // awaited; past the last stage they read it again and nobody uses them)
    load_acts(min(s + 2, nstages - 1), apre);
    load_weights(min(s + 2, nstages - 1), pre);
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      Frag af[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt].r = lds[b][mt * 16 + c][(kh * (KU * 4) + u * 4 + g) ^ c];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[rt][u].v, af[mt].v, acc[rt][mt], 0, 0, 0);
    }
  };

  Frag w0[RT][KU], w1[RT][KU], w2[RT][KU];
  u32x4_t a0[NA], a1[NA], a2[NA];
  if (nstages > 0) {
    load_acts(0, a0);
    load_weights(0, w0);
    load_acts(min(1, nstages - 1), a1);
    load_weights(min(1, nstages - 1), w1);
  }
  // three stages a turn so that the register sets take turns without copies; the turn has no
  // branches inside, which keeps the compiler's count of loads in flight exact
  int s = 0;
  for (; s + 3 <= nstages; s += 3) {
    stage(s, w0, w2, a0, a2);
    stage(s + 1, w1, w0, a1, a0);
    stage(s + 2, w2, w1, a2, a1);
  }
  if (s < nstages) {
    stage(s, w0, w2, a0, a2);
    if (s + 1 < nstages) stage(s + 1, w1, w0, a1, a0);
  }

  // add the slices of K in a fixed order: the waves of slices 1.. hand their sums over through LDS
  float* red = reinterpret_cast<float*>(&lds[0][0][0]);
  __syncthreads();
  if (kh > 0) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          red[((((kh - 1) * NR + rg) * RT * MT + rt * MT + mt) * 4 + r) * 64 + lane] = acc[rt][mt][r];
  }
  __syncthreads();
  if (kh > 0) return;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float sum = acc[rt][mt][r];
#pragma unroll
        for (int h = 1; h < KH; ++h) sum += red[((((h - 1) * NR + rg) * RT * MT + rt * MT + mt) * 4 + r) * 64 + lane];
        acc[rt][mt][r] = sum;
      }
  if (QKV && head >= qa.Hq + 2 * qa.Hk) return;
  store_tiles<RT, MT, TC, EPI>(acc, C, M, N, m0, n0, head, t16, qa, ql, g, c);
}

template <int RT, int MT, int NR, int KH, typename TC, int EPI>
static int launch_mid(const void* A, const void* W, void* C, int M, int N, int K, int up_offset, int parts,
                      const QkvRopeArgs& qa, hipStream_t stream) {
  unsigned tiles;
  if (EPI == EPI_SWIGLU) tiles = (N + 15) / 16;
  else if (EPI == EPI_QKV_ROPE) tiles = (qa.Hq + 2 * qa.Hk) * (qa.D >> 4);
  else tiles = (N + RT * 16 - 1) / (RT * 16);
  dim3 grid((tiles + NR - 1) / NR, (M + MT * 16 - 1) / (MT * 16), parts);
  if (grid.y > 65535 || parts < 1 || parts > 64) return SA_ERR_ARG;
  hipLaunchKernelGGL((gemm_mid_kernel<RT, MT, NR, KH, TC, EPI>), grid, dim3(64 * NR * KH), 0, stream,
                     (const bf16_t*)A, (const bf16_t*)W, (TC*)C, M, N, K, up_offset, qa);
  SA_LAUNCH_CHECK();
  return 0;
}

// The same products with both operands loaded straight into LDS (global_load_lds: 16 bytes a lane,
// no registers in between, so nothing has to be held for stages that are on their way).  A
// workgroup owns NT tiles of 16 rows of W (four; eight for matrices with so many rows that four
// would give more workgroups than one round of the chip holds; sixteen for the head over a large
// vocabulary) and BM = 64 MW rows of A; a stage is 64 columns of K of both, one kilobyte an
// instruction (8 rows of 128 bytes), in a ring of NB stages.  A row of a stage holds 8 segments of
// 16 bytes; segment s of row r lies at slot s ^ ((r >> 1) & 7).  A 16-byte LDS read serves 16 lanes
// a cycle, and not 16 neighbours: lanes 0-3, 12-15, 20-23, 24-27 together, then 4-7, 8-11, 16-19,
// 28-31, then the same plus 32; with this exchange each such group of a fragment read (lane l: row
// l % 16, segment l / 16 of its half stage) touches every bank once (the counter of bank
// conflicts stays at zero).  The loads apply the same exchange on their way in by choosing which
// segment a lane fetches.  Eight waves:
// wave = (mw, kh), mw = which quarter of the rows (MW tiles of 16), kh = which half (32 columns)
// of every stage; the two halves add their sums through LDS at the end, in a fixed order.  A
// wave waits for its own loads with the counter of loads in flight (they land in order), then
// the workgroup's barrier says that everybody's have landed and that the stage before has been
// read, so its place in the ring can be filled again.  Needs K to be whole stages for every part
// (K % (64 parts) == 0: a stage cannot be zeroed on its way into LDS); rows beyond M and N are
// read from the last row and their sums never stored.
#define SA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | (0x7 << 4) | (0xf << 8))

template <int MW, int NT, int NB, typename TC, int EPI, int SPB = 1>
__global__ __launch_bounds__(512) void gemm_wide_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                       TC* __restrict__ C, int M, int N, int K, int up_offset,
                                                       QkvRopeArgs qa) {
  constexpr bool SWIGLU = EPI == EPI_SWIGLU;
  constexpr bool QKV = EPI == EPI_QKV_ROPE;
  static_assert(NT == 1 || NT == 2 || NT == 4 || NT == 8 || NT == 16, "tiles of 16 weight rows, 8 rows a wave and instruction");
  static_assert(!SWIGLU || NT >= 2, "SwiGLU: half of the tiles are the gate's, half are up's");
  constexpr int BM = 64 * MW;
  constexpr int BN = 16 * NT;
  constexpr int A_BYTES = BM * 128;
  constexpr int STAGE_BYTES = A_BYTES + BN * 128;
  constexpr int COLS = SWIGLU ? BN / 2 : BN;       // output columns of a workgroup
  // weight loads per stage: 2 NT instructions of 8 rows; with four tiles and more every wave issues NT / 4
  // of them, with fewer the first 2 NT waves issue one each
  constexpr int NWI = NT >= 4 ? NT / 4 : 1;
  constexpr int ND = MW + NWI;
  static_assert(ND * (NB - 1) < 64, "the counter of loads in flight has six bits");
  static_assert(SPB >= 1 && NB % SPB == 0 && NB >= 2 * SPB, "SPB stages between two barriers, in a ring of whole groups of them");
  static_assert(NB * STAGE_BYTES >= 4 * MW * NT * 4 * 64 * 4, "the sums of the second K half reuse the ring");
  extern __shared__ __attribute__((aligned(16))) u32x4_t wide_lds[];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int mw = wave & 3;
  const int kh = wave >> 2;
  const int m0 = blockIdx.z * BM;
  const int n0 = blockIdx.x * COLS;
  const bool has_w = NT >= 4 || wave < 2 * NT;     // (wave-uniform) whether this wave fetches weight rows
  // the rotating epilogue: a tile holds eight dims of a head and their partners half a head further on
  const int tph = QKV ? (qa.D >> 4) : 1;
  const int tile0 = blockIdx.x * NT;

  const int nstages = (K >> 6) / gridDim.y;
  const int k_begin = blockIdx.y * nstages * 64;
  // (stages walked in an order rotated per workgroup, as in gemm_mid_kernel; it depends on the
  // weight rows only)
  const int rot = (int)(blockIdx.x % (unsigned)nstages);
  auto stage_k = [&](int s) __attribute__((always_inline)) {
    int t = min(s, nstages - 1) + rot;             // past the last stage: the last again (nobody reads it)
    if (t >= nstages) t -= nstages;
    return k_begin + t * 64;
  };
  C += (size_t)blockIdx.y * M * N;

  // what this lane fetches: instruction d of wave w fills rows 8 (w MW + d) .. + 7 of the stage's
  // activations, 8 lanes a row; the wave's last instructions fill 8 weight rows each
  const bf16_t* src[ND];
#pragma unroll
  for (int d = 0; d < MW; ++d) {
    const int row = (wave * MW + d) * 8 + (lane >> 3);
    const int seg = (lane & 7) ^ ((row >> 1) & 7);
    src[d] = A + (size_t)min(m0 + row, M - 1) * K + seg * 8;
  }
#pragma unroll
  for (int d = 0; d < NWI; ++d) {
    const int row = ((has_w ? wave : 0) * NWI + d) * 8 + (lane >> 3);       // of the workgroup's BN weight rows
    const int seg = (lane & 7) ^ ((row >> 1) & 7);
    int n;
    if (SWIGLU) {
      n = row < BN / 2 ? min(n0 + row, N - 1) : up_offset + min(n0 + row - BN / 2, N - 1);
    } else if (QKV) {
      const int tile = tile0 + (row >> 4), cc = row & 15;
      const int head = tile / tph, t16 = tile - head * tph;
      n = head < qa.Hq + 2 * qa.Hk ? head * qa.D + t16 * 8 + (cc < 8 ? cc : (qa.D >> 1) + cc - 8) : 0;
    } else {
      n = min(n0 + row, N - 1);
    }
    src[MW + d] = W + (size_t)n * K + seg * 8;
  }
  typedef __attribute__((address_space(3))) u32x4_t* lds_ptr_t;
  typedef const __attribute__((address_space(1))) void* gptr_t;
  const lds_ptr_t lds0 = (lds_ptr_t)wide_lds;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds0;
  // this lane's fragment of tile 0 of its rows (and of weight tile 0), in the first place of the ring
  const uint32_t slot16 = (uint32_t)(((kh * 4 + g) ^ ((c >> 1) & 7)) * 16);
  const uint32_t a_addr = lds_base + (uint32_t)((mw * MW * 16 + c) * 128) + slot16;
  const uint32_t w_addr = lds_base + A_BYTES + (uint32_t)(c * 128) + slot16;

  // what the rotating epilogue needs besides the sums, fetched beside the first stages
  QkvLane<MW> ql[QKV ? NT : 1] = {};
  if (QKV && kh == 0) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tile = tile0 + nt, head = tile / tph;
      ql[nt] = load_qkv_lane<MW>(qa, M, m0 + mw * MW * 16, head, tile - head * tph, g, c);
    }
  }

  floatx4_t acc[MW][NT];
#pragma unroll
  for (int mt = 0; mt < MW; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  auto fetch = [&](int s) __attribute__((always_inline)) {
    const int k0 = stage_k(s);
    const lds_ptr_t buf = lds0 + (s % NB) * (STAGE_BYTES / 16);
#pragma unroll
    for (int d = 0; d < MW; ++d)
      __builtin_amdgcn_global_load_lds((gptr_t)(src[d] + k0), (__attribute__((address_space(3))) void*)
                                       (buf + (wave * MW + d) * 64), 16, 0, 0);
    if (has_w) {
#pragma unroll
      for (int d = 0; d < NWI; ++d)
        __builtin_amdgcn_global_load_lds((gptr_t)(src[MW + d] + k0), (__attribute__((address_space(3))) void*)
                                         (buf + A_BYTES / 16 + (wave * NWI + d) * 64), 16, 0, 0);
    }
  };

  // SPB stages between two barriers (two where a stage is so little work, one product a wave, that the
  // barrier and the trip through LDS are what a stage takes; the launcher then gives an even number of stages)
#pragma unroll
  for (int i = 0; i < NB - SPB; ++i) fetch(i);
  for (int s = 0; s < nstages; s += SPB) {
    // this wave's part of stages s .. s + SPB - 1 lies in LDS: all of its loads but those of the NB - 2 SPB
    // stages after them have landed
    if (has_w) SA_WAIT_VMCNT(ND * (NB - 2 * SPB));
    else SA_WAIT_VMCNT(MW * (NB - 2 * SPB));
    __builtin_amdgcn_s_barrier();              // everybody's does, and everybody has read the stages before s
#pragma unroll
    for (int u = 0; u < SPB; ++u) fetch(s + NB - SPB + u);
    // (the reads are written as instructions of their own: the compiler does not see the loads
    // into LDS as stores, and would otherwise wait for all of them before every read)
    Frag af[SPB][MW], wf[SPB][NT];
#pragma unroll
    for (int u = 0; u < SPB; ++u) {
      const uint32_t boff = (uint32_t)(((s + u) % NB) * STAGE_BYTES);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(wf[u][nt].r) : "v"(w_addr + boff), "n"(nt * 16 * 128));
#pragma unroll
      for (int mt = 0; mt < MW; ++mt)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[u][mt].r) : "v"(a_addr + boff), "n"(mt * 16 * 128));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int u = 0; u < SPB; ++u) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) asm volatile("" : "+v"(wf[u][nt].r));
#pragma unroll
      for (int mt = 0; mt < MW; ++mt) asm volatile("" : "+v"(af[u][mt].r));
    }
#pragma unroll
    for (int u = 0; u < SPB; ++u)
#pragma unroll
      for (int mt = 0; mt < MW; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][nt].v, af[u][mt].v, acc[mt][nt], 0, 0, 0);
  }

  // the second half of K hands its sums over through LDS (no load into LDS may still be on its way)
  float* red = reinterpret_cast<float*>(wide_lds);
  SA_WAIT_VMCNT(0);
  __syncthreads();
  if (kh == 1) {
#pragma unroll
    for (int mt = 0; mt < MW; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        *reinterpret_cast<floatx4_t*>(&red[((((mw * MW + mt) * NT + nt) * 64) + lane) * 4]) = acc[mt][nt];
  }
  __syncthreads();
  if (kh == 1) return;
#pragma unroll
  for (int mt = 0; mt < MW; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      acc[mt][nt] += *reinterpret_cast<const floatx4_t*>(&red[((((mw * MW + mt) * NT + nt) * 64) + lane) * 4]);

  if constexpr (QKV) {
    // tile by tile through the epilogue of the kernels above: rotation, q to its buffer, k and v into the cache
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tile = tile0 + nt, head = tile / tph, t16 = tile - head * tph;
      if (head >= qa.Hq + 2 * qa.Hk) continue;             // (wave-uniform)
      floatx4_t one[1][MW];
#pragma unroll
      for (int mt = 0; mt < MW; ++mt) one[0][mt] = acc[mt][nt];
      store_tiles<1, MW, TC, EPI>(one, C, M, N, m0 + mw * MW * 16, head * qa.D + t16 * 8, head, t16, qa, ql[nt], g, c);
    }
    return;
  }
  // lane l holds C[m = row tile's row l % 16][n = 4 (l / 16) .. + 3] of every tile pair
#pragma unroll
  for (int mt = 0; mt < MW; ++mt) {
    const int m = m0 + (mw * MW + mt) * 16 + c;
    if (m >= M) continue;
#pragma unroll
    for (int nt = 0; nt < (SWIGLU ? NT / 2 : NT); ++nt) {
      const int n = n0 + nt * 16 + 4 * g;
      float o[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (SWIGLU) {
          const float gt = acc[mt][nt][r];
          o[r] = (gt / (1.f + __expf(-gt))) * acc[mt][SWIGLU ? nt + NT / 2 : nt][r];
        } else {
          o[r] = acc[mt][nt][r];
        }
      }
      if (n + 3 < N) {
        store4(C + (size_t)m * N + n, o, (N & 3) == 0);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) C[(size_t)m * N + n + r] = from_float<TC>(o[r]);
      }
    }
  }
}

template <int MW, int NT, int NB, typename TC, int EPI, int SPB = 1>
static int launch_wide(const void* A, const void* W, void* C, int M, int N, int K, int up_offset, int parts,
                       const QkvRopeArgs& qa, hipStream_t stream) {
  if (SPB > 1 && ((K >> 6) / parts) % SPB) return SA_ERR_ARG;      // whole groups of SPB stages
  constexpr int BM = 64 * MW;
  constexpr int COLS = EPI == EPI_SWIGLU ? 8 * NT : 16 * NT;
  constexpr size_t lds_bytes = (size_t)NB * (BM + 16 * NT) * 128;
  static_assert(lds_bytes <= 160 * 1024, "the LDS of a compute unit");
  unsigned gx = (N + COLS - 1) / COLS;
  if (EPI == EPI_QKV_ROPE) gx = ((qa.Hq + 2 * qa.Hk) * (qa.D >> 4) + NT - 1) / NT;
  dim3 grid(gx, parts, (M + BM - 1) / BM);
  if (grid.z > 65535 || parts < 1 || parts > 64) return SA_ERR_ARG;
  auto kernel = gemm_wide_kernel<MW, NT, NB, TC, EPI, SPB>;
  if (lds_bytes > 64 * 1024) {  // more dynamic LDS than a kernel gets without asking
    static bool allowed[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return SA_ERR_ARG;
    if (!allowed[dev]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
      if (e != hipSuccess) return (int)e;
      allowed[dev] = true;
    }
  }
  hipLaunchKernelGGL(kernel, grid, dim3(512), lds_bytes, stream, (const bf16_t*)A, (const bf16_t*)W, (TC*)C, M, N, K,
                     up_offset, qa);
  SA_LAUNCH_CHECK();
  return 0;
}

// Which products gemm_wide_kernel takes, from timings beside the two kernels above at the sizes of the
// Llama-3 family (widths 2048, 3072, 4096) with cold weights, 1 to 128 rows; in microseconds, this kernel
// against the other:
//   gate/up + SwiGLU: K 2048, 2 x 8192 rows of W: level up to 12 rows, 13.7 / 14.1 at 16, 13.7 / 16.7 at 32,
//     14.5 / 18.6 at 64, 19.0 / 24.5 at 128; K 3072, 2 x 8192: 20.2 / 21.0 at one row, 20.1 / 23.4 at 16,
//     22.5 / 27.8 at 64, 29.8 / 35.5 at 128; K 4096, 2 x 14336 (128 rows of W a workgroup): 45.3 / 48.6 at one
//     row, 45.4 / 47.7 at 16, 45.8 / 54.8 at 64, 53.2 / 81.7 at 128;
//   the head over 128,256 rows of W: K 2048: 99 / 95 at 8 rows, 118 / 118 at 48, 145 / 163 at 96, 159 / 185 at
//     128; K 3072: 135 / 148 at one row, 139 / 153 at 16, 169 / 197 at 64, 210 / 266 at 128; K 4096: 177 / 204
//     at one row, 176 / 290 at 12, 197 / 302 at 64, 238 / 319 at 128;
//   narrow matrices in fp32 parts: down_proj K 8192, 2048 rows of W (eight parts against four): 8.9 / 8.4 at 8
//     rows, 9.5 / 9.5 at 32, 10.8 / 12.3 at 64, 15.3 / 17.8 at 128; K 8192, 3072 rows (four parts): 12.6 /
//     10.7 at one row, 12.3 / 12.9 at 4, 13.4 / 16.0 at 32, 15.9 / 21.2 at 64, 22.2 / 32.3 at 128; K 14336, 4096
//     rows: level up to 8 rows, 23.0 / 27.6 at 32, 26.4 / 35.6 at 64, 48 / 53 at 128; o_proj K 2048: 5.4 / 4.2
//     at 8 rows, 7.4 / 6.1 at 64, 10.5 / 8.7 at 128 (the other kernel stays); K 3072: 7.4 / 7.0 at one row,
//     6.8 / 8.1 at 4, 9.4 / 14.1 at 64, 13.9 / 20.2 at 128; K 4096: 9.0 / 8.1 at one row, 9.0 / 9.2 at 8, 10.9 /
//     14.7 at 64, 15.1 / 22.5 at 128.
//   q/k/v + rotation + cache write (16 weight rows a workgroup, 32 where 16 would give more workgroups than
//     compute units): K 2048, 3072 rows of W: 10.0 / 6.0 at one row, 10.2 / 8.4 at 32, 10.7 / 11.5 at 64, 13.6 / 17.3
//     at 128; K 3072, 5120 rows: 15.8 / 16.5 at 48, 16.0 / 19.4 at 64, 21.8 / 28.5 at 128; K 4096, 6144 rows: 19.6 /
//     19.5 at 48, 20.5 / 22.2 at 64, 26.8 / 33.5 at 128.  (Measured with one stage between two barriers; with two,
//     see pick_wide, it is ahead from 40 rows on.)
// 129 to 192 rows, against the BLAS library (and its SwiGLU pass): gate/up 22.7 / 30.6 at 160 rows and 24.4 / 31.0
// at 192 with K 2048, 34.5 / 36.4 and 37.2 / 40.6 with K 3072, 62.2 / 65.8 and 64.0 / 68.7 with K 4096; down_proj
// 18.4 / 25.7 and 20.8 / 26.9 (K 8192, 2048 rows), 26.0 / 27.6 and 29.2 / 58.5 (3072 rows), 57.4 / 83.4 and 64.9 /
// 102.6 (K 14336); o_proj 15.9 / 16.6 and 17.8 / 26.6 (K 3072), 17.9 / 26.7 and 19.5 / 32.2 (K 4096).  Beyond 192
// rows the library is ahead for most of them (and for the head from 129 on), but not for gate/up of the smaller
// models: 26.9 / 32.8 at 224 rows and 28.2 / 34.5 at 256 with K 2048, 40.4 / 44.6 and 42.3 / 46.7 with K 3072
// (K 4096, 2 x 14336 rows: 78 / 75 and 81 / 78).
// So: the longer a workgroup's walk along K, the fewer rows it takes for this kernel to be ahead.
template <typename TC, int EPI>
static bool takes_wide(int M, int N, int K, int parts) {
  if (M < 1 || M > 256 || (K & 63) || parts < 1 || (K >> 6) % parts) return false;
  const int stages = (K >> 6) / parts;             // of a workgroup
  if (stages < 2) return false;
  // q/k/v: from 64 rows; from 40 where the stages come in pairs (two of them between two barriers, see pick_wide)
  if (EPI == EPI_QKV_ROPE) return M <= 128 && (M >= 64 || (M >= 40 && (stages & 1) == 0));
  // gate/up: beyond 192 rows only for matrices of up to 64 M elements, for which the library's fixed costs weigh most
  if (EPI == EPI_SWIGLU) return (K >= 3072 || M >= 16) && (M <= 192 || 2ll * N * K <= (64ll << 20));
  if (M > 192) return false;
  // the head: from 48 rows, from one row with a long walk along K, and from 8 rows over a vocabulary of 64 K
  // rows and more, which takes 256 weight rows a workgroup (see pick_wide)
  if (N >= 8192) return parts == 1 && M <= 128 && (K >= 3072 || M >= 48 || (N >= 65536 && M >= 8));
  // narrow matrices: a walk of twelve stages and more, and enough parts to give half the compute units a
  // workgroup; from three rows on for matrices of 24 M elements and more, above 32 rows for smaller ones
  if (stages < 12 || ((N + 63) / 64) * parts < 128) return false;
  return M > 32 || (M > 2 && (long long)N * K >= (24ll << 20));
}

template <typename TC, int EPI>
static int pick_wide(const void* A, const void* W, void* C, int M, int N, int K, int up_offset, int parts,
                     const QkvRopeArgs& qa, hipStream_t stream) {
  // one to four groups of 64 rows of A; 64 rows of W a workgroup, or 128 where 64 would give more workgroups
  // than there are compute units (K 4096, 2 x 14336 rows of W, 64 rows of A: 45 us against 60; the
  // head over 128,256 rows at 128 rows of A: 161 against 180 with K 2048, 239 against 294 with K 4096);
  // the ring as deep as measured to pay
#define GO(MW, NT, NB) return launch_wide<MW, NT, NB, TC, EPI>(A, W, C, M, N, K, up_offset, parts, qa, stream)
  if constexpr (EPI == EPI_QKV_ROPE) {
    // few weight rows in all: 16 of them a workgroup, or 32 where that still gives every compute unit one
    // With one product a wave and stage, the barrier and the trip through LDS are what a stage takes: up to
    // 64 rows two stages go between two barriers, in a ring of eight (K 2048, 3072 rows of W: 8.1 us
    // against 10.2 at 40 rows and 9.1 with gemm_mid_kernel, 8.9 against 10.9 at 64; K 3072, 5120 rows: 13.8
    // against 15.8 at 40 and 15.6 with gemm_mid_kernel, 15.6 against 16.1 at 64; K 4096, 6144 rows: 17.9
    // against 19.8 at 40 and 19.1, 20.2 against 20.5 at 64; no gain with more rows)
    const int tiles = (qa.Hq + 2 * qa.Hk) * (qa.D >> 4);
    const bool two = tiles > compute_units();
    if (M <= 64) {
      if ((((K >> 6) / parts) & 1) == 0) {
        if (two) return launch_wide<1, 2, 8, TC, EPI, 2>(A, W, C, M, N, K, up_offset, parts, qa, stream);
        return launch_wide<1, 1, 8, TC, EPI, 2>(A, W, C, M, N, K, up_offset, parts, qa, stream);
      }
      if (two) GO(1, 2, 6);
      GO(1, 1, 6);
    }
    if (two) GO(2, 2, 5);
    GO(2, 1, 5);
  } else {
    const long long rows_w = EPI == EPI_SWIGLU ? 2ll * N : N;
    const bool many = (rows_w + 63) / 64 * parts > compute_units();
    // the head over a vocabulary of 64 K rows and more: 256 weight rows a workgroup (two rounds of the chip
    // and more), which halves what a workgroup reads of the activations per weight row once more.  Over
    // 128,256 rows against 128 rows a workgroup, in microseconds: K 2048: 95 / 103 at 8 rows of A (99 with
    // gemm_mid_kernel), 104 / 111 at 32, 116 / 127 at 64, 139 / 160 at 128; K 3072: level up to 32 rows, 152 /
    // 155 at 40, 166 / 174 at 64, 192 / 211 at 128; K 4096: 186 / 180 at 8, 207 / 204 at 64, 220 / 228 at 96,
    // 230 / 241 at 128.
    if constexpr (EPI == EPI_PLAIN) {
      if (parts == 1 && N >= 65536 && M <= 128 && (K < 3072 || (K < 4096 ? M >= 40 : M > 64))) {
        if (M <= 64) GO(1, 16, 3);
        GO(2, 16, 3);
      }
    }
    if (M <= 64) {
      if (many) GO(1, 8, 4);
      GO(1, 4, 4);
    }
    if (M <= 128) {
      if (many) GO(2, 8, 4);
      GO(2, 4, 5);
    }
    if (M <= 192) {
      if (many) GO(3, 8, 3);
      GO(3, 4, 4);
    }
    if (many) GO(4, 8, 3);
    GO(4, 4, 3);
  }
#undef GO
  return SA_ERR_ARG;
}

// up to this many rows take gemm_skinny_kernel, more take gemm_mid_kernel
// Which kernel and which workgroup shape a product takes, from a sweep over both kernels and their
// shapes at the sizes of the Llama-3 family (widths 2048 to 4096), 1 to 64 rows, weights cold.
// gemm_skinny_kernel, where every wave fetches its own activation rows, wins only at one or two rows
// (and for the small fused q/k/v products up to eight); from there on sharing the activations of a
// workgroup through LDS is faster, and the question is how many weight rows a workgroup takes
// (more halve the activation traffic, fewer give more workgroups) and how many ways it cuts a stage
// of K.  Few weight rows in all: small workgroups, K cut often; many: 128 rows a workgroup.
template <typename TC, int EPI>
static bool takes_skinny(int M, int N, const QkvRopeArgs& qa) {
  if (EPI == EPI_QKV_ROPE) return (qa.Hq + 2 * qa.Hk) * (qa.D >> 4) < 256 && M <= 8;
  return M <= 2;
}

// workgroup shapes (row groups x K slices) of products with 65 to 128 rows of activations
constexpr int MID8_PLAIN_NR = 2, MID8_PLAIN_KH = 4;
constexpr int MID8_SWIGLU_NR = 2, MID8_SWIGLU_KH = 4;
constexpr int MID8_HEAD_NR = 4, MID8_HEAD_KH = 2;

template <typename TC, int EPI>
static int pick_mid(const void* A, const void* W, void* C, int M, int N, int K, int up_offset, int parts,
                    const QkvRopeArgs& qa, hipStream_t stream) {
  // 16-row tiles of activations per pass, as many as the rows need: up to 128 rows in one pass
  // (more rows: more passes, each streaming the weights again, which the caller avoids)
  const int mt = min(8, (M + 15) / 16);
#define GO(RT, MT, NR, KH) \
  return launch_mid<RT, MT, NR, KH, TC, EPI>(A, W, C, M, N, K, up_offset, parts, qa, stream)
  // up to four tiles: a workgroup shape for one, for two, and for three or four tiles
#define GO3(RT, NR1, KH1, NR2, KH2, NR4, KH4) \
  do {                                         \
    if (mt == 1) GO(RT, 1, NR1, KH1);          \
    if (mt == 2) GO(RT, 2, NR2, KH2);          \
    if (mt == 3) GO(RT, 3, NR4, KH4);          \
    if (mt == 4) GO(RT, 4, NR4, KH4);          \
  } while (0)
  // five to eight tiles: one shape (a workgroup then has 512 threads or more: fewer would hold too
  // many activation segments each on their way into LDS)
#define GO8(RT, NR, KH)                   \
  do {                                    \
    if (mt == 5) GO(RT, 5, NR, KH);       \
    if (mt == 6) GO(RT, 6, NR, KH);       \
    if (mt == 7) GO(RT, 7, NR, KH);       \
    GO(RT, 8, NR, KH);                    \
  } while (0)
  if constexpr (EPI == EPI_PLAIN) {
    if (N < 8192) {
      GO3(1, 2, 4, 2, 4, 2, 4);                // 32 weight rows a workgroup, K cut four ways inside it
      GO8(1, MID8_PLAIN_NR, MID8_PLAIN_KH);
    }
    if (M <= 8) GO(1, 1, 4, 2);                // the head: 64 weight rows, or 128 with two passes' worth of rows
    if (M <= 32) GO(1, 2, 8, 2);
    if (M <= 64) GO(1, 4, 8, 2);
    GO8(1, MID8_HEAD_NR, MID8_HEAD_KH);
  }
  if constexpr (EPI == EPI_QKV_ROPE) {
    const int tiles = (qa.Hq + 2 * qa.Hk) * (qa.D >> 4);
    if (tiles < 256) {
      // one 16-row tile a workgroup, K cut eight ways.  From 49 rows on two passes of half the rows
      // (the second finds the weights in L2) fill the chip better than one pass with half as many
      // workgroups (about 3 us less at 128 rows, 1 us at 64, 1B shape)
      if (mt == 4) GO(1, 2, 1, 8);
      GO3(1, 1, 8, 1, 8, 1, 8);
      if (mt <= 6) GO(1, 3, 1, 8);
      GO(1, 4, 1, 8);
    }
    GO3(1, 2, 2, 2, 4, 2, 4);                    // two tiles
    GO8(1, 2, 4);
  }
  if constexpr (EPI == EPI_SWIGLU) {
    const int tiles = (N + 15) / 16;             // N: rows of the gate (and of the up) matrix
    if (tiles < 768) {
      GO3(2, 1, 8, 2, 2, 2, 2);                  // 32 to 64 weight rows a workgroup
      GO8(2, MID8_SWIGLU_NR, MID8_SWIGLU_KH);
    }
    GO3(2, 4, 2, 4, 2, 4, 2);                    // 128
    GO8(2, MID8_SWIGLU_NR, MID8_SWIGLU_KH);
  }
#undef GO8
#undef GO3
#undef GO
  return SA_ERR_ARG;
}

template <int RT, int MT, int KS, int KU, typename TC, int EPI>
static int launch_skinny(const void* A, const void* W, void* C, int M, int N, int K, int up_offset,
                         int parts, const QkvRopeArgs& qa, hipStream_t stream) {
  unsigned gx;
  if (EPI == EPI_SWIGLU) gx = (N + 15) / 16;
  else if (EPI == EPI_QKV_ROPE) gx = (qa.Hq + 2 * qa.Hk) * (qa.D >> 4);
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
  // one or two rows of activations, eight for a small fused q/k/v product (more take the kernel above).
  // Many weight rows: 2 row tiles per wave and few waves; few rows: more waves splitting K.
#define GO(RT, MT, KS, KU) \
  return launch_skinny<RT, MT, KS, KU, TC, EPI>(A, W, C, M, N, K, up_offset, parts, qa, stream)
  // (the choices below are the best of a sweep over RT, KS and KU at the Llama-3.2-1B sizes; the
  // sweep is flat: every shape that fills the chip runs at about 3 us + bytes / 5.3 TB/s)
  if constexpr (EPI == EPI_QKV_ROPE) GO(1, 1, 8, 8);
  if constexpr (EPI == EPI_SWIGLU) {
    if (K >= 4096) GO(2, 1, 4, 8);   // a long inner dimension: four waves share it
    GO(2, 1, 2, 8);
  }
  if constexpr (EPI == EPI_PLAIN) {
    if (N >= 8192) GO(2, 1, 2, 8);
    if (parts > 1) GO(1, 1, 2, 8);   // K is already cut across workgroups: 2 waves each
    GO(1, 1, 16, 4);
  }
#undef GO
  return SA_ERR_ARG;
}

// whether a product of these sizes goes to gemm_wide_kernel (epi: EPI_PLAIN, EPI_SWIGLU, for which N is the
// number of gate rows, or EPI_QKV_ROPE): for the caller's choice of `parts`, and for tests
extern "C" int sa_gemm_bf16_takes_wide(int epi, int M, int N, int K, int parts) {
  if (epi == EPI_SWIGLU) return takes_wide<bf16_t, EPI_SWIGLU>(M, N, K, parts) ? 1 : 0;
  if (epi == EPI_QKV_ROPE) return takes_wide<bf16_t, EPI_QKV_ROPE>(M, N, K, parts) ? 1 : 0;
  if (epi == EPI_PLAIN) return takes_wide<float, EPI_PLAIN>(M, N, K, parts) ? 1 : 0;
  return 0;
}

// C = A W^T; c_dtype SA_BF16 or SA_F32.  parts > 1 (fp32 only): C is [parts, M, N] and holds
// partial sums over `parts` slices of K, to be added by the consumer.
extern "C" int sa_gemm_bf16_skinny(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K,
                                   int parts, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || parts < 1) return SA_ERR_ARG;
  const QkvRopeArgs none = {};
  if (takes_wide<float, EPI_PLAIN>(M, N, K, parts)) {
    if (c_dtype == SA_BF16 && parts == 1) return pick_wide<bf16_t, EPI_PLAIN>(A, W, C, M, N, K, 0, 1, none, stream);
    if (c_dtype == SA_F32) return pick_wide<float, EPI_PLAIN>(A, W, C, M, N, K, 0, parts, none, stream);
    return SA_ERR_UNSUPPORTED;
  }
  if (!takes_skinny<float, EPI_PLAIN>(M, N, none)) {
    if (c_dtype == SA_BF16 && parts == 1) return pick_mid<bf16_t, EPI_PLAIN>(A, W, C, M, N, K, 0, 1, none, stream);
    if (c_dtype == SA_F32) return pick_mid<float, EPI_PLAIN>(A, W, C, M, N, K, 0, parts, none, stream);
    return SA_ERR_UNSUPPORTED;
  }
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
  if (takes_wide<bf16_t, EPI_SWIGLU>(M, I, K, 1)) return pick_wide<bf16_t, EPI_SWIGLU>(A, W, C, M, I, K, I, 1, none, stream);
  if (!takes_skinny<bf16_t, EPI_SWIGLU>(M, I, none)) return pick_mid<bf16_t, EPI_SWIGLU>(A, W, C, M, I, K, I, 1, none, stream);
  return pick_skinny<bf16_t, EPI_SWIGLU>(A, W, C, M, I, K, I, 1, none, stream);
}

// q, k, v = A [Wq; Wk; Wv]^T with W stacked as [(Hq + 2 Hk) D, K]; q and k rotated by position
// (pairs (j, j + D/2), all D dims); q goes to Q [M, Hq D], k and v into the cache pages.
// Needs D % 16 == 0.
extern "C" int sa_gemm_bf16_qkv_rope(const void* A, const void* W, void* Q, const int* positions,
                                     const float* inv_freq, const int* slots, void* k_pages, void* v_pages,
                                     int M, int K, int Hq, int Hk, int D, int page_size, hipStream_t stream) {
  if (M <= 0) return 0;
  if (K <= 0 || (K & 7) || Hq <= 0 || Hk <= 0 || D <= 0 || (D & 15) || page_size <= 0) return SA_ERR_ARG;
  const QkvRopeArgs qa = {positions, inv_freq, slots, (bf16_t*)k_pages, (bf16_t*)v_pages, Hq, Hk, D, page_size};
  if (takes_wide<bf16_t, EPI_QKV_ROPE>(M, 0, K, 1)) return pick_wide<bf16_t, EPI_QKV_ROPE>(A, W, Q, M, (Hq + 2 * Hk) * D, K, 0, 1, qa, stream);
  if (!takes_skinny<bf16_t, EPI_QKV_ROPE>(M, 0, qa)) return pick_mid<bf16_t, EPI_QKV_ROPE>(A, W, Q, M, (Hq + 2 * Hk) * D, K, 0, 1, qa, stream);
  return pick_skinny<bf16_t, EPI_QKV_ROPE>(A, W, Q, M, (Hq + 2 * Hk) * D, K, 0, 1, qa, stream);
}
