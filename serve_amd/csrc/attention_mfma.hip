// Paged attention on the matrix cores, bf16 in, fp32 softmax and accumulation, for prompt
// portions and single decoded tokens alike.  Compiled once per head size: -DHEAD_DIM=<multiple
// of 16, at most 128>.
//
// Formulas: serve/kernels/attn_prefill.py:56-72,205 and attn_decode.py:99-111,236 (scores scaled
// by D^-0.5 with log2(e) folded in so that exp2 is used, causal mask by absolute position, online
// softmax m/l/O, O/l at the end; query head h reads KV head h / G).  Unlike the reference, the
// key tile (32 keys) is independent of the page size (any multiple of 4), queries of a prompt
// portion sit at positions ctx_before + j, and long contexts are split over several waves whose
// partial (m, l, O) are merged with the running maximum (the reference's merge,
// attn_decode.py:341-348, has none and is switched off).
//
// The rows of a segment are its (token, query head of the group) pairs, row = token * G +
// head_in_group, so the G heads that share a KV head share every K and V load.  Single decoded
// tokens take one wave per (segment, KV head, split of the key range), as workgroups of one wave
// whose parts a merge kernel joins, or, for few requests with short contexts, as workgroups of four
// waves that join their parts through LDS; prompt portions take workgroups that share K and V
// through LDS.
//
// MFMA use (v_mfma_f32_16x16x32_bf16: D[i][j] += sum_k A[i][k] B[k][j]; lane l holds A row l%16,
// B column l%16, k-slots 8*(l/16)..+7, and D[4*(l/16)+r][l%16]):
//   S^T = K Q^T : A = 16 keys x 32 dims of K (16-byte loads along D), B = Q^T.  A lane then holds,
//                 for ITS query column, the scores of eight keys: exactly the eight k-slots it
//                 must supply for the next product, so P never moves between lanes.  The keys of
//                 a block are dealt to the tile rows so that those eight keys are consecutive.
//   O^T = V^T P^T: A = 16 dims x 32 keys of V^T.  Values are stored transposed inside a page
//                 ([Hk, D, page_size]), so eight consecutive keys at one dim are one 16-byte load
//                 (two 8-byte loads when the page size is a multiple of 4 only).
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

union Frag {
  uint4 u;
  uint2 h[2];
  uint16_t s[8];
  bf16x8_t v;
};

constexpr int HD = HEAD_DIM;
constexpr int DC = (HD + 31) / 32;   // 32-wide chunks of the head dim for Q K^T
constexpr int DT = HD / 16;          // 16-wide tiles of the head dim for P V
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 128, "head size must be a multiple of 16 up to 128");

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// two floats to two bf16 (round to nearest even) in one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack2bf(float a, float b) {
  const float2_t f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// maximum over the four lanes l, l^16, l^32, l^48 (the four lane groups of a column) with the row
// swaps of gfx950 instead of two trips through LDS
__device__ __forceinline__ float max_across_groups(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const uint32_t v = __float_as_uint(y);
  const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

struct Masked { static constexpr bool value = true; };
struct Unmasked { static constexpr bool value = false; };

// Single decoded tokens (at most 16 rows per KV head and segment): one wave per (segment, KV head,
// split of the key range), K and V straight from the cache into registers.  PM: how keys map to pages:
//   0  any page size that is a multiple of 4: division per key, 8-byte value runs;
//   1  a power of two of at least 8: shift, 16-byte value runs; a block of 32 keys spans up to four
//      pages and each lane picks its own;
//   2  a power of two of at least 32: a block lies in one page, and every address is a scalar base
//      plus a constant of the lane.
template <int PM, bool LOCAL = false>
__device__ __forceinline__ void attention_tile(
    const int tile, const int seg, const int hk, const int sp, const int q_begin, const int q_len,
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ ctx_len, int Hq, int Hk,
    int page_size, int page_shift, float scale_log2e, int window, int num_splits,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int NT = 1;                                     // column tiles of 16 rows per wave
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int G = Hq / Hk;
  const int rows_total = q_len * G;
  const int r0 = tile * (16 * NT);
  if (r0 >= rows_total) return;
  const int ctx = ctx_len[seg];
  const int ctx_before = ctx - q_len;
  const int j_lo = r0 / G;
  const int j_hi = min(rows_total - 1, r0 + 16 * NT - 1) / G;
  const int hi_key = ctx_before + j_hi;
  int lo_key = 0;
  if (window > 0) lo_key = max(0, ctx_before + j_lo - window + 1);
  const int kb_lo = lo_key >> 5;
  const int kb_hi = hi_key >> 5;
  const int per = (kb_hi - kb_lo + num_splits) / num_splits;   // ceil((kb_hi - kb_lo + 1) / splits)
  // the same for every lane: say so, or the integer division makes the whole loop control vector work
  const int b0 = __builtin_amdgcn_readfirstlane(kb_lo + sp * per);
  const int b1 = __builtin_amdgcn_readfirstlane(min(kb_hi + 1, b0 + per));
  // blocks full_lo .. full_hi are visible as a whole to every row of the tile and need no mask:
  // their last key is at most the first row's position, their first key inside the last row's window
  const int full_hi = __builtin_amdgcn_readfirstlane((ctx_before + j_lo - 31) >> 5);
  const int full_lo = window > 0 ? __builtin_amdgcn_readfirstlane(((ctx_before + j_hi - window) >> 5) + 1) : 0;
  const int* bt = block_table + (size_t)seg * max_pages;

  // this lane's query column in each column tile
  int qpos[NT], tok[NT], head[NT];
  bool rvalid[NT];
  Frag qf[NT][DC];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    const int row = r0 + n * 16 + c;
    rvalid[n] = row < rows_total;
    const int rowc = min(row, rows_total - 1);
    const int j = rowc / G;
    tok[n] = q_begin + j;
    head[n] = hk * G + (rowc - j * G);
    qpos[n] = ctx_before + j;
    const bf16_t* qp = q + (size_t)tok[n] * q_stride + (size_t)head[n] * HD;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      qf[n][dc].u = make_uint4(0, 0, 0, 0);
      if (dc * 32 + g * 8 < HD) qf[n][dc].u = *reinterpret_cast<const uint4*>(qp + dc * 32 + g * 8);
    }
  }

  float m[NT], l[NT];
  floatx4_t acc[DT][NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    m[n] = -INFINITY;
    l[n] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt][n] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
  }

  const size_t k_page_stride = (size_t)Hk * page_size * HD;   // elements per page (K and V alike)
  constexpr bool wide_v = PM >= 1;                             // 8 consecutive keys lie in one page

  // Which key sits in which row of the two 16-key tiles is free to choose.  Row i of tile t holds
  // key 8*(i/4) + 4*t + (i%4) of the block, so that after S^T = K Q^T lane group g holds the
  // scores of keys 8g .. 8g+7: one 16-byte run of V^T per dim when a page holds a multiple of 8 keys.
  struct Block {
    Frag kf[2][DC];
    Frag vf[DT];
  };
  // Page ids.  With a power-of-two page size a block of 32 keys spans at most four pages, the
  // same for every lane: they are fetched with scalar loads one block ahead (`pgn`), which keeps
  // them out of the vector-memory queue, so that waiting for them does not drain the K/V loads.
  const int last_idx = PM >= 1 ? ((ctx - 1) >> page_shift) : 0;
  int pgn[4] = {0, 0, 0, 0};
  auto prefetch_pages = [&](int kb) __attribute__((always_inline)) {
    if (PM == 1) {
      const int first = (kb << 5) >> page_shift;
      int raw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) raw[j] = bt[__builtin_amdgcn_readfirstlane(min(first + j, last_idx))];
#pragma unroll
      for (int j = 0; j < 4; ++j) pgn[j] = __builtin_amdgcn_readfirstlane(max(raw[j], 0));
    } else if (PM == 2) {
      const int idx = __builtin_amdgcn_readfirstlane(min(kb >> (page_shift - 5), last_idx));
      pgn[0] = __builtin_amdgcn_readfirstlane(max(bt[idx], 0));
    }
  };
  auto pick = [&](const int (&pg)[4], int j) __attribute__((always_inline)) {   // two-level select, no branches
    const int lo = (j & 1) ? pg[1] : pg[0];
    const int hi = (j & 1) ? pg[3] : pg[2];
    return (j & 2) ? hi : lo;
  };
  // key index -> (page, offset in the page) for page sizes that are no power of two
  auto locate = [&](int key, int& page, int& off) __attribute__((always_inline)) {
    const int idx = key / page_size;
    off = key - idx * page_size;
    page = max(bt[idx], 0);
  };
  // PM 2: where this lane's 16 bytes lie relative to the block's first key (in elements)
  const unsigned koff0 = (unsigned)(8 * (c >> 2) + (c & 3)) * HD + g * 8;   // tile 1: + 4 keys
  const unsigned voff0 = (unsigned)c * page_size + 8 * g;
  auto load_block = [&](int kb, Block& blk) __attribute__((always_inline)) {
    const int key0 = kb << 5;
    if (PM == 2) {
      // the whole block lies in page pgn[0].  Keys at or beyond the end of the context are read as
      // they lie in the page (it is the request's own) and masked afterwards.
      const int inpage = key0 & (page_size - 1);
      const bf16_t* kbase = k_pages + (size_t)pgn[0] * k_page_stride + ((size_t)hk * page_size + inpage) * HD;
      const bf16_t* vbase = v_pages + (size_t)pgn[0] * k_page_stride + (size_t)hk * HD * page_size + inpage;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
          blk.kf[t][dc].u = make_uint4(0, 0, 0, 0);
          if (dc * 32 + g * 8 < HD)
            blk.kf[t][dc].u = *reinterpret_cast<const uint4*>(kbase + (koff0 + t * 4 * HD + dc * 32));
        }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        blk.vf[dt].u = *reinterpret_cast<const uint4*>(vbase + (voff0 + (unsigned)(dt * 16) * page_size));
      prefetch_pages(kb + 1);
      return;
    }
    int pg[4] = {pgn[0], pgn[1], pgn[2], pgn[3]};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int ko = 8 * (c >> 2) + 4 * t + (c & 3);
      const int kk = min(key0 + ko, ctx - 1);
      int page, off;
      if (PM == 1) {
        page = pick(pg, ko >> page_shift);
        off = kk & (page_size - 1);
      } else {
        locate(kk, page, off);
      }
      const bf16_t* kp = k_pages + (size_t)page * k_page_stride + ((size_t)hk * page_size + off) * HD;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) {
        blk.kf[t][dc].u = make_uint4(0, 0, 0, 0);
        if (dc * 32 + g * 8 < HD) blk.kf[t][dc].u = *reinterpret_cast<const uint4*>(kp + dc * 32 + g * 8);
      }
    }
    if (wide_v) {
      const int run = min(key0 + 8 * g, (ctx - 1) & ~7);
      const int page = pick(pg, (8 * g) >> page_shift);
      const int off = run & (page_size - 1);
      const bf16_t* vp = v_pages + (size_t)page * k_page_stride + (size_t)hk * HD * page_size + off;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        blk.vf[dt].u = *reinterpret_cast<const uint4*>(vp + (size_t)(dt * 16 + c) * page_size);
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int run = min(key0 + 8 * g + 4 * h, (ctx - 1) & ~3);
        int page, off;
        locate(run, page, off);
        const bf16_t* vp = v_pages + (size_t)page * k_page_stride + (size_t)hk * HD * page_size + off;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          blk.vf[dt].h[h] = *reinterpret_cast<const uint2*>(vp + (size_t)(dt * 16 + c) * page_size);
      }
    }
    prefetch_pages(kb + 1);
  };

  // MASKED: some key of the block is invisible to some row (the causal edge, the window's edge,
  // the end of the context); otherwise no comparison is made at all
  auto compute = [&](int kb, Block& blk, auto masked) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked)::value;
    const int key0 = kb << 5;

    // ---- S^T = K Q^T --------------------------------------------------------------------
    floatx4_t s[2][NT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        s[t][n] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dc = 0; dc < DC; ++dc)
          s[t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kf[t][dc].v, qf[n][dc].v, s[t][n], 0, 0, 0);
      }

    if (MASKED) {
      // keys at or beyond the end of the context, and keys before the window (whose pages may have
      // been given back), hold whatever the page held before: their probability is 0, and 0 times
      // such a value must stay 0
      const int first = key0 + 8 * g;
      uint32_t keep[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k0 = first + 2 * i, k1 = k0 + 1;
        keep[i] = (k0 < ctx && k0 >= lo_key ? 0x0000ffffu : 0u) | (k1 < ctx && k1 >= lo_key ? 0xffff0000u : 0u);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        blk.vf[dt].u.x &= keep[0];
        blk.vf[dt].u.y &= keep[1];
        blk.vf[dt].u.z &= keep[2];
        blk.vf[dt].u.w &= keep[3];
      }
    }

    // ---- online softmax over this lane's 8 keys per column, shared across the 4 lane groups.
    // The scale is positive, so the maximum is taken on the raw scores and the scale is applied
    // inside the exponent: p = 2^(s * scale - m).
    Frag pf[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      float v[2][4];
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float x = s[t][n][r];
          if (MASKED) {
            const int key = key0 + 8 * g + 4 * t + r;
            const bool vis = key <= qpos[n] && (window <= 0 || key > qpos[n] - window);
            x = vis ? x : -INFINITY;
          }
          v[t][r] = x;
          mx = fmaxf(mx, x);
        }
      mx = max_across_groups(mx);
      const float m_new = fmaxf(m[n], mx * scale_log2e);
      // a row that has seen no visible key yet keeps m = -inf; only masked blocks can do that
      const float m_safe = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m[n] - m_safe);
      m[n] = m_new;
      float ps = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v[t][r] = __builtin_amdgcn_exp2f(fmaf(v[t][r], scale_log2e, -m_safe));
          ps += v[t][r];
        }
      l[n] = l[n] * alpha + ps;
      // the running maximum rarely moves after the first blocks: skip the rescaling then
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[dt][n] *= alpha;
      }
      pf[n].u = make_uint4(pack2bf(v[0][0], v[0][1]), pack2bf(v[0][2], v[0][3]),
                           pack2bf(v[1][0], v[1][1]), pack2bf(v[1][2], v[1][3]));
    }

    // ---- O^T += V^T P^T -------------------------------------------------------------------
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int n = 0; n < NT; ++n)
        acc[dt][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.vf[dt].v, pf[n].v, acc[dt][n], 0, 0, 0);
  };

  // Three buffers in turn: the loads of the next two blocks are in flight while one is computed.
  // The loads carry no conditions: a block beyond the last is read from clamped keys and pages and
  // never used.  With a branch around them the compiler no longer knows how many loads are in
  // flight where a block's data is awaited, and waits for all of them, the newest included.
  if (b0 < b1) {
    Block buf_a, buf_b, buf_c;
    prefetch_pages(b0);
    load_block(b0, buf_a);
    load_block(b0 + 1, buf_b);
    int kb = b0;
    for (; kb + 3 <= b1; kb += 3) {
      if (kb >= full_lo && kb + 2 <= full_hi) {
        load_block(kb + 2, buf_c);
        compute(kb, buf_a, Unmasked{});
        load_block(kb + 3, buf_a);
        compute(kb + 1, buf_b, Unmasked{});
        load_block(kb + 4, buf_b);
        compute(kb + 2, buf_c, Unmasked{});
      } else {
        load_block(kb + 2, buf_c);
        compute(kb, buf_a, Masked{});
        load_block(kb + 3, buf_a);
        compute(kb + 1, buf_b, Masked{});
        load_block(kb + 4, buf_b);
        compute(kb + 2, buf_c, Masked{});
      }
    }
    if (kb < b1) {
      compute(kb, buf_a, Masked{});
      if (kb + 1 < b1) compute(kb + 1, buf_b, Masked{});
    }
  }

  // ---- finish ---------------------------------------------------------------------------
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    float lt = l[n];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (!rvalid[n]) continue;
    if (num_splits == 1) {
      const float inv = 1.f / lt;
      bf16_t* op = out + ((size_t)tok[n] * Hq + head[n]) * HD;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint2 w;
        w.x = pack2bf(acc[dt][n][0] * inv, acc[dt][n][1] * inv);
        w.y = pack2bf(acc[dt][n][2] * inv, acc[dt][n][3] * inv);
        *reinterpret_cast<uint2*>(op + dt * 16 + 4 * g) = w;
      }
    } else {
      // LOCAL: the parts stay in the workgroup (part_o, part_ml lie in LDS), indexed [split][row of the tile]
      const size_t slot = LOCAL ? (size_t)sp * 16 + c : ((size_t)tok[n] * Hq + head[n]) * num_splits + sp;
      float* po = part_o + slot * HD;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<float4*>(po + dt * 16 + 4 * g) =
            make_float4(acc[dt][n][0], acc[dt][n][1], acc[dt][n][2], acc[dt][n][3]);
      if (g == 0) {
        part_ml[slot * 2] = m[n];
        part_ml[slot * 2 + 1] = lt;
      }
    }
  }
}

template <int PM>
__global__ __launch_bounds__(256) void paged_attention_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, int Hq, int Hk, int page_size, int page_shift, float scale_log2e,
    int window, int num_splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
  const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int hk = blockIdx.y;
  const int seg = blockIdx.z / num_splits;
  const int sp = blockIdx.z - seg * num_splits;
  const int q_begin = cu_q[seg];
  const int q_len = cu_q[seg + 1] - q_begin;
  attention_tile<PM>(w, seg, hk, sp, q_begin, q_len, q, q_stride, out, k_pages, v_pages, block_table, max_pages,
                     ctx_len, Hq, Hk, page_size, page_shift, scale_log2e, window, num_splits, part_o, part_ml);
}

// The same for short contexts: the WS waves of a workgroup take the WS parts of the key range of one
// (segment, KV head) and merge their (m, l, O) through LDS, in the order of the parts, so that no
// merge kernel follows: out = sum_s O_s 2^(m_s - M) / sum_s l_s 2^(m_s - M), an empty part weighs 0.
// Short contexts only: the keys and values of a (segment, KV head) then pass through one compute unit.
constexpr int WG_SPLITS = 4;

template <int PM>
__global__ __launch_bounds__(64 * WG_SPLITS) void paged_attention_mfma_wg_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, int Hq, int Hk, int page_size, int page_shift, float scale_log2e,
    int window) {
  __shared__ float part_o[WG_SPLITS * 16 * HD];
  __shared__ float part_ml[WG_SPLITS * 16 * 2];
  const int wave = threadIdx.x >> 6;
  const int hk = blockIdx.y;
  const int seg = blockIdx.z;
  const int q_begin = cu_q[seg];
  const int q_len = cu_q[seg + 1] - q_begin;
  attention_tile<PM, true>(0, seg, hk, wave, q_begin, q_len, q, q_stride, out, k_pages, v_pages, block_table,
                           max_pages, ctx_len, Hq, Hk, page_size, page_shift, scale_log2e, window, WG_SPLITS,
                           part_o, part_ml);
  __syncthreads();
  if (wave != 0) return;
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int G = Hq / Hk;
  if (c >= q_len * G) return;
  float ms[WG_SPLITS], M = -INFINITY;
#pragma unroll
  for (int s = 0; s < WG_SPLITS; ++s) {
    ms[s] = part_ml[(s * 16 + c) * 2];
    M = fmaxf(M, ms[s]);
  }
  float L = 0.f;
  floatx4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < WG_SPLITS; ++s) {
    const float w = ms[s] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms[s] - M);
    L += part_ml[(s * 16 + c) * 2 + 1] * w;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const float4 p = *reinterpret_cast<const float4*>(part_o + (s * 16 + c) * HD + dt * 16 + 4 * g);
      o[dt][0] += p.x * w;
      o[dt][1] += p.y * w;
      o[dt][2] += p.z * w;
      o[dt][3] += p.w * w;
    }
  }
  const float inv = 1.f / L;
  const int j = c / G;
  bf16_t* op = out + ((size_t)(q_begin + j) * Hq + hk * G + (c - j * G)) * HD;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    uint2 w;
    w.x = pack2bf(o[dt][0] * inv, o[dt][1] * inv);
    w.y = pack2bf(o[dt][2] * inv, o[dt][3] * inv);
    *reinterpret_cast<uint2*>(op + dt * 16 + 4 * g) = w;
  }
}

// ---------------------------------------------------------------------------------------------
// Prompt portions (more than 16 rows in a segment).  A workgroup of eight waves takes TW tiles of
// 32 rows, next to one another in the segment, and walks over the keys in stages of KW * KB blocks
// of 32 keys (TW * KW = 8).  All eight waves fetch a stage together, 16 bytes a thread at a time,
// into registers two stages ahead and from there into LDS one stage ahead (K and V^T have two
// buffers each: while stage i is multiplied from one, stage i + 1 is written to the other, which
// takes one barrier a stage; a second barrier, with the stage written just before it is read, cost
// 6 % of the time at head size 64 and 10 % at 128 over long contexts); then wave
// (tw, kw) multiplies tile tw with the kw-th run of KB blocks of the stage, reading K and V^T from
// LDS in the lane order of the matrix instruction, with one softmax update (maximum, rescaling of
// O) for the 32 * KB keys.  The KW waves of a tile hold partial (m, l, O), merged through LDS at
// the end.  K and V cross the chip's caches once per 32 * TW rows instead of once per wave.
//
// What the time goes to is the number of instructions a SIMD has to issue: measured on this chip,
// a SIMD whose two waves keep the vector unit busy gains little from matrix instructions of the
// other wave running beside them (288 vector + 32 matrix instructions: 429 ns + 229 ns apart,
// 589 ns together); exponentials, three and a half times as slow as plain vector instructions when
// alone, do run beside those.  Hence one softmax update per 64 or 128 keys (the stage's share of a wave), three-way maxima, row sums taken by the matrix cores, O
// rescaled only when a maximum has moved, and page addresses that are a constant plus a product.
//
// The work per stage is the same straight line of code for every wave and stage: a block that is
// partly or wholly invisible to the tile (the causal edge, the window's edge, beyond the tile's
// last key) has its scores masked under a branch that touches nothing else, and contributes
// p = 0.  A branch around the matrix products themselves would make the compiler copy O at every
// stage.
//
// LDS of a stage: K as [key][16-byte slot] with rows of 128 bytes (256 above head size 64), slot
// s of key row r stored at s ^ ((r & 3) | ((r >> 1) & 4)): the eight lanes that read together
// (c = 0..7 -> rows 0..3, 8..11 of a block, one slot) then fall into eight different 16-byte bank
// groups, and so do the eight threads that write one key's row.  V^T as [block][dim][4 runs of
// 8 keys], run g of dim d at g ^ ((d >> 1) & 3).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int log2_of(int x) { return x <= 1 ? 0 : 1 + log2_of(x / 2); }

template <int KW>
struct PromptShape {
  static constexpr int TW = 8 / KW;                        // tiles of 32 rows per workgroup
#ifndef PROMPT_KB_SMALL_HEADS
#define PROMPT_KB_SMALL_HEADS 4
#endif
#ifndef PROMPT_KB_BIG_HEADS
#define PROMPT_KB_BIG_HEADS 2
#endif
  // blocks of 32 keys per wave and stage
  static constexpr int KB = HD <= 64 ? (KW == 2 ? PROMPT_KB_SMALL_HEADS : 2) : (KW == 2 ? PROMPT_KB_BIG_HEADS : 1);
  static constexpr int BLOCKS = KW * KB;
  static constexpr int KEYS = 32 * BLOCKS;                 // keys per stage
  static constexpr int K_ROW = HD <= 64 ? 128 : 256;       // bytes of a key's row in LDS
  static constexpr int K_BYTES = KEYS * K_ROW;
  static constexpr int V_BYTES = BLOCKS * HD * 64;
  static constexpr int RING_BYTES = 2 * K_BYTES + 2 * V_BYTES;  // two buffers of K, two of V^T
  static constexpr int CHUNKS = 4 * BLOCKS * HD;           // 16-byte pieces of K, and of V, per stage
  static constexpr int PER_THREAD = (CHUNKS + 511) / 512;
  static constexpr int MERGE_FLOATS = DT * 8 + 4;          // per lane: O, m and l of two column tiles
  static constexpr int MERGE_BYTES = (KW - 1) * TW * MERGE_FLOATS * 64 * 4;   // the merge reuses the stages' memory
  static constexpr int LDS_BYTES = RING_BYTES > MERGE_BYTES ? RING_BYTES : MERGE_BYTES;
  static_assert(TW * KW == 8, "eight waves");
};

template <int KW, int PM>
__global__ __launch_bounds__(512) void prompt_attention_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, int Hq, int Hk, int page_size, int page_shift, float scale_log2e,
    int window, int num_splits, int pair, float* __restrict__ part_o, float* __restrict__ part_ml) {
  using S = PromptShape<KW>;
  constexpr int TW = S::TW, KB = S::KB, NT = 2, PT = S::PER_THREAD;
  constexpr int VL = PM == 0 ? 2 : 1;                      // loads per 16 bytes of V^T
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tw = wave % TW;
  const int kw = wave / TW;
  // neighbours in the grid take different KV heads: with eight of them each of the chip's eight
  // dies (workgroups are dealt to them in turn) reads one head's keys and values only
  const int hk = blockIdx.x % Hk;
  const int item = blockIdx.x / Hk;
  const int seg = blockIdx.y / num_splits;
  const int sp = blockIdx.y - seg * num_splits;
  const int q_begin = cu_q[seg];
  const int q_len = cu_q[seg + 1] - q_begin;
  const int G = Hq / Hk;
  const int rows_total = q_len * G;
  const int ngroups = (rows_total + 32 * TW - 1) / (32 * TW);
  if (item >= (pair ? (ngroups + 1) / 2 : ngroups)) return;
  const int ctx = ctx_len[seg];
  const int ctx_before = ctx - q_len;
  const int* bt = block_table + (size_t)seg * max_pages;
  const uint32_t page_bytes = (uint32_t)Hk * page_size * HD * 2;   // of a page of K, and of V (checked by the host)
  const int last_page = PM == 1 ? (ctx - 1) >> page_shift : (ctx - 1) / page_size;
  const char* k_base = reinterpret_cast<const char*>(k_pages);
  const char* v_base = reinterpret_cast<const char*>(v_pages);

  // ---- what this thread fetches of every stage ---------------------------------------------
  // With a power-of-two page size a stage begins at a multiple of its own length or of the page
  // size, so a key's place in its page is a constant of the thread plus (stage begin mod page):
  // k_off / v_off hold the constant, in bytes from the page's begin.  Keys beyond the context are
  // read from the last page, at their own place in it, and are never visible.
  int k_key[PT], k_seg[PT], k_off[PT], k_lds[PT], v_run[PT], v_dim[PT], v_off[PT], v_lds[PT];
  bool fetches[PT];
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int raw = tid + i * 512;
    fetches[i] = raw < S::CHUNKS;
    const int ch = min(raw, S::CHUNKS - 1);
    k_key[i] = ch / (HD / 8);
    k_seg[i] = ch - k_key[i] * (HD / 8);
    k_lds[i] = k_key[i] * S::K_ROW + ((k_seg[i] ^ ((k_key[i] & 3) | ((k_key[i] >> 1) & 4))) << 4);
    if (PM == 1) {
      // consecutive threads take consecutive 16 bytes of a page's [D, page_size] values: runs
      // of 8 keys along a dim, then the next dim
      const int rs = min(page_shift - 3, log2_of(4 * S::BLOCKS));   // a page's piece in the stage: 2^rs runs
      const int piece = (ch >> rs) / HD;
      const int within = ch - ((piece * HD) << rs);
      v_dim[i] = within >> rs;
      v_run[i] = (piece << rs) + (within & ((1 << rs) - 1));
      k_off[i] = (((hk * page_size + (k_key[i] & (page_size - 1))) * HD) + k_seg[i] * 8) * 2;
      v_off[i] = ((hk * HD + v_dim[i]) * page_size + ((v_run[i] * 8) & (page_size - 1))) * 2;
    } else {
      v_run[i] = ch / HD;
      v_dim[i] = ch - v_run[i] * HD;
      k_off[i] = v_off[i] = 0;
    }
    v_lds[i] = (((v_run[i] >> 2) * HD + v_dim[i]) * 4 + ((v_run[i] & 3) ^ ((v_dim[i] >> 1) & 3))) << 4;
  }
  // page ids of a stage's keys, and of its values, fetched one step before the keys and values are
  auto lookup_k = [&](int sb, int (&pk)[PT]) __attribute__((always_inline)) {
    const int key0 = sb * S::KEYS;
#pragma unroll
    for (int i = 0; i < PT; ++i)
      pk[i] = PM == 1 ? bt[min((key0 + k_key[i]) >> page_shift, last_page)] : bt[min((key0 + k_key[i]) / page_size, last_page)];
  };
  auto lookup_v = [&](int sb, int (&pv)[PT * VL]) __attribute__((always_inline)) {
    const int key0 = sb * S::KEYS;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      if (PM == 1) {
        pv[i] = bt[min((key0 + v_run[i] * 8) >> page_shift, last_page)];
      } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) pv[i * VL + h] = bt[min((key0 + v_run[i] * 8 + 4 * h) / page_size, last_page)];
      }
    }
  };
  // The loads carry no conditions: a stage beyond the last is read from the last page and never used.
  // With a power-of-two page size, (stage begin mod page) is 0 unless a page holds several stages.
  auto issue_k = [&](int sb, const int (&pk)[PT], u32x4_t (&r)[PT]) __attribute__((always_inline)) {
    const int key0 = sb * S::KEYS;
    if (PM == 1) {
      const char* kb = k_base + (size_t)(key0 & (page_size - 1)) * (HD * 2);
#pragma unroll
      for (int i = 0; i < PT; ++i)
        r[i] = *reinterpret_cast<const u32x4_t*>(kb + ((uint64_t)(uint32_t)max(pk[i], 0) * page_bytes + (uint32_t)k_off[i]));
    } else {
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const int off = (key0 + k_key[i]) % page_size;
        r[i] = *reinterpret_cast<const u32x4_t*>(k_base + (uint64_t)(uint32_t)max(pk[i], 0) * page_bytes +
                                                 ((size_t)(hk * page_size + off) * HD + k_seg[i] * 8) * 2);
      }
    }
  };
  auto issue_v = [&](int sb, const int (&pv)[PT * VL], u32x4_t (&r)[PT]) __attribute__((always_inline)) {
    const int key0 = sb * S::KEYS;
    if (PM == 1) {
      const char* vb = v_base + (size_t)(key0 & (page_size - 1)) * 2;
#pragma unroll
      for (int i = 0; i < PT; ++i)
        r[i] = *reinterpret_cast<const u32x4_t*>(vb + ((uint64_t)(uint32_t)max(pv[i], 0) * page_bytes + (uint32_t)v_off[i]));
    } else {
#pragma unroll
      for (int i = 0; i < PT; ++i) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int run = key0 + v_run[i] * 8 + 4 * h;
          const u32x2_t half = *reinterpret_cast<const u32x2_t*>(
              v_base + (uint64_t)(uint32_t)max(pv[i * VL + h], 0) * page_bytes +
              ((size_t)(hk * HD + v_dim[i]) * page_size + run % page_size) * 2);
          r[i][2 * h] = half[0];
          r[i][2 * h + 1] = half[1];
        }
      }
    }
  };
  // registers -> LDS: keys into K buffer `buf`, values into V buffer `buf`.  Values of keys at or
  // beyond the end of the context, and of keys before the window of the workgroup's first row (their
  // pages may have been given back), hold whatever the page held before: their probability is 0, and
  // 0 times such a value must stay 0, so they are zeroed.
  int lo_visible = 0;                                       // first key any row of the workgroup's group sees
  auto stash_k = [&](int buf, const u32x4_t (&r)[PT]) __attribute__((always_inline)) {
    unsigned char* st = smem + buf * S::K_BYTES;
#pragma unroll
    for (int i = 0; i < PT; ++i)
      if (S::CHUNKS % 512 == 0 || fetches[i]) *reinterpret_cast<u32x4_t*>(st + k_lds[i]) = r[i];
  };
  auto stash_v = [&](int sb, int buf, const u32x4_t (&r)[PT]) __attribute__((always_inline)) {
    unsigned char* st = smem + 2 * S::K_BYTES + buf * S::V_BYTES;
    const int key0 = sb * S::KEYS;
    const bool at_edge = key0 + S::KEYS > ctx || key0 < lo_visible;   // the same for every thread
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      u32x4_t v = r[i];
      if (at_edge) {
        const int first = key0 + v_run[i] * 8;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int k0 = first + 2 * e, k1 = k0 + 1;
          v[e] &= (k0 < ctx && k0 >= lo_visible ? 0x0000ffffu : 0u) | (k1 < ctx && k1 >= lo_visible ? 0xffff0000u : 0u);
        }
      }
      if (S::CHUNKS % 512 == 0 || fetches[i]) *reinterpret_cast<u32x4_t*>(st + v_lds[i]) = v;
    }
  };

  // ---- where this lane reads its operands in a stage ----------------------------------------
  const int krow = kw * KB * 32 + 8 * (c >> 2) + (c & 3);   // key row of tile 0 of the wave's first block
  const int kswz = c & 7;                                    // the row's slot mask: (r & 3) | ((r >> 1) & 4), all tiles
  const int ka0 = krow * S::K_ROW + ((g ^ kswz) << 4);       // dims 0..31 (and 64..95, 128 bytes on)
  const int ka1 = krow * S::K_ROW + (((4 + g) ^ kswz) << 4); // dims 32..63 (and 96..127)
  const int va = ((kw * KB * HD + c) * 4 + (g ^ ((c >> 1) & 3))) << 4;
  Frag ones;
  ones.u = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);   // bf16 1.0 throughout

  for (int pass = 0; pass < 2; ++pass) {
    // paired: group `item`, then its mirror image; alone: the groups with the most keys first
    const int group = (pass == 0) == (pair != 0) ? item : ngroups - 1 - item;
    if (pass == 1) {
      if (!pair || group <= item) break;
      __syncthreads();                                      // the first group's merge has been read
    }
    // the workgroup's range of stages, and this split's part of it
    const int r0g = group * (32 * TW);
    const int hi_key_g = ctx_before + min(rows_total - 1, r0g + 32 * TW - 1) / G;
    const int lo_key_g = window > 0 ? max(0, ctx_before + r0g / G - window + 1) : 0;
    lo_visible = lo_key_g;
    const int sb_lo = lo_key_g / S::KEYS;
    const int sb_hi = hi_key_g / S::KEYS;
    const int per = (sb_hi - sb_lo + num_splits) / num_splits;
    const int s0 = __builtin_amdgcn_readfirstlane(sb_lo + sp * per);
    const int nsb = __builtin_amdgcn_readfirstlane(max(0, min(sb_hi + 1, s0 + per) - s0));
    // this wave's tile (a tile beyond the segment's rows computes the last row over again and
    // writes nothing)
    const int r0 = r0g + tw * 32;
    const bool active = r0 < rows_total;
    const int j_lo = min(r0, rows_total - 1) / G;
    const int j_hi = min(rows_total - 1, r0 + 31) / G;
    // blocks full_lo .. full_hi are visible as a whole to every row of the tile
    const int full_hi = __builtin_amdgcn_readfirstlane((ctx_before + j_lo - 31) >> 5);
    const int full_lo = window > 0 ? __builtin_amdgcn_readfirstlane(((ctx_before + j_hi - window) >> 5) + 1) : 0;

    int qpos[NT], tok[NT], head[NT];
    bool rvalid[NT];
    Frag qf[NT][DC];
    float m[NT], m_raw[NT];
    floatx4_t lsum[NT];                                     // every element: the sum of p over all keys so far
    floatx4_t acc[DT][NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      const int row = r0 + n * 16 + c;
      rvalid[n] = row < rows_total;
      const int rowc = min(row, rows_total - 1);
      const int j = rowc / G;
      tok[n] = q_begin + j;
      head[n] = hk * G + (rowc - j * G);
      qpos[n] = ctx_before + j;
      const bf16_t* qp = q + (size_t)tok[n] * q_stride + (size_t)head[n] * HD;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) {
        qf[n][dc].u = make_uint4(0, 0, 0, 0);
        if (dc * 32 + g * 8 < HD) qf[n][dc].u = *reinterpret_cast<const uint4*>(qp + dc * 32 + g * 8);
      }
      m[n] = m_raw[n] = -INFINITY;
      lsum[n] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[dt][n] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
    }

    struct Scores {
      floatx4_t v[KB][2][NT];
    };
    // S^T = K Q^T for this wave's KB blocks of the stage in K buffer `buf`
    auto qk = [&](int buf, Scores& sc) __attribute__((always_inline)) {
      const unsigned char* st = smem + buf * S::K_BYTES;
      auto& s = sc.v;
#pragma unroll
      for (int h = 0; h < KB; ++h) {
        Frag kf[2][DC];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int dc = 0; dc < DC; ++dc) {
            kf[t][dc].u = *reinterpret_cast<const uint4*>(st + ((dc & 1) ? ka1 : ka0) + (h * 32 + t * 4) * S::K_ROW +
                                                          (dc >> 1) * 128);
            // dims beyond the head size were never written: they must read as 0, not as what LDS held
            if (HD % 32 != 0 && dc == DC - 1 && dc * 32 + g * 8 >= HD) kf[t][dc].u = make_uint4(0, 0, 0, 0);
          }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int n = 0; n < NT; ++n) {
            s[h][t][n] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dc = 0; dc < DC; ++dc)
              s[h][t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][dc].v, qf[n][dc].v, s[h][t][n], 0, 0, 0);
          }
      }
    };
    // blocks kb .. kb + KB - 1 of the keys: softmax update with their scores, O^T += V^T P^T with
    // the values in V buffer `buf`
    auto softmax_pv = [&](int kb, int buf, Scores& sc) __attribute__((always_inline)) {
      const unsigned char* st = smem + 2 * S::K_BYTES + buf * S::V_BYTES;
      auto& s = sc.v;
      // some key of these blocks is invisible to some row: the causal edge, the window's edge, a
      // block beyond the tile's last key
      if (kb < full_lo || kb + KB - 1 > full_hi) {
#pragma unroll
        for (int h = 0; h < KB; ++h)
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int n = 0; n < NT; ++n)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int key = ((kb + h) << 5) + 8 * g + 4 * t + r;
                const bool vis = key <= qpos[n] && (window <= 0 || key > qpos[n] - window);
                s[h][t][n][r] = vis ? s[h][t][n][r] : -INFINITY;
              }
      }
      // online softmax over this lane's 8 * KB keys per column, shared across the 4 lane groups.
      // The scale is positive, so the maximum is taken on the raw scores and the scale is applied
      // inside the exponent: p = 2^(s * scale - m).  Chains of dependent operations are kept short
      // (four running maxima; the row sums l come from the matrix cores, see below): a wave waits
      // several cycles for a result it has just asked for.
      Frag pf[KB][NT];
      float alpha[NT];
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        // two chains of three-way maxima over the lane's scores and the maximum so far (kept unscaled
        // in m_raw for this), then across the four lane groups
        float ma = fmaxf(fmaxf(m_raw[n], s[0][0][n][0]), s[0][0][n][1]);
        ma = fmaxf(fmaxf(ma, s[0][0][n][2]), s[0][0][n][3]);
        float mb = fmaxf(fmaxf(s[0][1][n][0], s[0][1][n][1]), s[0][1][n][2]);
#pragma unroll
        for (int h = 1; h < KB; ++h) {
          ma = fmaxf(fmaxf(ma, s[h][0][n][0]), s[h][0][n][1]);
          ma = fmaxf(fmaxf(ma, s[h][0][n][2]), s[h][0][n][3]);
          mb = fmaxf(fmaxf(mb, s[h][1][n][0]), s[h][1][n][1]);
          mb = fmaxf(fmaxf(mb, s[h][1][n][2]), s[h][1][n][3]);
        }
        m_raw[n] = max_across_groups(fmaxf(fmaxf(ma, mb), s[0][1][n][3]));
        const float m_new = m_raw[n] * scale_log2e;
        // a row that has seen no visible key yet keeps m = -inf
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        alpha[n] = __builtin_amdgcn_exp2f(m[n] - m_safe);
        m[n] = m_new;
#pragma unroll
        for (int h = 0; h < KB; ++h)
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) s[h][t][n][r] = fmaf(s[h][t][n][r], scale_log2e, -m_safe);
#pragma unroll
        for (int h = 0; h < KB; ++h)
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) s[h][t][n][r] = __builtin_amdgcn_exp2f(s[h][t][n][r]);
#pragma unroll
        for (int h = 0; h < KB; ++h)
          pf[h][n].u = make_uint4(pack2bf(s[h][0][n][0], s[h][0][n][1]), pack2bf(s[h][0][n][2], s[h][0][n][3]),
                                  pack2bf(s[h][1][n][0], s[h][1][n][1]), pack2bf(s[h][1][n][2], s[h][1][n][3]));
      }
      // the running maximum rarely moves after the first stages: O and l are rescaled only when it
      // has, for some row of the wave
      if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.f || alpha[1] != 1.f) != 0) {
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          lsum[n] *= alpha[n];
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) acc[dt][n] *= alpha[n];
        }
      }
      // O^T += V^T P^T, and l += 1^T P^T: a product with a tile of ones sums p over the keys of the
      // block (as it was rounded to bf16, which is what multiplies V), in every row of the result
#pragma unroll
      for (int h = 0; h < KB; ++h) {
#pragma unroll
        for (int n = 0; n < NT; ++n)
          lsum[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pf[h][n].v, lsum[n], 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          Frag vf;
          vf.u = *reinterpret_cast<const uint4*>(st + va + (h * HD + dt * 16) * 64);
#pragma unroll
          for (int n = 0; n < NT; ++n)
            acc[dt][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[h][n].v, acc[dt][n], 0, 0, 0);
        }
      }
    };

    if (nsb > 0) {
      // scores, softmax and the product with V of a stage in the same step: in step i, K(i) and V(i)
      // are read from LDS while K(i + 1) and V(i + 1) are written to the other buffers (one barrier a
      // step), and stage i + 2 is on its way into registers
      int pk[PT], pv[PT * VL];
      u32x4_t rk[PT], rv[PT];
      lookup_k(s0, pk);
      lookup_v(s0, pv);
      issue_k(s0, pk, rk);
      issue_v(s0, pv, rv);
      lookup_k(s0 + 1, pk);
      lookup_v(s0 + 1, pv);
      stash_k(0, rk);
      stash_v(s0, 0, rv);
      issue_k(s0 + 1, pk, rk);
      issue_v(s0 + 1, pv, rv);
      lookup_k(s0 + 2, pk);
      lookup_v(s0 + 2, pv);
      for (int i = 0; i < nsb; ++i) {
        const int b = i & 1;
        __syncthreads();
        stash_k(b ^ 1, rk);
        stash_v(s0 + i + 1, b ^ 1, rv);
        issue_k(s0 + i + 2, pk, rk);
        issue_v(s0 + i + 2, pv, rv);
        lookup_k(s0 + i + 3, pk);
        lookup_v(s0 + i + 3, pv);
        Scores sc;
        qk(b, sc);
        softmax_pv(((s0 + i) * KW + kw) * KB, b, sc);
      }
    }

    // ---- the KW waves of a tile merge through LDS, wave kw = 0 writes ---------------------------
    float lt[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) lt[n] = lsum[n][0];
    __syncthreads();                                        // every wave is done with the stages
    float* mg = reinterpret_cast<float*>(smem);
    if (kw > 0 && active) {
      float* mine = mg + (size_t)((kw - 1) * TW + tw) * S::MERGE_FLOATS * 64 + lane;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        mine[(n * 2) * 64] = m[n];
        mine[(n * 2 + 1) * 64] = lt[n];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) mine[(4 + (dt * NT + n) * 4 + r) * 64] = acc[dt][n][r];
      }
    }
    __syncthreads();
    if (kw > 0 || !active) continue;
#pragma unroll
    for (int o = 1; o < KW; ++o) {
      const float* other = mg + (size_t)((o - 1) * TW + tw) * S::MERGE_FLOATS * 64 + lane;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const float mo = other[(n * 2) * 64];
        const float lo = other[(n * 2 + 1) * 64];
        const float mm = fmaxf(m[n], mo);
        const float wa = m[n] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[n] - mm);   // an empty part weighs 0
        const float wb = mo == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mo - mm);
        m[n] = mm;
        lt[n] = lt[n] * wa + lo * wb;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            acc[dt][n][r] = acc[dt][n][r] * wa + other[(4 + (dt * NT + n) * 4 + r) * 64] * wb;
      }
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      if (!rvalid[n]) continue;
      if (num_splits == 1) {
        const float inv = 1.f / lt[n];
        bf16_t* op = out + ((size_t)tok[n] * Hq + head[n]) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          uint2 w;
          w.x = pack2bf(acc[dt][n][0] * inv, acc[dt][n][1] * inv);
          w.y = pack2bf(acc[dt][n][2] * inv, acc[dt][n][3] * inv);
          *reinterpret_cast<uint2*>(op + dt * 16 + 4 * g) = w;
        }
      } else {
        const size_t slot = ((size_t)tok[n] * Hq + head[n]) * num_splits + sp;
        float* po = part_o + slot * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          *reinterpret_cast<float4*>(po + dt * 16 + 4 * g) =
              make_float4(acc[dt][n][0], acc[dt][n][1], acc[dt][n][2], acc[dt][n][3]);
        if (g == 0) {
          part_ml[slot * 2] = m[n];
          part_ml[slot * 2 + 1] = lt[n];
        }
      }
    }
  }
}

template <int KW, int PM>
static int launch_prompt(dim3 grid, hipStream_t stream, const bf16_t* q, int q_stride, bf16_t* out,
                         const bf16_t* k_pages, const bf16_t* v_pages, const int* block_table, int max_pages,
                         const int* cu_q, const int* ctx_len, int Hq, int Hk, int page_size, int page_shift,
                         float scale_log2e, int window, int num_splits, int pair, float* part_o, float* part_ml) {
  constexpr int lds = PromptShape<KW>::LDS_BYTES;
  static bool sized = false;          // more than 64 KB of LDS has to be asked for, once per kernel
  if (!sized) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prompt_attention_kernel<KW, PM>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    sized = true;
  }
  hipLaunchKernelGGL((prompt_attention_kernel<KW, PM>), grid, dim3(512), lds, stream, q, q_stride, out, k_pages,
                     v_pages, block_table, max_pages, cu_q, ctx_len, Hq, Hk, page_size, page_shift, scale_log2e,
                     window, num_splits, pair, part_o, part_ml);
  return 0;
}

// out = sum_s O_s 2^(m_s - M) / sum_s l_s 2^(m_s - M), M = max_s m_s; at most 64 splits.
// One wave per (token, head): the lanes first share the work over the splits (weights), then over
// the head dims (weighted sum).  S: upper bound of the number of splits; the partial outputs are
// loaded (all at once, no conditions: a split beyond the last is read from the last and weighs 0)
// before the weights are known, so that the kernel costs one trip to memory and not two.
template <int S>
__global__ __launch_bounds__(64) void merge_splits_kernel(const float* __restrict__ part_o,
                                                          const float* __restrict__ part_ml,
                                                          bf16_t* __restrict__ out, int num_splits) {
  __shared__ float wgt[64];
  const size_t item = blockIdx.x;                 // token * Hq + head
  const int lane = threadIdx.x;
  constexpr int NA = (HD + 63) / 64;
  const float* po = part_o + item * num_splits * HD;
  float o[NA][S];
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int d = min(lane + a * 64, HD - 1);
#pragma unroll
    for (int s = 0; s < S; ++s) o[a][s] = po[(size_t)min(s, num_splits - 1) * HD + d];
  }
  float ms = -INFINITY, ls = 0.f;
  if (lane < num_splits) {
    ms = part_ml[(item * num_splits + lane) * 2];
    ls = part_ml[(item * num_splits + lane) * 2 + 1];
  }
  const float M = wave_max(ms);
  const float w = (ms == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ms - M);   // an empty split weighs 0
  const float L = wave_sum(ls * w);
  wgt[lane] = w;
  __syncthreads();
  const float inv = 1.f / L;
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int d = lane + a * 64;
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < S; ++s) sum += o[a][s] * wgt[s];
    if (d < HD) out[item * HD + d] = from_float<bf16_t>(sum * inv);
  }
}

extern "C" int sa_attention_mfma_head_dim() { return HD; }

// A step whose segments have at most 16 rows each (single decoded tokens) takes the one-wave kernel,
// any other the prompt kernel.  `in_workgroup` (such steps only, num_splits 1): the key range of every
// (segment, KV head) is cut four ways over the waves of one workgroup, which merges the parts itself.
extern "C" int sa_paged_attention_mfma(const void* q, int q_stride, void* out, const void* k_pages,
                                       const void* v_pages, const int* block_table, int max_pages,
                                       const int* cu_q, const int* ctx_len, int B, int T, int max_q_len,
                                       int Hq, int Hk, int D, int page_size, float scale, int window,
                                       int num_splits, float* part_o, float* part_ml, int in_workgroup,
                                       hipStream_t stream) {
  if (T <= 0 || B <= 0) return 0;
  if (D != HD || Hq <= 0 || Hk <= 0 || Hq % Hk || page_size <= 0 || (page_size & 3) || max_pages <= 0 ||
      max_q_len <= 0 || num_splits < 1 || num_splits > 64 || (q_stride & 7))
    return SA_ERR_ARG;
  if (num_splits > 1 && (!part_o || !part_ml)) return SA_ERR_ARG;
  if ((long long)B * num_splits > 65535 || Hk > 65535) return SA_ERR_ARG;
  const int G = Hq / Hk;
  const bool small = (long long)max_q_len * G <= 16;
  const float scale_log2e = scale * 1.4426950408889634f;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  if (in_workgroup && (!small || num_splits != 1 || B > 65535)) return SA_ERR_ARG;
  if (small && in_workgroup) {
    // the key range cut four ways inside a workgroup and merged there: for short contexts
    dim3 grid(1, Hk, B), block(64 * WG_SPLITS);
    const int pm = page_shift >= 5 ? 2 : (page_shift >= 3 ? 1 : 0);
#define GO(PM)                                                                                         \
  hipLaunchKernelGGL((paged_attention_mfma_wg_kernel<PM>), grid, block, 0, stream,                     \
                     (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages,                 \
                     (const bf16_t*)v_pages, block_table, max_pages, cu_q, ctx_len, Hq, Hk, page_size, \
                     page_shift, scale_log2e, window)
    if (pm == 2) GO(2);
    else if (pm == 1) GO(1);
    else GO(0);
#undef GO
    SA_LAUNCH_CHECK();
    return 0;
  }
  if (small) {
    // single decoded tokens (at most 16 rows per KV head): one wave per (segment, KV head, split)
    dim3 grid(1, Hk, B * num_splits), block(64);   // one wave: tile 0 is the only tile of such a segment
    const int pm = page_shift >= 5 ? 2 : (page_shift >= 3 ? 1 : 0);
#define GO(PM)                                                                                         \
  hipLaunchKernelGGL((paged_attention_mfma_kernel<PM>), grid, block, 0, stream,                        \
                     (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages,                 \
                     (const bf16_t*)v_pages, block_table, max_pages, cu_q, ctx_len, Hq, Hk, page_size, \
                     page_shift, scale_log2e, window, num_splits, part_o, part_ml)
    if (pm == 2) GO(2);
    else if (pm == 1) GO(1);
    else GO(0);
#undef GO
  } else {
    // prompt portions: 128 rows per workgroup and two waves along the keys, or 64 rows and four
    // when no segment has more rows than that.  Where that still leaves more workgroups than
    // compute units, a workgroup takes row groups w and last - w: under the causal mask the two
    // together are one full context long, so all finish at about the same time.
    const long long rows = (long long)max_q_len * G;
    const int kw = rows > 64 ? 2 : 4;
    const long long groups = (rows + 256 / kw - 1) / (256 / kw);
    const int pair = num_splits == 1 && (groups + 1) / 2 * Hk * B >= compute_units();
    const long long items = pair ? (groups + 1) / 2 : groups;
    if (items * Hk > 0x7fffffffLL || (long long)Hk * page_size * HD * 2 > 0x7fffffffLL) return SA_ERR_ARG;
    dim3 grid((unsigned)(items * Hk), B * num_splits);
    const int pm = page_shift >= 3 ? 1 : 0;
    int rc;
#define GO(KW, PM)                                                                                       \
  rc = launch_prompt<KW, PM>(grid, stream, (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages, \
                             (const bf16_t*)v_pages, block_table, max_pages, cu_q, ctx_len, Hq, Hk, page_size, \
                             page_shift, scale_log2e, window, num_splits, pair, part_o, part_ml)
    if (kw == 2 && pm == 1) GO(2, 1);
    else if (kw == 2) GO(2, 0);
    else if (pm == 1) GO(4, 1);
    else GO(4, 0);
#undef GO
    if (rc != 0) return rc;
  }
  SA_LAUNCH_CHECK();
  if (num_splits > 1) {
#define MERGE(S)                                                                                      \
  hipLaunchKernelGGL(merge_splits_kernel<S>, dim3((unsigned)T * Hq), dim3(64), 0, stream, part_o, part_ml, \
                     (bf16_t*)out, num_splits)
    if (num_splits <= 4) MERGE(4);
    else if (num_splits <= 8) MERGE(8);
    else if (num_splits <= 16) MERGE(16);
    else if (num_splits <= 32) MERGE(32);
    else MERGE(64);
#undef MERGE
    SA_LAUNCH_CHECK();
  }
  return 0;
}
