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
// Work item of one wave: (segment, KV head, tile of 16*NT "rows", split of the key range).  The
// rows of a segment are its (token, query head of the group) pairs, row = token * G + head_in_group,
// so the G heads that share a KV head share every K and V load.
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

// NT: column tiles (16 query rows each) per wave.  PM: how keys map to pages:
//   0  any page size that is a multiple of 4: division per key, 8-byte value runs;
//   1  a power of two of at least 8: shift, 16-byte value runs; a block of 32 keys spans up to four
//      pages and each lane picks its own;
//   2  a power of two of at least 32: a block lies in one page, and every address is a scalar base
//      plus a constant of the lane.
// One tile of one (segment, KV head, split): everything a wave does.
template <int NT, int PM>
__device__ __forceinline__ void attention_tile(
    const int tile, const int seg, const int hk, const int sp, const int q_begin, const int q_len,
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ ctx_len, int Hq, int Hk,
    int page_size, int page_shift, float scale_log2e, int window, int num_splits,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
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
      // keys at or beyond the end of the context hold whatever the page held before: their
      // probability is 0, and 0 times such a value must stay 0
      const int first = key0 + 8 * g;
      uint32_t keep[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        keep[i] = (first + 2 * i < ctx ? 0x0000ffffu : 0u) | (first + 2 * i + 1 < ctx ? 0xffff0000u : 0u);
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

  // Three buffers in turn: the loads of the next two blocks are in flight while one is computed
  // (two buffers, one block in flight, for prompt tiles of head sizes above 64, whose blocks are
  // twice as large and would push the registers over the edge).
  // The loads carry no conditions: a block beyond the last is read from clamped keys and pages and
  // never used.  With a branch around them the compiler no longer knows how many loads are in
  // flight where a block's data is awaited, and waits for all of them, the newest included.
  if (b0 < b1 && HD > 64 && NT > 1) {
    Block buf_a, buf_b;
    prefetch_pages(b0);
    load_block(b0, buf_a);
    int kb = b0;
    for (; kb + 2 <= b1; kb += 2) {
      if (kb >= full_lo && kb + 1 <= full_hi) {
        load_block(kb + 1, buf_b);
        compute(kb, buf_a, Unmasked{});
        load_block(kb + 2, buf_a);
        compute(kb + 1, buf_b, Unmasked{});
      } else {
        load_block(kb + 1, buf_b);
        compute(kb, buf_a, Masked{});
        load_block(kb + 2, buf_a);
        compute(kb + 1, buf_b, Masked{});
      }
    }
    if (kb < b1) compute(kb, buf_a, Masked{});
  } else if (b0 < b1) {
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
      const size_t slot = ((size_t)tok[n] * Hq + head[n]) * num_splits + sp;
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

// A wave takes tile w of its (segment, KV head).  With PAIR it takes tile ntiles-1-w as well: under
// the causal mask tile t reads keys up to about t's end, so the two together are always one full
// context long and all waves of a prompt finish at about the same time.
template <int NT, int PM, bool PAIR>
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
  if (!PAIR) {
    attention_tile<NT, PM>(w, seg, hk, sp, q_begin, q_len, q, q_stride, out, k_pages, v_pages, block_table,
                             max_pages, ctx_len, Hq, Hk, page_size, page_shift, scale_log2e, window, num_splits,
                             part_o, part_ml);
    return;
  }
  const int ntiles = (q_len * (Hq / Hk) + 16 * NT - 1) / (16 * NT);
  if (w >= (ntiles + 1) / 2) return;                                  // the second half is done by pairing
  attention_tile<NT, PM>(w, seg, hk, sp, q_begin, q_len, q, q_stride, out, k_pages, v_pages, block_table,
                           max_pages, ctx_len, Hq, Hk, page_size, page_shift, scale_log2e, window, num_splits,
                           part_o, part_ml);
  const int other = ntiles - 1 - w;
  if (other > w)
    attention_tile<NT, PM>(other, seg, hk, sp, q_begin, q_len, q, q_stride, out, k_pages, v_pages, block_table,
                             max_pages, ctx_len, Hq, Hk, page_size, page_shift, scale_log2e, window, num_splits,
                             part_o, part_ml);
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

// Tiles of 16*nt rows per wave: nt = 1 when a segment has at most 16 rows (decode steps).  Prompt
// portions take the largest tile the registers hold (fewest reads of K and V) when that still gives
// every SIMD of the chip a wave, and 32 rows otherwise.
#if HEAD_DIM <= 64
#define NT_PREFILL 4
#else
#define NT_PREFILL 2
#endif
constexpr int WAVES_TO_FILL = 1024;     // 256 compute units x 4 SIMDs

extern "C" int sa_paged_attention_mfma(const void* q, int q_stride, void* out, const void* k_pages,
                                       const void* v_pages, const int* block_table, int max_pages,
                                       const int* cu_q, const int* ctx_len, int B, int T, int max_q_len,
                                       int Hq, int Hk, int D, int page_size, float scale, int window,
                                       int num_splits, float* part_o, float* part_ml, hipStream_t stream) {
  if (T <= 0 || B <= 0) return 0;
  if (D != HD || Hq <= 0 || Hk <= 0 || Hq % Hk || page_size <= 0 || (page_size & 3) || max_pages <= 0 ||
      max_q_len <= 0 || num_splits < 1 || num_splits > 64 || (q_stride & 7))
    return SA_ERR_ARG;
  if (num_splits > 1 && (!part_o || !part_ml)) return SA_ERR_ARG;
  if ((long long)B * num_splits > 65535 || Hk > 65535) return SA_ERR_ARG;
  const int G = Hq / Hk;
  const bool small = (long long)max_q_len * G <= 16;
  // prompt portions: a wave takes tiles w and tiles-1-w, so half as many waves are launched
  const bool pair = !small && num_splits == 1;
  int nt = small ? 1 : NT_PREFILL;
  auto waves_for = [&](int n) {
    const long long tiles = ((long long)max_q_len * G + 16 * n - 1) / (16 * n);
    return pair ? (tiles + 1) / 2 : tiles;
  };
  if (nt > 2 && waves_for(nt) * Hk * B < WAVES_TO_FILL) nt = 2;
  const int waves = (int)waves_for(nt);
  dim3 grid((waves + 3) / 4, Hk, B * num_splits), block(256);
  const float scale_log2e = scale * 1.4426950408889634f;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
#define GO(NT, PM, PAIR)                                                                               \
  hipLaunchKernelGGL((paged_attention_mfma_kernel<NT, PM, PAIR>), grid, block, 0, stream,              \
                     (const bf16_t*)q, q_stride, (bf16_t*)out, (const bf16_t*)k_pages,                 \
                     (const bf16_t*)v_pages, block_table, max_pages, cu_q, ctx_len, Hq, Hk, page_size, \
                     page_shift, scale_log2e, window, num_splits, part_o, part_ml)
  const int pm = page_shift >= 5 ? 2 : (page_shift >= 3 ? 1 : 0);
#define GO3(NT, PAIR)           \
  do {                          \
    if (pm == 2) GO(NT, 2, PAIR);      \
    else if (pm == 1) GO(NT, 1, PAIR); \
    else GO(NT, 0, PAIR);              \
  } while (0)
  if (small) GO3(1, false);
  else if (nt == 2 && pair) GO3(2, true);
  else if (nt == 2) GO3(2, false);
#if NT_PREFILL > 2
  else if (pair) GO3(NT_PREFILL, true);
  else GO3(NT_PREFILL, false);
#endif
#undef GO3
#undef GO
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
