// Paged attention in fp32 arithmetic: one wave per (token, query head) (below), and for prompt
// portions of the float32 path a kernel that shares keys and values across 64 rows (further down).
//
// The first is the general form: any head_dim up to 256, any head counts, any page size, any mix of
// prompt portions and single tokens in one launch.  Formulas as in serve/kernels/attn_prefill.py:56-72,205 and attn_decode.py:99-111,236:
// scores = q.k * scale, key j visible to the query at absolute position p iff j <= p (and
// p - j < window when a window is set), online softmax (m, l, O), O / l at the end.  Query head
// h reads KV head h / (Hq / Hk).
//
// Batch layout: the T tokens of a step are the concatenation of B segments; segment r covers
// tokens cu_q[r] .. cu_q[r+1]-1, which are the last q_len positions of a context of ctx_len[r]
// tokens.  block_table[r, i] is the page of keys i*page_size .. (i+1)*page_size-1.
// k pages [page, Hk, page_size, D]; v pages [page, Hk, D, page_size].
#include "common.h"

#define SA_MAX_D 256

template <typename TA, typename TC>
__global__ __launch_bounds__(64) void paged_attention_simple_kernel(
    const TA* __restrict__ q, int q_stride, TA* __restrict__ out, const TC* __restrict__ k_pages,
    const TC* __restrict__ v_pages, const int* __restrict__ block_table, int max_pages,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ seg_of_token,
    int Hq, int Hk, int D, int page_size, float scale, int window, int t0) {
  __shared__ float qs[SA_MAX_D];
  __shared__ float ps[SA_WAVE];
  __shared__ int vbase_page[SA_WAVE];
  __shared__ int vbase_off[SA_WAVE];

  const int t = t0 + blockIdx.y;
  const int h = blockIdx.x;
  const int lane = threadIdx.x;
  const int r = seg_of_token[t];
  const int q_len = cu_q[r + 1] - cu_q[r];
  const int qpos = ctx_len[r] - q_len + (t - cu_q[r]);
  const int g = h / (Hq / Hk);
  const int* bt = block_table + (size_t)r * max_pages;

  const TA* qrow = q + (size_t)t * q_stride + (size_t)h * D;
  for (int i = lane; i < D; i += SA_WAVE) qs[i] = to_float(qrow[i]);
  __syncthreads();

  int lo = 0;
  if (window > 0 && qpos - window + 1 > 0) lo = qpos - window + 1;
  const int hi = qpos;  // inclusive

  float m = -INFINITY, l = 0.f;
  float acc[SA_MAX_D / SA_WAVE];
#pragma unroll
  for (int a = 0; a < SA_MAX_D / SA_WAVE; ++a) acc[a] = 0.f;

  for (int base = lo; base <= hi; base += SA_WAVE) {
    const int kpos = base + lane;
    const bool valid = kpos <= hi;
    float s = -INFINITY;
    int page = 0, off = 0;
    if (valid) {
      page = bt[kpos / page_size];
      off = kpos % page_size;
      const TC* kp = k_pages + (((size_t)page * Hk + g) * page_size + off) * D;
      float dot = 0.f;
      for (int i = 0; i < D; ++i) dot = fmaf(qs[i], to_float(kp[i]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));   // lane 0 is always valid, so m_new is finite
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);         // exp(-inf) = 0 on the first chunk
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int a = 0; a < SA_MAX_D / SA_WAVE; ++a) acc[a] *= alpha;
    ps[lane] = p;
    vbase_page[lane] = page;
    vbase_off[lane] = off;
    __syncthreads();
    const int n = min(SA_WAVE, hi - base + 1);
    for (int j = 0; j < n; ++j) {
      const float pj = ps[j];
      const TC* vp = v_pages + ((size_t)vbase_page[j] * Hk + g) * (size_t)D * page_size + vbase_off[j];
#pragma unroll
      for (int a = 0; a < SA_MAX_D / SA_WAVE; ++a) {
        const int i = lane + a * SA_WAVE;
        if (i < D) acc[a] = fmaf(pj, to_float(vp[(size_t)i * page_size]), acc[a]);
      }
    }
    __syncthreads();
  }
  const float inv_l = 1.f / l;
  TA* orow = out + (size_t)t * Hq * D + (size_t)h * D;
#pragma unroll
  for (int a = 0; a < SA_MAX_D / SA_WAVE; ++a) {
    const int i = lane + a * SA_WAVE;
    if (i < D) orow[i] = from_float<TA>(acc[a] * inv_l);
  }
}

// ---------------------------------------------------------------------------------------------
// The same attention for prompt portions of the float32 path, tiled: a workgroup of 256 threads
// takes 64 rows (a row = a token of the segment and one of the G query heads of a KV head, so the
// rows of a workgroup share every key and value) and walks over the keys in blocks of 64 that are
// staged in LDS, where the kernel above fetches every key once per row.  fp32 throughout, on the
// vector ALU: thread (tr, tc) of the 16 x 16 grid owns rows 4 tr .. 4 tr + 3; of a block's scores
// it computes keys tc, tc + 16, tc + 32, tc + 48, of the output dims tc, tc + 16, ...; row maxima
// and sums are taken across the 16 lanes of a row group.  Online softmax as above.
// Needs D % 16 == 0, D <= 128 and a page size that is a multiple of 4 (four consecutive keys then
// lie in one page, and their values, stored transposed, are one 16-byte load).
// ---------------------------------------------------------------------------------------------
#define TL_ROWS 64
#define TL_KEYS 64

template <int DV>   // D / 16
__global__ __launch_bounds__(256) void paged_attention_tiled_f32_kernel(
    const float* __restrict__ q, int q_stride, float* __restrict__ out, const float* __restrict__ k_pages,
    const float* __restrict__ v_pages, const int* __restrict__ block_table, int max_pages,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, int Hq, int Hk, int page_size, float scale,
    int window, int num_splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int D = DV * 16;
  constexpr int LD = D + 4;                       // row length in LDS: keeps 16-byte alignment, spreads banks
  extern __shared__ __attribute__((aligned(16))) float tl_smem[];
  float* Qs = tl_smem;                            // [64][LD]
  float* Ks = Qs + TL_ROWS * LD;                  // [64][LD]
  float* Vs = Ks + TL_KEYS * LD;                  // [64][LD]
  float* Ps = Vs + TL_KEYS * LD;                  // [64][68]
  constexpr int LP = TL_KEYS + 4;

  const int tid = threadIdx.x;
  const int tr = tid >> 4, tc = tid & 15;
  const int g = blockIdx.x % Hk;                  // KV head
  const int item = blockIdx.x / Hk;               // tile of 64 rows within the segment
  const int seg = blockIdx.y / num_splits;
  const int sp = blockIdx.y - seg * num_splits;   // this workgroup's part of the key range
  const int G = Hq / Hk;
  const int q_begin = cu_q[seg];
  const int q_len = cu_q[seg + 1] - q_begin;
  const int rows_total = q_len * G;
  const int r0 = item * TL_ROWS;
  if (r0 >= rows_total) return;
  const int ctx = ctx_len[seg];
  const int ctx_before = ctx - q_len;
  const int* bt = block_table + (size_t)seg * max_pages;

  // the tile's queries
  for (int i = tid; i < TL_ROWS * (D / 4); i += 256) {
    const int r = i / (D / 4), c4 = i - r * (D / 4);
    const int row = min(r0 + r, rows_total - 1);
    const int j = row / G, gi = row - j * G;
    *reinterpret_cast<float4*>(Qs + r * LD + c4 * 4) =
        *reinterpret_cast<const float4*>(q + (size_t)(q_begin + j) * q_stride + (size_t)(g * G + gi) * D + c4 * 4);
  }
  int qpos[4];
  bool rvalid[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = r0 + tr * 4 + r;
    rvalid[r] = row < rows_total;
    qpos[r] = ctx_before + min(row, rows_total - 1) / G;
  }
  const int hi = ctx_before + min(r0 + TL_ROWS - 1, rows_total - 1) / G;          // last key any row of the tile sees
  const int lo = window > 0 ? max(0, ctx_before + r0 / G - window + 1) : 0;      // first key any row sees

  float m[4], l[4], acc[4][DV];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int e = 0; e < DV; ++e) acc[r][e] = 0.f;
  }
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

  // the blocks of 64 keys that the tile sees, cut evenly into num_splits parts
  const int b_lo = lo / TL_KEYS, b_hi = hi / TL_KEYS;
  const int per = (b_hi - b_lo + num_splits) / num_splits;
  const int b_first = b_lo + sp * per;
  const int b_last = min(b_hi, b_first + per - 1);
  __syncthreads();                                // Qs is written (a part may have no block at all)
  for (int kb = b_first * TL_KEYS; kb <= b_last * TL_KEYS; kb += TL_KEYS) {
    __syncthreads();                              // the block before has been used
    // keys: 64 rows of D floats, 16 bytes a thread at a time
    for (int i = tid; i < TL_KEYS * (D / 4); i += 256) {
      const int key = i / (D / 4), c4 = i - key * (D / 4);
      const int kpos = kb + key;
      float4 v = zero4;
      if (kpos >= lo && kpos <= hi) {
        const int page = bt[kpos / page_size];
        const int off = kpos % page_size;
        v = *reinterpret_cast<const float4*>(k_pages + (((size_t)page * Hk + g) * page_size + off) * D + c4 * 4);
      }
      *reinterpret_cast<float4*>(Ks + key * LD + c4 * 4) = v;
    }
    // values: stored [D][page_size] in a page; four consecutive keys of a dim are one load
    for (int i = tid; i < (TL_KEYS / 4) * D; i += 256) {
      const int d = i / (TL_KEYS / 4), quad = i - d * (TL_KEYS / 4);
      const int kpos = kb + quad * 4;
      float4 v = zero4;
      if (kpos + 3 >= lo && kpos <= hi) {
        const int page = bt[kpos / page_size];
        const int off = kpos % page_size;
        v = *reinterpret_cast<const float4*>(v_pages + (((size_t)page * Hk + g) * D + d) * page_size + off);
        // a value beyond what any row sees may be anything (a page that holds another request's data,
        // or none): its weight is 0, and 0 times it must be 0
        if (kpos < lo || kpos > hi) v.x = 0.f;
        if (kpos + 1 < lo || kpos + 1 > hi) v.y = 0.f;
        if (kpos + 2 < lo || kpos + 2 > hi) v.z = 0.f;
        if (kpos + 3 < lo || kpos + 3 > hi) v.w = 0.f;
      }
      Vs[(quad * 4 + 0) * LD + d] = v.x;
      Vs[(quad * 4 + 1) * LD + d] = v.y;
      Vs[(quad * 4 + 2) * LD + d] = v.z;
      Vs[(quad * 4 + 3) * LD + d] = v.w;
    }
    __syncthreads();
    // scores of rows 4 tr .. + 3 with keys tc + 16 c
    float s[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int c = 0; c < 4; ++c) s[r][c] = 0.f;
    for (int d4 = 0; d4 < D / 4; ++d4) {
      float4 qv[4], kv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) qv[r] = *reinterpret_cast<const float4*>(Qs + (tr * 4 + r) * LD + d4 * 4);
#pragma unroll
      for (int c = 0; c < 4; ++c) kv[c] = *reinterpret_cast<const float4*>(Ks + (tc + 16 * c) * LD + d4 * 4);
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float t = s[r][c];
          t = fmaf(qv[r].x, kv[c].x, t);
          t = fmaf(qv[r].y, kv[c].y, t);
          t = fmaf(qv[r].z, kv[c].z, t);
          t = fmaf(qv[r].w, kv[c].w, t);
          s[r][c] = t;
        }
    }
    // mask, row maxima and sums across the 16 lanes of the row group, p into LDS
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float mx = -INFINITY;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int key = kb + tc + 16 * c;
        const bool vis = key <= qpos[r] && (window <= 0 || key > qpos[r] - window);
        s[r][c] = vis ? s[r][c] * scale : -INFINITY;
        mx = fmaxf(mx, s[r][c]);
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, SA_WAVE));
      const float m_new = fmaxf(m[r], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;      // a row that has seen no key yet
      const float alpha = expf(m[r] - m_safe);                    // exp(-inf) = 0 at the first visible block
      float sum = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float p = expf(s[r][c] - m_safe);                   // exp(-inf) = 0 for invisible keys
        Ps[(tr * 4 + r) * LP + tc + 16 * c] = p;
        sum += p;
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, SA_WAVE);
      l[r] = l[r] * alpha + sum;
      m[r] = m_new;
#pragma unroll
      for (int e = 0; e < DV; ++e) acc[r][e] *= alpha;
    }
    __syncthreads();
    // O += P V: dims tc + 16 e
    for (int j4 = 0; j4 < TL_KEYS / 4; ++j4) {
      float4 pv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) pv[r] = *reinterpret_cast<const float4*>(Ps + (tr * 4 + r) * LP + j4 * 4);
#pragma unroll
      for (int e = 0; e < DV; ++e) {
        const float v0 = Vs[(j4 * 4 + 0) * LD + tc + 16 * e];
        const float v1 = Vs[(j4 * 4 + 1) * LD + tc + 16 * e];
        const float v2 = Vs[(j4 * 4 + 2) * LD + tc + 16 * e];
        const float v3 = Vs[(j4 * 4 + 3) * LD + tc + 16 * e];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float t = acc[r][e];
          t = fmaf(pv[r].x, v0, t);
          t = fmaf(pv[r].y, v1, t);
          t = fmaf(pv[r].z, v2, t);
          t = fmaf(pv[r].w, v3, t);
          acc[r][e] = t;
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (!rvalid[r]) continue;
    const int row = r0 + tr * 4 + r;
    const int j = row / G, gi = row - j * G;
    const size_t orow_index = (size_t)(q_begin + j) * Hq + (g * G + gi);        // (token, head)
    if (num_splits > 1) {
      // unnormalised sums with their maximum and weight: merged by paged_attention_merge_f32_kernel
      float* po = part_o + (orow_index * num_splits + sp) * D;
#pragma unroll
      for (int e = 0; e < DV; ++e) po[tc + 16 * e] = acc[r][e];
      if (tc == 0) {
        part_ml[(orow_index * num_splits + sp) * 2] = m[r];
        part_ml[(orow_index * num_splits + sp) * 2 + 1] = l[r];
      }
      continue;
    }
    const float inv_l = 1.f / l[r];
    float* orow = out + orow_index * D;
#pragma unroll
    for (int e = 0; e < DV; ++e) orow[tc + 16 * e] = acc[r][e] * inv_l;
  }
}

// out[row] = sum_s w_s O_s / sum_s w_s l_s with w_s = exp(m_s - max m): the parts of a split key
// range (a part that saw no key has m = -inf and weight 0; at most 64 parts).  One wave per row: the
// lanes first share the parts (weights), then the head dims (weighted sums, whose loads do not wait
// for one another).
__global__ __launch_bounds__(64) void paged_attention_merge_f32_kernel(const float* __restrict__ part_o,
                                                                       const float* __restrict__ part_ml,
                                                                       float* __restrict__ out, int D, int num_splits) {
  __shared__ float wgt[64];
  const size_t row = blockIdx.x;
  const int lane = threadIdx.x;
  float ms = -INFINITY, ls = 0.f;
  if (lane < num_splits) {
    ms = part_ml[(row * num_splits + lane) * 2];
    ls = part_ml[(row * num_splits + lane) * 2 + 1];
  }
  const float mx = wave_max(ms);
  const float w = ms == -INFINITY ? 0.f : expf(ms - mx);
  const float inv = 1.f / wave_sum(w * ls);
  wgt[lane] = w;
  __syncthreads();
  const float* po = part_o + row * num_splits * D;
  for (int d = lane; d < D; d += 64) {
    float o = 0.f;
#pragma unroll 8
    for (int s = 0; s < num_splits; ++s) o = fmaf(wgt[s], po[(size_t)s * D + d], o);
    out[row * D + d] = o * inv;
  }
}

template <int DV>
static int launch_tiled(const void* q, int q_stride, void* out, const void* k_pages, const void* v_pages,
                        const int* block_table, int max_pages, const int* cu_q, const int* ctx_len, int B,
                        int max_q_len, int Hq, int Hk, int page_size, float scale, int window, int num_splits,
                        float* part_o, float* part_ml, hipStream_t stream) {
  constexpr int D = DV * 16;
  const size_t lds = (size_t)(3 * 64 * (D + 4) + 64 * 68) * sizeof(float);
  const long long items = ((long long)max_q_len * (Hq / Hk) + TL_ROWS - 1) / TL_ROWS;
  if (items * Hk > 0x7fffffffLL || (long long)B * num_splits > 65535) return SA_ERR_ARG;
  hipError_t e = hipFuncSetAttribute((const void*)paged_attention_tiled_f32_kernel<DV>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return (int)e;
  dim3 grid((unsigned)(items * Hk), B * num_splits), block(256);
  hipLaunchKernelGGL((paged_attention_tiled_f32_kernel<DV>), grid, block, lds, stream, (const float*)q, q_stride,
                     (float*)out, (const float*)k_pages, (const float*)v_pages, block_table, max_pages, cu_q,
                     ctx_len, Hq, Hk, page_size, scale, window, num_splits, part_o, part_ml);
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Single tokens of the float32 path over long contexts: every segment brings one token, so the rows
// that share a KV head's keys and values are only its G query heads, and the tiled kernel above
// would do the arithmetic of 64 rows for them.  Here one wave takes GR query heads of one KV head
// of one segment and one part of the key range, in blocks of 64 keys:
//   scores: four lanes per key, each with a quarter of the dims (the four lanes of a key read 64
//   contiguous bytes at a time), partial sums added across the four lanes;
//   softmax: online, maxima and sums across the wave, p of the block through LDS;
//   values: a lane per dim (V is stored [D, page_size]: the lanes of a wave read whole runs of a
//   page), four keys a load, O += p v for the GR heads.
// Every key and value is read once per GR heads instead of once per head.  Parts as in the kernels
// above: part_o [T Hq num_splits, D], part_ml [T Hq num_splits, 2], merged by
// paged_attention_merge_f32_kernel.  Needs D % 16 == 0, D <= 128, page_size % 4 == 0.
// ---------------------------------------------------------------------------------------------
template <int DV, int GR>   // D / 16; query heads per wave
__global__ __launch_bounds__(64) void paged_attention_decode_f32_kernel(
    const float* __restrict__ q, int q_stride, float* __restrict__ out, const float* __restrict__ k_pages,
    const float* __restrict__ v_pages, const int* __restrict__ block_table, int max_pages,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, int Hq, int Hk, int page_size, float scale,
    int window, int num_splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int D = DV * 16;
  constexpr int NA = (D + 63) / 64;               // dims per lane in the product with V
  __shared__ __attribute__((aligned(16))) float ps[GR][64];
  const int lane = threadIdx.x;
  const int kk = lane >> 2, part = lane & 3;      // key of a group of 16, quarter of the dims
  const int G = Hq / Hk;
  const int chunks = (G + GR - 1) / GR;
  const int g = blockIdx.x / chunks;              // KV head
  const int h0 = (blockIdx.x - g * chunks) * GR;  // first of this wave's query heads within the group
  const int seg = blockIdx.y;
  const int sp = blockIdx.z;
  const int t = cu_q[seg];                        // the segment's one token
  const int qpos = ctx_len[seg] - 1;
  const int* bt = block_table + (size_t)seg * max_pages;
  const int lo = window > 0 ? max(0, qpos - window + 1) : 0;
  const int hi = qpos;

  // this lane's quarter of the queries (a head beyond the group repeats the last and is not written)
  float4 qv[GR][DV];
#pragma unroll
  for (int r = 0; r < GR; ++r) {
    const int h = g * G + min(h0 + r, G - 1);
    const float* qp = q + (size_t)t * q_stride + (size_t)h * D;
#pragma unroll
    for (int e = 0; e < DV; ++e) {
      const float4 v = *reinterpret_cast<const float4*>(qp + (part + 4 * e) * 4);
      qv[r][e] = make_float4(v.x * scale, v.y * scale, v.z * scale, v.w * scale);
    }
  }
  float m[GR], l[GR], acc[GR][NA];
#pragma unroll
  for (int r = 0; r < GR; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int a = 0; a < NA; ++a) acc[r][a] = 0.f;
  }

  // the blocks of 64 keys that the token sees, cut evenly into num_splits parts
  const int b_lo = lo >> 6, b_hi = hi >> 6;
  const int per = (b_hi - b_lo + num_splits) / num_splits;
  const int b_first = b_lo + sp * per;
  const int b_last = min(b_hi, b_first + per - 1);
  for (int kb = b_first * 64; kb <= b_last * 64; kb += 64) {
    // scores: keys kb + 16 i + kk.  A key outside the range is read at the range's nearest key (the
    // pages before a window may have been given back) and masked.
    float s[GR][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kpos = min(max(kb + 16 * i + kk, lo), hi);
      const int page = bt[kpos / page_size];
      const float* kp = k_pages + (((size_t)page * Hk + g) * page_size + kpos % page_size) * D;
      float4 kv[DV];
#pragma unroll
      for (int e = 0; e < DV; ++e) kv[e] = *reinterpret_cast<const float4*>(kp + (part + 4 * e) * 4);
#pragma unroll
      for (int r = 0; r < GR; ++r) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < DV; ++e) {
          d = fmaf(qv[r][e].x, kv[e].x, d);
          d = fmaf(qv[r][e].y, kv[e].y, d);
          d = fmaf(qv[r][e].z, kv[e].z, d);
          d = fmaf(qv[r][e].w, kv[e].w, d);
        }
        d += __shfl_xor(d, 1, SA_WAVE);
        d += __shfl_xor(d, 2, SA_WAVE);
        const int key = kb + 16 * i + kk;
        s[r][i] = key >= lo && key <= hi ? d : -INFINITY;
      }
    }
    __syncthreads();                              // the block before has been multiplied
#pragma unroll
    for (int r = 0; r < GR; ++r) {
      const float mx = wave_max(fmaxf(fmaxf(s[r][0], s[r][1]), fmaxf(s[r][2], s[r][3])));
      const float m_new = fmaxf(m[r], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;      // a part that has seen no key yet
      const float alpha = expf(m[r] - m_safe);
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = expf(s[r][i] - m_safe);                  // exp(-inf) = 0 for invisible keys
        if (part == 0) {
          ps[r][16 * i + kk] = pr;
          sum += pr;
        }
      }
      l[r] = l[r] * alpha + wave_sum(sum);
      m[r] = m_new;
#pragma unroll
      for (int a = 0; a < NA; ++a) acc[r][a] *= alpha;
    }
    __syncthreads();
    // values: four keys of a dim are one load (they lie in one page, at a multiple of four)
    const bool edge = kb < lo || kb + 63 > hi;
#pragma unroll 4
    for (int j4 = 0; j4 < 16; ++j4) {
      const int kq = kb + 4 * j4;
      // (four keys outside the range are read from the page of its nearest key, at their own place in it)
      const int page = bt[min(max(kq, lo), hi) / page_size];
      float4 pv[GR];
#pragma unroll
      for (int r = 0; r < GR; ++r) pv[r] = *reinterpret_cast<const float4*>(&ps[r][4 * j4]);
#pragma unroll
      for (int a = 0; a < NA; ++a) {
        const int d = min(lane + 64 * a, D - 1);
        float4 v = *reinterpret_cast<const float4*>(v_pages + (((size_t)page * Hk + g) * D + d) * page_size +
                                                    kq % page_size);
        if (edge) {
          // a value that the token does not see may be anything: its weight is 0, and 0 times it must be 0
          if (kq < lo || kq > hi) v.x = 0.f;
          if (kq + 1 < lo || kq + 1 > hi) v.y = 0.f;
          if (kq + 2 < lo || kq + 2 > hi) v.z = 0.f;
          if (kq + 3 < lo || kq + 3 > hi) v.w = 0.f;
        }
#pragma unroll
        for (int r = 0; r < GR; ++r) {
          float o = acc[r][a];
          o = fmaf(pv[r].x, v.x, o);
          o = fmaf(pv[r].y, v.y, o);
          o = fmaf(pv[r].z, v.z, o);
          o = fmaf(pv[r].w, v.w, o);
          acc[r][a] = o;
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < GR; ++r) {
    if (h0 + r >= G) continue;
    const size_t row = (size_t)t * Hq + g * G + h0 + r;           // (token, head)
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      const int d = lane + 64 * a;
      if (d >= D) continue;
      if (num_splits > 1) part_o[(row * num_splits + sp) * D + d] = acc[r][a];
      else out[row * D + d] = acc[r][a] / l[r];
    }
    if (num_splits > 1 && lane == 0) {
      part_ml[(row * num_splits + sp) * 2] = m[r];
      part_ml[(row * num_splits + sp) * 2 + 1] = l[r];
    }
  }
}

template <int DV>
static int launch_decode_f32(const void* q, int q_stride, void* out, const void* k_pages, const void* v_pages,
                             const int* block_table, int max_pages, const int* cu_q, const int* ctx_len, int B,
                             int Hq, int Hk, int page_size, float scale, int window, int num_splits, float* part_o,
                             float* part_ml, hipStream_t stream) {
  const int G = Hq / Hk;
  const int gr = G >= 3 ? 4 : G;                  // heads per wave: 1, 2 or 4
  const long long gx = (long long)Hk * ((G + gr - 1) / gr);
  if (gx > 0x7fffffffLL || B > 65535 || num_splits > 65535) return SA_ERR_ARG;
  dim3 grid((unsigned)gx, B, num_splits), block(64);
#define GO(GR)                                                                                                    \
  hipLaunchKernelGGL((paged_attention_decode_f32_kernel<DV, GR>), grid, block, 0, stream, (const float*)q,        \
                     q_stride, (float*)out, (const float*)k_pages, (const float*)v_pages, block_table, max_pages, \
                     cu_q, ctx_len, Hq, Hk, page_size, scale, window, num_splits, part_o, part_ml)
  if (gr == 1) GO(1);
  else if (gr == 2) GO(2);
  else GO(4);
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}

// float32 attention of B segments of one token each (token r is the last of a context of ctx_len[r]
// tokens) over their cached keys.  D a multiple of 16 up to 128, page_size a multiple of 4.
// The segments are a run of the step's tokens: segment i is token first_token + i (cu_q[i] must say
// so; the host knows it and the kernels do not check it), which is the row of q, out and the parts it
// uses.  num_splits > 1 cuts every key range into that many parts over the grid; part_o
// [(first_token + B) Hq num_splits, D] and part_ml [(first_token + B) Hq num_splits, 2] (fp32) then
// take the parts, which a second kernel merges for the rows first_token .. first_token + B - 1.
extern "C" int sa_paged_attention_decode_f32(const void* q, int q_stride, void* out, const void* k_pages,
                                             const void* v_pages, const int* block_table, int max_pages,
                                             const int* cu_q, const int* ctx_len, int B, int first_token, int Hq,
                                             int Hk, int D, int page_size, float scale, int window, int num_splits,
                                             float* part_o, float* part_ml, hipStream_t stream) {
  if (B <= 0) return 0;
  if (Hq <= 0 || Hk <= 0 || Hq % Hk || D <= 0 || D > 128 || (D & 15) || page_size <= 0 || (page_size & 3) ||
      max_pages <= 0 || (q_stride & 3) || num_splits < 1 || num_splits > 64 || first_token < 0)
    return SA_ERR_ARG;
  if (num_splits > 1 && (!part_o || !part_ml)) return SA_ERR_ARG;
  int rc = SA_ERR_ARG;
#define GO(DV)                                                                                                   \
  case DV:                                                                                                       \
    rc = launch_decode_f32<DV>(q, q_stride, out, k_pages, v_pages, block_table, max_pages, cu_q, ctx_len, B, Hq, \
                               Hk, page_size, scale, window, num_splits, part_o, part_ml, stream);               \
    break
  switch (D / 16) {
    GO(1);
    GO(2);
    GO(3);
    GO(4);
    GO(5);
    GO(6);
    GO(7);
    GO(8);
  }
#undef GO
  if (rc != 0 || num_splits == 1) return rc;
  const size_t row0 = (size_t)first_token * Hq;
  hipLaunchKernelGGL(paged_attention_merge_f32_kernel, dim3((unsigned)B * Hq), dim3(64), 0, stream,
                     part_o + row0 * num_splits * D, part_ml + row0 * num_splits * 2, (float*)out + row0 * D, D,
                     num_splits);
  SA_LAUNCH_CHECK();
  return 0;
}

// float32 attention of every token of the B segments (T tokens) over their cached keys, 64 rows a
// workgroup.  D a multiple of 16 up to 128, page_size a multiple of 4; max_q_len: the longest
// segment.  num_splits > 1 cuts every tile's key range into that many parts over the grid; part_o
// [T Hq num_splits, D] and part_ml [T Hq num_splits, 2] (fp32) then take the parts, which a second
// kernel merges.
extern "C" int sa_paged_attention_tiled_f32(const void* q, int q_stride, void* out, const void* k_pages,
                                            const void* v_pages, const int* block_table, int max_pages,
                                            const int* cu_q, const int* ctx_len, int B, int T, int max_q_len,
                                            int Hq, int Hk, int D, int page_size, float scale, int window,
                                            int num_splits, float* part_o, float* part_ml, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0 || T <= 0) return 0;
  if (Hq <= 0 || Hk <= 0 || Hq % Hk || D <= 0 || D > 128 || (D & 15) || page_size <= 0 || (page_size & 3) ||
      max_pages <= 0 || (q_stride & 3) || num_splits < 1 || num_splits > 64)
    return SA_ERR_ARG;
  if (num_splits > 1 && (!part_o || !part_ml)) return SA_ERR_ARG;
  int rc = SA_ERR_ARG;
#define GO(DV)                                                                                                  \
  case DV:                                                                                                      \
    rc = launch_tiled<DV>(q, q_stride, out, k_pages, v_pages, block_table, max_pages, cu_q, ctx_len, B,         \
                          max_q_len, Hq, Hk, page_size, scale, window, num_splits, part_o, part_ml, stream);    \
    break
  switch (D / 16) {
    GO(1);
    GO(2);
    GO(3);
    GO(4);
    GO(5);
    GO(6);
    GO(7);
    GO(8);
  }
#undef GO
  if (rc != 0 || num_splits == 1) return rc;
  hipLaunchKernelGGL(paged_attention_merge_f32_kernel, dim3((unsigned)T * Hq), dim3(64), 0, stream, part_o, part_ml,
                     (float*)out, D, num_splits);
  SA_LAUNCH_CHECK();
  return 0;
}

extern "C" int sa_paged_attention_simple(const void* q, int q_stride, void* out, int act_dtype,
                                         const void* k_pages, const void* v_pages, int cache_dtype,
                                         const int* block_table, int max_pages, const int* cu_q,
                                         const int* ctx_len, const int* seg_of_token, int T, int Hq,
                                         int Hk, int D, int page_size, float scale, int window,
                                         hipStream_t stream) {
  if (T <= 0) return 0;
  if (Hq <= 0 || Hk <= 0 || Hq % Hk || D <= 0 || D > SA_MAX_D || page_size <= 0 || max_pages <= 0)
    return SA_ERR_ARG;
  if (T > 65535 * 16) return SA_ERR_ARG;
  // grid.y is limited to 65535: long steps are launched in slices of tokens
  const int slice = 32768;
  for (int t0 = 0; t0 < T; t0 += slice) {
    const int n = T - t0 < slice ? T - t0 : slice;
    dim3 grid(Hq, n), block(SA_WAVE);
#define GO(TA, TC)                                                                                   \
  hipLaunchKernelGGL((paged_attention_simple_kernel<TA, TC>), grid, block, 0, stream,                \
                     (const TA*)q, q_stride, (TA*)out, (const TC*)k_pages, (const TC*)v_pages,       \
                     block_table, max_pages, cu_q, ctx_len, seg_of_token, Hq, Hk, D, page_size,     \
                     scale, window, t0)
    if (act_dtype == SA_F32 && cache_dtype == SA_F32) GO(float, float);
    else if (act_dtype == SA_BF16 && cache_dtype == SA_BF16) GO(bf16_t, bf16_t);
    else return SA_ERR_UNSUPPORTED;
#undef GO
    SA_LAUNCH_CHECK();
  }
  return 0;
}
