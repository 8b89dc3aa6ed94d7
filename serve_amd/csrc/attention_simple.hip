// Paged attention, one wave per (token, query head), fp32 arithmetic throughout.
//
// This is the attention of the float32 path and the fallback-free general form: any head_dim up
// to 256, any head counts, any page size, any mix of prompt portions and single tokens in one
// launch.  Formulas as in serve/kernels/attn_prefill.py:56-72,205 and attn_decode.py:99-111,236:
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
