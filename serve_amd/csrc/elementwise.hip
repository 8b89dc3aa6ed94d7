// Row-wise kernels of the step: embedding gather, residual add + RMSNorm, rotation of q and k
// with the write of k and v into cache pages, and the SwiGLU gate.  All arithmetic is fp32;
// the template types are storage only.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// embedding: x[t, :] = table[tokens[t], :]   (serve/model.py:220), residual stream in fp32
// ---------------------------------------------------------------------------------------------
// A token id comes from `tokens[t]`, or, when src_row[t] >= 0, from prev[src_row[t]]: the token
// that an earlier step sampled on the device and that the host has not read back yet.
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ tokens,
                             const int* __restrict__ src_row, const int* __restrict__ prev,
                             float* __restrict__ x, int d, int V) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  if (src_row && src_row[t] >= 0) tok = prev[src_row[t]];
  tok = min(max(tok, 0), V - 1);
  const size_t row = (size_t)tok * (size_t)d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) x[(size_t)t * d + i] = to_float(table[row + i]);
}

// bf16 rows of whole groups of eight from aligned addresses: 16 bytes a lane in, two times 16 out
__global__ __launch_bounds__(256) void embed_bf16x8_kernel(const bf16_t* __restrict__ table, const int* __restrict__ tokens,
                                                            const int* __restrict__ src_row, const int* __restrict__ prev,
                                                            float* __restrict__ x, int d, int V) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  if (src_row && src_row[t] >= 0) tok = prev[src_row[t]];
  tok = min(max(tok, 0), V - 1);
  const bf16_t* row = table + (size_t)tok * (size_t)d;
  float* out = x + (size_t)t * d;
  for (int i = threadIdx.x * 8; i < d; i += blockDim.x * 8) {
    const uint4 v = *reinterpret_cast<const uint4*>(row + i);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      f[2 * k] = bf16_bits_to_float(w[k] & 0xffffu);
      f[2 * k + 1] = bf16_bits_to_float(w[k] >> 16);
    }
    *reinterpret_cast<float4*>(out + i) = make_float4(f[0], f[1], f[2], f[3]);
    *reinterpret_cast<float4*>(out + i + 4) = make_float4(f[4], f[5], f[6], f[7]);
  }
}

extern "C" int sa_embed(const void* table, int table_dtype, const int* tokens, const int* src_row,
                        const int* prev, float* x, int T, int d, int V, hipStream_t stream) {
  if (T <= 0) return 0;
  if (d <= 0 || V <= 0 || (src_row && !prev)) return SA_ERR_ARG;
  dim3 grid(T), block(256);
  if (table_dtype == SA_BF16 && (d & 7) == 0 && ((uintptr_t)table & 15) == 0 && ((uintptr_t)x & 15) == 0) {
    hipLaunchKernelGGL(embed_bf16x8_kernel, grid, block, 0, stream, (const bf16_t*)table, tokens, src_row, prev, x,
                       d, V);
    SA_LAUNCH_CHECK();
    return 0;
  }
  if (table_dtype == SA_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (const float*)table, tokens, src_row, prev,
                       x, d, V);
  else if (table_dtype == SA_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, tokens, src_row, prev,
                       x, d, V);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// residual add + RMSNorm (serve/model.py:63-68,147-148):
//   v = x[t] + delta[t];  x[t] = v (only when rows == nullptr);  y[r] = v * rsqrt(mean(v^2) + eps) * w
// rows != nullptr: output row r takes source row rows[r] and x is left untouched.
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TD, typename TW>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int parts,
                                   size_t part_stride, const TW* __restrict__ w, TA* __restrict__ y,
                                   const int* __restrict__ rows, float eps, int d) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int t = rows ? rows[r] : r;
  float* xr = x + (size_t)t * d;
  const TD* dr = delta ? delta + (size_t)t * d : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      for (int p = 0; p < parts; ++p) v += to_float(dr[p * part_stride + i]);
      if (!rows) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rs = rsqrtf(ss / (float)d + eps);
  TA* yr = y + (size_t)r * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = xr[i];
    if (dr && rows)
      for (int p = 0; p < parts; ++p) v += to_float(dr[p * part_stride + i]);
    yr[i] = from_float<TA>((v * rs) * to_float(w[i]));
  }
}

// The same in one pass for d % 4 == 0 and d <= 8192: a thread keeps its (up to 8) groups of four
// values in registers between the sum of squares and the scaling, and moves 16-byte vectors.
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_bits_to_float(u.x & 0xffffu), bf16_bits_to_float(u.x >> 16),
                     bf16_bits_to_float(u.y & 0xffffu), bf16_bits_to_float(u.y >> 16));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16);
  u.y = (uint32_t)float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// PMAX: upper bound of `parts` (1, 4 or 8).  All loads of a thread are issued before anything is
// added, without conditions around them: a group beyond the row and a part beyond `parts` are read
// from a clamped address and dropped, so that a row costs one trip to memory and not one per part.
template <typename TA, typename TD, typename TW, int PMAX>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                                              int parts, size_t part_stride,
                                                              const TW* __restrict__ w, TA* __restrict__ y,
                                                              const int* __restrict__ rows, float eps, int d) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int t = rows ? rows[r] : r;
  float* xr = x + (size_t)t * d;
  const TD* dr = delta ? delta + (size_t)t * d : nullptr;
  const int groups = d >> 2;
  const int nk = (groups + 255) >> 8;            // rounds of 256 groups, at most 8
  float4 v[8], wv[8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    if (k < nk) {
      const int gi = threadIdx.x + k * 256;
      const int i = min(gi, groups - 1) * 4;
      v[k] = load4(xr + i);
      wv[k] = load4(w + i);
      if (dr) {
        float4 a[PMAX];
#pragma unroll
        for (int p = 0; p < PMAX; ++p) a[p] = load4(dr + (size_t)min(p, parts - 1) * part_stride + i);
#pragma unroll
        for (int p = 0; p < PMAX; ++p) {
          const float on = p < parts ? 1.f : 0.f;
          v[k].x += on * a[p].x; v[k].y += on * a[p].y; v[k].z += on * a[p].z; v[k].w += on * a[p].w;
        }
      }
      const float in = gi < groups ? 1.f : 0.f;
      ss += in * (v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w);
    }
  }
  ss = block_sum(ss, scratch);
  const float rs = rsqrtf(ss / (float)d + eps);
  TA* yr = y + (size_t)r * d;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int gi = threadIdx.x + k * 256;
    const int i = gi * 4;
    if (k < nk && gi < groups) {
      if (dr && !rows) store4(xr + i, v[k]);
      store4(yr + i, make_float4((v[k].x * rs) * wv[k].x, (v[k].y * rs) * wv[k].y,
                                 (v[k].z * rs) * wv[k].z, (v[k].w * rs) * wv[k].w));
    }
  }
}

// delta: [T, d] in the activation dtype (delta_dtype == act_dtype, parts == 1), or fp32
// [parts, T, d] partial sums that are added in order.
extern "C" int sa_add_rmsnorm(float* x, const void* delta, int delta_dtype, int parts, const void* w,
                              int w_dtype, void* y, int act_dtype, const int* rows, float eps, int R,
                              int T, int d, hipStream_t stream) {
  if (R <= 0) return 0;
  if (d <= 0 || parts < 1) return SA_ERR_ARG;
  if (delta && delta_dtype != act_dtype && delta_dtype != SA_F32) return SA_ERR_UNSUPPORTED;
  if (delta && parts > 1 && delta_dtype != SA_F32) return SA_ERR_UNSUPPORTED;
  const size_t part_stride = (size_t)T * d;
  const bool vec = (d & 3) == 0 && d <= 8192 && d >= 256;
  dim3 grid(R), block(vec || d >= 1024 ? 256 : 64);
#define GO(TA, TD, TW)                                                                                   \
  do {                                                                                                   \
    if (vec && parts == 1)                                                                               \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TA, TD, TW, 1>), grid, block, 0, stream, x,             \
                         (const TD*)delta, parts, part_stride, (const TW*)w, (TA*)y, rows, eps, d);      \
    else if (vec && parts <= 4)                                                                          \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TA, TD, TW, 4>), grid, block, 0, stream, x,             \
                         (const TD*)delta, parts, part_stride, (const TW*)w, (TA*)y, rows, eps, d);      \
    else if (vec && parts <= 8)                                                                          \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TA, TD, TW, 8>), grid, block, 0, stream, x,             \
                         (const TD*)delta, parts, part_stride, (const TW*)w, (TA*)y, rows, eps, d);      \
    else                                                                                                 \
      hipLaunchKernelGGL((add_rmsnorm_kernel<TA, TD, TW>), grid, block, 0, stream, x, (const TD*)delta,  \
                         parts, part_stride, (const TW*)w, (TA*)y, rows, eps, d);                        \
  } while (0)
  const bool dfloat = delta && delta_dtype == SA_F32;
  if (act_dtype == SA_F32 && w_dtype == SA_F32) GO(float, float, float);
  else if (act_dtype == SA_F32 && w_dtype == SA_BF16) GO(float, float, bf16_t);
  else if (act_dtype == SA_BF16 && w_dtype == SA_F32) { if (dfloat) GO(bf16_t, float, float); else GO(bf16_t, bf16_t, float); }
  else if (act_dtype == SA_BF16 && w_dtype == SA_BF16) { if (dfloat) GO(bf16_t, float, bf16_t); else GO(bf16_t, bf16_t, bf16_t); }
  else return SA_ERR_UNSUPPORTED;
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// rotation of q and k (serve/model.py:234-244) fused with the cache write
// (serve/kernels/cache_write.py:49-165).
//   qkv: [T, (Hq + 2 Hk) D]; q is rotated in place, rotated k and plain v go to the pages.
//   angle = float(position) * inv_freq[j] in fp32, pair j = (j, j + rot/2) ("half") or
//   (2j, 2j + 1) ("adjacent"); dims >= rot_dim pass through.
//   k page layout [page, Hk, page_size, D]; v page layout [page, Hk, D, page_size].
//   slot[t] = page * page_size + offset of token t, or < 0 for "do not store".
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TC>
__global__ void rope_kv_write_kernel(TA* __restrict__ qkv, const int* __restrict__ positions,
                                     const float* __restrict__ inv_freq, const int* __restrict__ slot,
                                     TC* __restrict__ k_pages, TC* __restrict__ v_pages, int Hq, int Hk,
                                     int D, int rot_dim, int adjacent, int page_size, int write_kv) {
  const int t = blockIdx.x;
  TA* row = qkv + (size_t)t * (size_t)(Hq + 2 * Hk) * D;
  const float pos = (float)positions[t];
  const int s = write_kv ? slot[t] : -1;
  const int page = s >= 0 ? s / page_size : 0;
  const int off = s >= 0 ? s % page_size : 0;
  const int half = rot_dim / 2;

  // rotated pairs of q heads and k heads
  const int npairs = (Hq + Hk) * half;
  for (int idx = threadIdx.x; idx < npairs; idx += blockDim.x) {
    const int h = idx / half;
    const int j = idx - h * half;
    const int i0 = adjacent ? 2 * j : j;
    const int i1 = adjacent ? 2 * j + 1 : j + half;
    float sn, cs;
    if (sizeof(TA) == 2) sincos_reduced(pos * inv_freq[j], &sn, &cs);   // bf16 keeps 8 bits of it
    else sincosf(pos * inv_freq[j], &sn, &cs);
    TA* hp = row + (size_t)h * D;
    const float a = to_float(hp[i0]);
    const float b = to_float(hp[i1]);
    const float o0 = a * cs - b * sn;
    const float o1 = b * cs + a * sn;
    if (h < Hq) {
      hp[i0] = from_float<TA>(o0);
      hp[i1] = from_float<TA>(o1);
    } else if (s >= 0) {
      TC* kp = k_pages + (((size_t)page * Hk + (h - Hq)) * page_size + off) * D;
      kp[i0] = from_float<TC>(o0);
      kp[i1] = from_float<TC>(o1);
    }
  }
  if (s < 0) return;
  // k dims that are not rotated
  const int rest = D - rot_dim;
  for (int idx = threadIdx.x; idx < Hk * rest; idx += blockDim.x) {
    const int h = idx / rest;
    const int i = rot_dim + (idx - h * rest);
    TC* kp = k_pages + (((size_t)page * Hk + h) * page_size + off) * D;
    kp[i] = from_float<TC>(to_float(row[(size_t)(Hq + h) * D + i]));
  }
  // v, stored transposed inside the page
  for (int idx = threadIdx.x; idx < Hk * D; idx += blockDim.x) {
    const int h = idx / D;
    const int i = idx - h * D;
    TC* vp = v_pages + (((size_t)page * Hk + h) * D + i) * page_size + off;
    *vp = from_float<TC>(to_float(row[(size_t)(Hq + Hk + h) * D + i]));
  }
}

// The same for bf16 with (j, j + D/2) pairs over the whole head (rot_dim == D, D % 16 == 0), 16-byte
// vectors, `tpb` (1, 2, 4 or 8) consecutive tokens per block.  A thread takes eight pairs of one head of
// one token (two loads, two stores).  The values go through LDS: they are read as rows of tokens and written
// so that neighbouring lanes hold neighbouring tokens of one dim, which in the transposed page
// ([Hk, D, page_size]) are neighbouring addresses when the tokens' slots are (a prompt portion's
// are): the two-byte stores of eight lanes then fill one 16-byte run instead of eight memory lines.
// The kernel is bound by the latency of its loads, so the host picks tokens per block and threads
// per block for many loads in flight: few tokens per block when the step has few tokens.
__global__ __launch_bounds__(1024) void rope_kv_write_bf16_vec_kernel(
    bf16_t* __restrict__ qkv, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    const int* __restrict__ slot, bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, int T, int Hq, int Hk,
    int D, int page_size, int write_kv, int tpb) {
  extern __shared__ __attribute__((aligned(16))) unsigned char rope_lds[];
  const int t0 = blockIdx.x * tpb;
  const int nt = min(tpb, T - t0);
  const size_t row_len = (size_t)(Hq + (write_kv ? 2 * Hk : 0)) * D;
  const int half = D >> 1;
  const int gph = half >> 3;                                  // groups of eight pairs per head
  const int Hr = Hq + (write_kv ? Hk : 0);
  const int per_token = Hr * gph;
  for (int idx = threadIdx.x; idx < nt * per_token; idx += blockDim.x) {
    const int i = idx / per_token;
    const int rem = idx - i * per_token;
    const int h = rem / gph;
    const int j0 = (rem - h * gph) * 8;
    const int t = t0 + i;
    const float pos = (float)positions[t];
    bf16_t* hp = qkv + (size_t)t * row_len + (size_t)h * D;
    const uint4 lo = *reinterpret_cast<const uint4*>(hp + j0);
    const uint4 hi = *reinterpret_cast<const uint4*>(hp + half + j0);
    const float4 f0 = *reinterpret_cast<const float4*>(inv_freq + j0);
    const float4 f1 = *reinterpret_cast<const float4*>(inv_freq + j0 + 4);
    const float fr[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
    const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w}, hw[4] = {hi.x, hi.y, hi.z, hi.w};
    uint32_t ol[4], oh[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float o0[2], o1[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float a = bf16_bits_to_float(e ? lw[k] >> 16 : lw[k] & 0xffffu);
        const float b = bf16_bits_to_float(e ? hw[k] >> 16 : hw[k] & 0xffffu);
        float sn, cs;
        sincos_reduced(pos * fr[2 * k + e], &sn, &cs);
        o0[e] = a * cs - b * sn;
        o1[e] = b * cs + a * sn;
      }
      ol[k] = (uint32_t)float_to_bf16_bits(o0[0]) | ((uint32_t)float_to_bf16_bits(o0[1]) << 16);
      oh[k] = (uint32_t)float_to_bf16_bits(o1[0]) | ((uint32_t)float_to_bf16_bits(o1[1]) << 16);
    }
    bf16_t* dst = hp;
    if (h >= Hq) {
      const int s = slot[t];
      if (s < 0) continue;
      const int page = s / page_size;
      dst = k_pages + (((size_t)page * Hk + (h - Hq)) * page_size + (s - page * page_size)) * D;
    }
    *reinterpret_cast<uint4*>(dst + j0) = make_uint4(ol[0], ol[1], ol[2], ol[3]);
    *reinterpret_cast<uint4*>(dst + half + j0) = make_uint4(oh[0], oh[1], oh[2], oh[3]);
  }
  if (!write_kv) return;
  // values: rows of tokens into LDS (16 bytes of padding per row spread the tokens over the banks) ...
  const int HD = Hk * D;
  const int stride = HD + 8;                                  // elements
  uint16_t* tile = reinterpret_cast<uint16_t*>(rope_lds);
  const int vecs = HD >> 3;
  for (int idx = threadIdx.x; idx < nt * vecs; idx += blockDim.x) {
    const int i = idx / vecs;
    const int e0 = (idx - i * vecs) * 8;
    *reinterpret_cast<uint4*>(tile + i * stride + e0) =
        *reinterpret_cast<const uint4*>(qkv + (size_t)(t0 + i) * row_len + (size_t)(Hq + Hk) * D + e0);
  }
  __syncthreads();
  // ... and out again with the token as the fastest index
  const int i = threadIdx.x & (tpb - 1);
  const int s = i < nt ? slot[t0 + i] : -1;
  if (s < 0) return;
  const int page = s / page_size;
  bf16_t* vp = v_pages + (size_t)page * HD * page_size + (s - page * page_size);
  for (int e = threadIdx.x / tpb; e < HD; e += blockDim.x / tpb)
    vp[(size_t)e * page_size].v = tile[i * stride + e];
}

extern "C" int sa_rope_kv_write(void* qkv, int act_dtype, const int* positions, const float* inv_freq,
                                const int* slot, void* k_pages, void* v_pages, int cache_dtype, int T,
                                int Hq, int Hk, int D, int rot_dim, int adjacent, int page_size,
                                int write_kv, hipStream_t stream) {
  if (T <= 0) return 0;
  if (Hq <= 0 || Hk < 0 || D <= 0 || rot_dim < 0 || rot_dim > D || (rot_dim & 1) || page_size <= 0)
    return SA_ERR_ARG;
  dim3 grid(T), block(256);
  int tpb = T >= 1024 ? 8 : (T >= 512 ? 4 : (T >= 256 ? 2 : 1));
  while (tpb > 1 && (size_t)tpb * ((size_t)Hk * D + 8) * 2 > 65536) tpb >>= 1;   // the values' tile has to fit LDS
  const size_t tile_bytes = (size_t)tpb * ((size_t)Hk * D + 8) * 2;
  if (act_dtype == SA_BF16 && cache_dtype == SA_BF16 && !adjacent && rot_dim == D && (D & 15) == 0 &&
      ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)inv_freq & 15) == 0 && tile_bytes <= 65536) {
    const long long items = (long long)tpb * (Hq + (write_kv ? Hk : 0)) * (D >> 4);   // eight pairs each
    const int threads = (int)(items >= 1024 ? 1024 : (items <= 256 ? 256 : (items + 63) / 64 * 64));
    hipLaunchKernelGGL(rope_kv_write_bf16_vec_kernel, dim3((T + tpb - 1) / tpb), dim3(threads),
                       write_kv ? tile_bytes : 0, stream, (bf16_t*)qkv, positions, inv_freq, slot, (bf16_t*)k_pages,
                       (bf16_t*)v_pages, T, Hq, Hk, D, page_size, write_kv, tpb);
    SA_LAUNCH_CHECK();
    return 0;
  }
#define GO(TA, TC)                                                                               \
  hipLaunchKernelGGL((rope_kv_write_kernel<TA, TC>), grid, block, 0, stream, (TA*)qkv, positions, \
                     inv_freq, slot, (TC*)k_pages, (TC*)v_pages, Hq, Hk, D, rot_dim, adjacent,   \
                     page_size, write_kv)
  if (act_dtype == SA_F32 && cache_dtype == SA_F32) GO(float, float);
  else if (act_dtype == SA_BF16 && cache_dtype == SA_BF16) GO(bf16_t, bf16_t);
  else return SA_ERR_UNSUPPORTED;
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// SwiGLU gate (serve/model.py:85): a[t, i] = silu(gu[t, i]) * gu[t, I + i]
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ void silu_mul_kernel(const TA* __restrict__ gu, TA* __restrict__ a, int T, int I) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= I) return;
  for (int t = blockIdx.y; t < T; t += gridDim.y) {
    const float g = to_float(gu[(size_t)t * 2 * I + i]);
    const float u = to_float(gu[(size_t)t * 2 * I + I + i]);
    a[(size_t)t * I + i] = from_float<TA>((g / (1.f + expf(-g))) * u);
  }
}

// the same, eight bf16 values per thread in 16-byte vectors (I % 8 == 0)
__global__ __launch_bounds__(256) void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ a,
                                                               int T, int I) {
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= I) return;
  for (int t = blockIdx.y; t < T; t += gridDim.y) {
    const uint4 gv = *reinterpret_cast<const uint4*>(gu + (size_t)t * 2 * I + i);
    const uint4 uv = *reinterpret_cast<const uint4*>(gu + (size_t)t * 2 * I + I + i);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w};
    const uint32_t uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g0 = bf16_bits_to_float(gw[k] & 0xffffu), g1 = bf16_bits_to_float(gw[k] >> 16);
      const float u0 = bf16_bits_to_float(uw[k] & 0xffffu), u1 = bf16_bits_to_float(uw[k] >> 16);
      const float o0 = (g0 / (1.f + expf(-g0))) * u0;
      const float o1 = (g1 / (1.f + expf(-g1))) * u1;
      ow[k] = (uint32_t)float_to_bf16_bits(o0) | ((uint32_t)float_to_bf16_bits(o1) << 16);
    }
    *reinterpret_cast<uint4*>(a + (size_t)t * I + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

extern "C" int sa_silu_mul(const void* gu, void* a, int act_dtype, int T, int I, hipStream_t stream) {
  if (T <= 0) return 0;
  if (I <= 0) return SA_ERR_ARG;
  if (act_dtype == SA_BF16 && (I & 7) == 0) {
    dim3 grid((I / 8 + 255) / 256, T < 32768 ? T : 32768), block(256);
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)a, T, I);
    SA_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((I + 255) / 256, T < 32768 ? T : 32768), block(256);
  if (act_dtype == SA_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)a, T, I);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)a, T, I);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}
