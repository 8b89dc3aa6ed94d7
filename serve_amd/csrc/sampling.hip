// Token choice from fp32 logits: greedy argmax, or a categorical draw at a temperature.
//
// The reference draws with argmax(softmax(logits / T) / q), q ~ Exp(1) per vocabulary entry
// (serve/run.py:48-60).  log is monotone, so the same draw is argmax(logits / T - log q) and no
// softmax pass over the vocabulary is needed.  q comes from a counter-based generator: a 64-bit
// mix of a per-row key (made on the host from seed, request and index of the generated token)
// and the vocabulary index, so a request's draws do not depend on what else is in the batch.
// Ties go to the lowest index.
#include "common.h"

__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ void take_better(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) {
    bv = v;
    bi = i;
  }
}

__global__ __launch_bounds__(256) void sample_kernel(const float* __restrict__ logits,
                                                     const float* __restrict__ temperature,
                                                     const unsigned long long* __restrict__ keys,
                                                     int* __restrict__ out, int V) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * V;
  const float temp = temperature ? temperature[r] : 0.f;
  const bool greedy = !(temp > 0.f);
  const float inv_t = greedy ? 1.f : 1.f / temp;
  const unsigned long long key = greedy ? 0ull : keys[r];
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    float v = row[i];
    if (!greedy) {
      const unsigned int bits = (unsigned int)(mix64(key ^ (unsigned long long)i) >> 41);
      const float u = ((float)bits + 0.5f) * (1.0f / 8388608.0f);
      v = v * inv_t - logf(-logf(u));
    }
    take_better(bv, bi, v, i);
  }
#pragma unroll
  for (int o = SA_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, SA_WAVE);
    const int oi = __shfl_xor(bi, o, SA_WAVE);
    take_better(bv, bi, ov, oi);
  }
  const int lane = threadIdx.x & (SA_WAVE - 1);
  const int wave = threadIdx.x / SA_WAVE;
  if (lane == 0) {
    sv[wave] = bv;
    si[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) take_better(bv, bi, sv[w], si[w]);
    out[r] = bi == 0x7fffffff ? 0 : bi;
  }
}

extern "C" int sa_sample(const float* logits, const float* temperature, const unsigned long long* keys,
                         int* out, int R, int V, hipStream_t stream) {
  if (R <= 0) return 0;
  if (V <= 0) return SA_ERR_ARG;
  hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(256), 0, stream, logits, temperature, keys, out, V);
  SA_LAUNCH_CHECK();
  return 0;
}
