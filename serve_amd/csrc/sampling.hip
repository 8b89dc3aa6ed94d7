// Token choice from fp32 logits: greedy argmax, or a categorical draw at a temperature.
//
// The reference draws with argmax(softmax(logits / T) / q), q ~ Exp(1) per vocabulary entry
// (serve/run.py:48-60).  log is monotone, so the same draw is argmax(logits / T - log q) and no
// softmax pass over the vocabulary is needed.  q comes from a counter-based generator: a 64-bit
// mix of a per-row key (made on the host from seed, request and index of the generated token)
// and the vocabulary index, so a request's draws do not depend on what else is in the batch.
// Ties go to the lowest index.
#include "common.h"
#include "sampling.h"

#include <mutex>

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

// Stage 1: block (chunk, row) scans its chunk of the vocabulary and writes its best (score, index).
__global__ __launch_bounds__(256) void sample_partial_kernel(const float* __restrict__ logits,
                                                             const float* __restrict__ temperature,
                                                             const unsigned long long* __restrict__ keys,
                                                             float* __restrict__ part_v, int* __restrict__ part_i,
                                                             int V, int chunk, int by_four) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int r = blockIdx.y;
  const float* row = logits + (size_t)r * V;
  const float temp = temperature ? temperature[r] : 0.f;
  const bool greedy = !(temp > 0.f);
  const float inv_t = greedy ? 1.f : 1.f / temp;
  const unsigned long long key = greedy ? 0ull : keys[r];
  const int lo = blockIdx.x * chunk;
  const int hi = min(V, lo + chunk);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  auto score = [&](float v, int i) __attribute__((always_inline)) {
    if (!greedy) {
      const unsigned int bits = (unsigned int)(mix64(key ^ (unsigned long long)i) >> 41);
      const float u = ((float)bits + 0.5f) * (1.0f / 8388608.0f);
      v = v * inv_t - logf(-logf(u));
    }
    take_better(bv, bi, v, i);
  };
  if (by_four) {
    // rows and chunks begin on 16-byte boundaries and hold whole groups of four: 16 bytes a load
    const float4* row4 = reinterpret_cast<const float4*>(row + lo);
    const int n4 = (hi - lo) >> 2;
    for (int j = threadIdx.x; j < n4; j += blockDim.x) {
      const float4 q = row4[j];
      const int i = lo + 4 * j;
      score(q.x, i);
      score(q.y, i + 1);
      score(q.z, i + 2);
      score(q.w, i + 3);
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) score(row[i], i);
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
    part_v[(size_t)r * gridDim.x + blockIdx.x] = bv;
    part_i[(size_t)r * gridDim.x + blockIdx.x] = bi;
  }
}

// Stage 2: one wave per row picks the best of the chunks (ties still go to the lowest index).
__global__ __launch_bounds__(64) void sample_final_kernel(const float* __restrict__ part_v,
                                                          const int* __restrict__ part_i,
                                                          int* __restrict__ out, int nchunks) {
  const int r = blockIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < nchunks; c += SA_WAVE)
    take_better(bv, bi, part_v[(size_t)r * nchunks + c], part_i[(size_t)r * nchunks + c]);
#pragma unroll
  for (int o = SA_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, SA_WAVE);
    const int oi = __shfl_xor(bi, o, SA_WAVE);
    take_better(bv, bi, ov, oi);
  }
  if (threadIdx.x == 0) out[r] = bi == 0x7fffffff ? 0 : bi;
}

// how many chunks the vocabulary is cut into (the caller sizes the scratch arrays with it)
extern "C" int sa_sample_chunks(int V) {
  const int chunk = 2048;
  int n = (V + chunk - 1) / chunk;
  return n < 1 ? 1 : n;
}

extern "C" int sa_sample(const float* logits, const float* temperature, const unsigned long long* keys,
                         int* out, float* part_v, int* part_i, int R, int V, hipStream_t stream) {
  if (R <= 0) return 0;
  if (V <= 0 || R > 65535 || !part_v || !part_i) return SA_ERR_ARG;
  const int nchunks = sa_sample_chunks(V);
  int chunk = (V + nchunks - 1) / nchunks;
  // a vocabulary of whole groups of four from an aligned address is read 16 bytes a lane (chunks of whole
  // groups too; the last chunks may then be shorter or empty, which the second stage does not mind)
  const int by_four = (V & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0;
  if (by_four) chunk = (chunk + 3) & ~3;
  hipLaunchKernelGGL(sample_partial_kernel, dim3(nchunks, R), dim3(256), 0, stream, logits, temperature, keys,
                     part_v, part_i, V, chunk, by_four);
  SA_LAUNCH_CHECK();
  hipLaunchKernelGGL(sample_final_kernel, dim3(R), dim3(64), 0, stream, part_v, part_i, out, nchunks);
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The same two kernels with their partial results in an array of the library's own, for callers
// that cannot allocate (see sampling.h).  `scratch` is a device symbol: in host code its name is
// only a stand-in, the array's address on a device comes from hipGetSymbolAddress, once per
// device (every GPU holds its own copy of the array at its own address).
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[SA_SAMPLE_NOALLOC_ENTRIES * 8];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// the address of `scratch` on the current device; 0 and *err set if the lookup fails
void* scratch_on_current_device(int* err) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    *err = (int)e;
    return nullptr;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    *err = SA_ERR_ARG;
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      *err = e != hipSuccess ? (int)e : SA_ERR_ARG;
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int sa_sample_noalloc_max_entries(void) { return SA_SAMPLE_NOALLOC_ENTRIES; }

extern "C" int sa_sample_noalloc(const float* logits, const float* temperature, const unsigned long long* keys,
                                 int* out, int R, int V, hipStream_t stream) {
  if (R <= 0) return 0;
  if (V <= 0 || R > 65535 || !logits || !out) return SA_ERR_ARG;
  const long long entries = (long long)R * sa_sample_chunks(V);
  if (entries > SA_SAMPLE_NOALLOC_ENTRIES) return SA_ERR_ARG;
  int err = 0;
  void* base = scratch_on_current_device(&err);
  if (!base) return err;
  // first half: the chunks' best scores, second half: their indices
  float* part_v = reinterpret_cast<float*>(base);
  int* part_i = reinterpret_cast<int*>(static_cast<unsigned char*>(base) + (size_t)SA_SAMPLE_NOALLOC_ENTRIES * 4);
  return sa_sample(logits, temperature, keys, out, part_v, part_i, R, V, stream);
}
