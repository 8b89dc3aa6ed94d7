// Shared device helpers for the gfx950 kernels: storage types, conversions, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SA_WAVE 64

// dtype codes of the C interface
enum { SA_F32 = 0, SA_BF16 = 1 };

// error codes of the C interface (0 = ok, >0 = hipError_t of the launch)
enum { SA_ERR_ARG = -1, SA_ERR_UNSUPPORTED = -2 };

struct bf16_t {
  uint16_t v;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return bf16_bits_to_float(x.v); }

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
  bf16_t r;
  r.v = float_to_bf16_bits(x);
  return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = SA_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, SA_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = SA_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, SA_WAVE));
  return v;
}

// sum over a block of up to 1024 threads; `scratch` holds at least 16 floats of LDS
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (SA_WAVE - 1);
  const int wave = threadIdx.x / SA_WAVE;
  const int nwaves = (blockDim.x + SA_WAVE - 1) / SA_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

// sin and cos of an angle of up to 4e6 rad (a position times a frequency of at most 1), to about
// 1e-6: the library's sincosf spends over a thousand cycles on arguments this large.  The multiple
// of 2 pi is taken off in three steps whose constants have few enough bits for the first two
// remainders to be exact (6.28125 = 201/32; 2029/2^20; the rest: with k < 2^20 the first remainder
// is a multiple of 2^-5 below 2^11, the second a multiple of 2^-20 below 4), the last remainder
// goes to the hardware's sine and cosine, which take their argument in turns.  Callers keep their
// angles within the bound (the rotary part refuses longer contexts when it is loaded).
__device__ __forceinline__ void sincos_reduced(float x, float* sn, float* cs) {
  const float k = rintf(x * 0.15915494309189535f);
  float r = fmaf(-k, 6.28125f, x);
  r = fmaf(-k, 1.93500518798828125e-3f, r);
  r = fmaf(-k, 3.0199159776e-7f, r);
  const float t = r * 0.15915494309189535f;
  *sn = __builtin_amdgcn_sinf(t);
  *cs = __builtin_amdgcn_cosf(t);
}

#define SA_LAUNCH_CHECK()                      \
  do {                                         \
    hipError_t e__ = hipGetLastError();        \
    if (e__ != hipSuccess) return (int)e__;    \
  } while (0)

// compute units of the current device (asked once per device; 256 if the runtime will not say)
static inline int compute_units() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cached[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}
