// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wavefront (64 lanes) and workgroup reductions, and the host-side error slot.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace shk {

constexpr int kWave = 64;

// bfloat16 is handled as its 16 bit pattern; all arithmetic is done in float.
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16 x) {
  return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}

// Round to nearest, ties to even; NaN stays NaN.
__device__ __forceinline__ uint16_t bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float x) {
  return bf16{bf16_bits(x)};
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats and may be reused after the call returns.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// ------------------------------------------------------- layout of cached keys
// The keys of one key/value head in one page are stored in slabs of 32
// elements, [head_dim / 32][page_size][32] (the whole row as one slab where
// head_dim is no multiple of 32): the 16 bytes a lane of an MFMA operand needs
// from each of four consecutive keys then lie side by side, 64 bytes per key,
// and a wavefront's operand load touches whole cache lines.  Values are stored
// transposed, [head_dim][page_size].
__host__ __device__ inline int key_slab(int head_dim) { return head_dim % 32 == 0 ? 32 : head_dim; }

// Offset of element d of the key in `slot`, in elements from the start of its page's head.
__host__ __device__ inline size_t key_offset(int slot, int d, int page_size, int head_dim) {
  const int slab = key_slab(head_dim);
  return (static_cast<size_t>(d / slab) * page_size + slot) * slab + d % slab;
}

// ---------------------------------------------------------------- host side

enum DType : int { kF32 = 0, kBF16 = 1 };

// Records the message of the first failure of a call; shk_last_error returns it.
void set_error(const char* fmt, ...);

inline size_t dtype_size(int dtype) { return dtype == kBF16 ? 2 : 4; }

}  // namespace shk

#define SHK_REQUIRE(cond, ...)        \
  do {                                \
    if (!(cond)) {                    \
      ::shk::set_error(__VA_ARGS__);  \
      return 1;                       \
    }                                 \
  } while (0)

#define SHK_LAUNCH_CHECK(name)                                              \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      ::shk::set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return 2;                                                             \
    }                                                                       \
  } while (0)
