// Embedding lookup, residual add + RMSNorm, gate activation times up.
// All arithmetic is float32; storage is float32 or bfloat16.
#include <stdarg.h>
#include <stdio.h>

#include "api.h"
#include "common.h"

namespace shk {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// ------------------------------------------------------------------ embedding

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                             float* __restrict__ out, int hidden) {
  const int row = blockIdx.x;
  const T* src = table + static_cast<size_t>(ids[row]) * hidden;
  float* dst = out + static_cast<size_t>(row) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]);
}

// ------------------------------------------------------------ add + RMSNorm
// One workgroup per row.  add_rmsnorm_vec_kernel holds the row in registers
// (hidden a multiple of 4, at most 8192 elements): all loads are issued
// before the first use, so a row costs one memory round trip.
// add_rmsnorm_kernel takes every other size.

constexpr int kNormThreads = 256;
constexpr int kNormVecs = 2;  // float4 per thread: rows of up to 8192 elements with 1024 threads

__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                     __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  uint2 u;
  u.x = bf16_bits(v.x) | (static_cast<uint32_t>(bf16_bits(v.y)) << 16);
  u.y = bf16_bits(v.z) | (static_cast<uint32_t>(bf16_bits(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// TD is the type of delta: T, or float for the partial sums of a split product
// ([splits][resid_rows][hidden], added in order).  THREADS * 4 * kNormVecs
// elements fit; wide rows get 1024 threads so that few loads follow each other.
template <typename T, typename TD, int THREADS>
__global__ void __launch_bounds__(THREADS)
    add_rmsnorm_vec_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                           const float* __restrict__ weight, float eps, T* __restrict__ out,
                           const int32_t* __restrict__ rows, int hidden, int write_resid,
                           int splits, size_t split_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t row = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* x = resid + row * hidden;
  const TD* d = delta ? delta + row * hidden : nullptr;
  T* y = out + static_cast<size_t>(r) * hidden;
  const int nvec = hidden / 4;

  float4 v[kNormVecs], dv[kNormVecs], w[kNormVecs];
#pragma unroll
  for (int i = 0; i < kNormVecs; ++i) {
    const int c = threadIdx.x + i * THREADS;
    v[i] = dv[i] = w[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < nvec) {
      v[i] = load4(x + c * 4);
      if (d) dv[i] = load4(d + c * 4);
      w[i] = load4(weight + c * 4);
    }
  }
  // further parts, four at a time in flight, added in order
  for (int z0 = 1; z0 < splits; z0 += 4) {
    float4 more[4][kNormVecs];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < kNormVecs; ++i) {
        const int c = threadIdx.x + i * THREADS;
        more[u][i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < nvec && z0 + u < splits) more[u][i] = load4(d + (z0 + u) * split_stride + c * 4);
      }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < kNormVecs; ++i)
        dv[i].x += more[u][i].x, dv[i].y += more[u][i].y, dv[i].z += more[u][i].z,
            dv[i].w += more[u][i].w;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kNormVecs; ++i) {
    v[i].x += dv[i].x, v[i].y += dv[i].y, v[i].z += dv[i].z, v[i].w += dv[i].w;
    ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int i = 0; i < kNormVecs; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) continue;
    if (d && write_resid) store4(x + c * 4, v[i]);
    store4(y + c * 4, make_float4((v[i].x * inv) * w[i].x, (v[i].y * inv) * w[i].y,
                                  (v[i].z * inv) * w[i].z, (v[i].w * inv) * w[i].w));
  }
}

template <typename T>
__global__ void __launch_bounds__(kNormThreads)
    add_rmsnorm_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                       const float* __restrict__ weight, float eps, T* __restrict__ out,
                       const int32_t* __restrict__ rows, int hidden, int write_resid) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t row = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* x = resid + row * hidden;
  const T* d = delta ? delta + row * hidden : nullptr;
  T* y = out + static_cast<size_t>(r) * hidden;

  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    float v = x[i];
    if (d) {
      v += to_float(d[i]);
      if (write_resid) x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    float v = x[i];
    if (d && !write_resid) v += to_float(d[i]);
    y[i] = from_float<T>((v * inv) * weight[i]);
  }
}

// ------------------------------------------------------------ act(gate) * up
// act 1: SiLU, g / (1 + exp(-g)).  act 2: the tanh form of GELU,
// 0.5 g (1 + tanh(u)), u = sqrt(2/pi) (g + 0.044715 g^3), written as g / (1 + exp(-2u)).

template <typename T>
__global__ void act_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int act) {
  const size_t row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= inter) return;
  const float g = to_float(gu[row * 2 * inter + j]);
  const float u = to_float(gu[row * 2 * inter + inter + j]);
  const float x = act == 2 ? 2.f * 0.7978845608028654f * (g + 0.044715f * g * g * g) : g;
  const float s = g / (1.f + expf(-x));
  out[row * inter + j] = from_float<T>(s * u);
}

// dst[i] = src[i], except dst[patch_at + j] = patch[j] for j < patch_n.  Either side
// may be page-locked host memory: a step's index arrays come to the device, and
// its chosen tokens go back, without the copy engine, whose hand-overs to and from
// the compute queue cost more than these few hundred words.
__global__ void __launch_bounds__(256)
    copy_words_kernel(const int32_t* __restrict__ src, int32_t* __restrict__ dst, int n,
                      const int32_t* __restrict__ patch, int patch_at, int patch_n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int j = i - patch_at;
  dst[i] = (j >= 0 && j < patch_n) ? patch[j] : src[i];
}

// dst[r, :] = src[index[r], :], rows of `width` 32-bit words.
__global__ void __launch_bounds__(256)
    gather_rows_kernel(const int32_t* __restrict__ src, long long ld, const int32_t* __restrict__ index,
                       int32_t* __restrict__ dst, int width) {
  const int32_t* from = src + static_cast<long long>(index[blockIdx.y]) * ld;
  int32_t* to = dst + static_cast<long long>(blockIdx.y) * width;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < width; i += gridDim.x * blockDim.x) to[i] = from[i];
}

// Zeroes `bytes` bytes from dst (4-byte aligned): whole words, then the odd bytes.
__global__ void __launch_bounds__(256) zero_bytes_kernel(uint8_t* __restrict__ dst, long long bytes) {
  const long long words = bytes / 4;
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x; i < words; i += stride)
    reinterpret_cast<uint32_t*>(dst)[i] = 0u;
  if (blockIdx.x == 0 && threadIdx.x < bytes - words * 4) dst[words * 4 + threadIdx.x] = 0;
}

}  // namespace shk

using namespace shk;

extern "C" const char* shk_last_error(void) { return g_error; }
extern "C" int shk_version(void) { return 1; }

extern "C" int shk_copy_words(const int32_t* src, int32_t* dst, int n, const int32_t* patch,
                              int patch_at, int patch_n, void* stream) {
  SHK_REQUIRE(n >= 0 && patch_n >= 0 && patch_at >= 0 && patch_at + patch_n <= n,
              "copy_words: bad sizes n=%d patch [%d, %d)", n, patch_at, patch_at + patch_n);
  if (n == 0) return 0;
  SHK_REQUIRE(src && dst && (patch || patch_n == 0), "copy_words: null pointer");
  copy_words_kernel<<<(n + 255) / 256, 256, 0, static_cast<hipStream_t>(stream)>>>(src, dst, n, patch,
                                                                                 patch_at, patch_n);
  SHK_LAUNCH_CHECK("copy_words");
  return 0;
}

extern "C" int shk_gather_rows(const int32_t* src, long long ld, int src_rows, const int32_t* index,
                               int32_t* dst, int rows, int width, void* stream) {
  SHK_REQUIRE(rows >= 0 && width > 0 && ld >= width && src_rows >= 0,
              "gather_rows: bad sizes rows=%d width=%d ld=%lld", rows, width, ld);
  if (rows == 0) return 0;
  SHK_REQUIRE(src && index && dst, "gather_rows: null pointer");
  SHK_REQUIRE(rows <= 65535, "gather_rows: at most 65535 rows per call, got %d", rows);
  const int per_row = (width + 255) / 256 < 64 ? (width + 255) / 256 : 64;
  gather_rows_kernel<<<dim3(per_row, rows), 256, 0, static_cast<hipStream_t>(stream)>>>(src, ld, index, dst,
                                                                                       width);
  SHK_LAUNCH_CHECK("gather_rows");
  return 0;
}

extern "C" int shk_zero_bytes(void* dst, long long bytes, void* stream) {
  SHK_REQUIRE(bytes >= 0, "zero_bytes: negative size");
  if (bytes == 0) return 0;
  SHK_REQUIRE(dst && reinterpret_cast<uintptr_t>(dst) % 4 == 0, "zero_bytes: dst must be 4-byte aligned");
  const long long blocks = (bytes / 4 + 255) / 256;
  zero_bytes_kernel<<<static_cast<int>(blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks)), 256, 0,
                      static_cast<hipStream_t>(stream)>>>(static_cast<uint8_t*>(dst), bytes);
  SHK_LAUNCH_CHECK("zero_bytes");
  return 0;
}

extern "C" int shk_embed(const void* table, int dtype, const int32_t* ids, float* out, int n,
                         int hidden, int vocab, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "embed: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes n=%d hidden=%d vocab=%d", n,
              hidden, vocab);
  if (n == 0) return 0;
  SHK_REQUIRE(table && ids && out, "embed: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = hidden >= 256 ? 256 : 64;
  if (dtype == kF32)
    embed_kernel<float><<<n, threads, 0, s>>>(static_cast<const float*>(table), ids, out, hidden);
  else
    embed_kernel<bf16><<<n, threads, 0, s>>>(static_cast<const bf16*>(table), ids, out, hidden);
  SHK_LAUNCH_CHECK("embed");
  return 0;
}

extern "C" int shk_add_rmsnorm(float* resid, const void* delta, const float* weight, float eps,
                               void* out, int dtype, const int32_t* rows, int n, int hidden,
                               int write_resid, int delta_splits, int resid_rows, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "add_rmsnorm: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0, "add_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
  SHK_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be > 0");
  if (n == 0) return 0;
  SHK_REQUIRE(resid && weight && out, "add_rmsnorm: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = hidden % 4 == 0 && hidden <= 1024 * 4 * kNormVecs && aligned(resid) &&
                   aligned(weight) && aligned(out) && (!delta || aligned(delta));
  SHK_REQUIRE(delta_splits == 0 || (delta && vec && dtype == kBF16 && resid_rows > 0),
              "add_rmsnorm: partial sums need bfloat16 output, hidden %% 4 == 0 and at most 8192");
  const size_t stride = static_cast<size_t>(resid_rows) * hidden;
  const int splits = delta_splits > 0 ? delta_splits : 1;
#define SHK_NORM(T, TD, THREADS)                                                              \
  add_rmsnorm_vec_kernel<T, TD, THREADS><<<n, THREADS, 0, s>>>(                               \
      resid, static_cast<const TD*>(delta), weight, eps, static_cast<T*>(out), rows, hidden,  \
      write_resid, splits, stride)
#define SHK_NORM_T(T, TD)                \
  do {                                   \
    if (hidden <= 256 * 4 * kNormVecs)   \
      SHK_NORM(T, TD, 256);              \
    else                                 \
      SHK_NORM(T, TD, 1024);             \
  } while (0)
  if (delta_splits > 0) {
    SHK_NORM_T(bf16, float);
  } else if (vec && dtype == kF32) {
    SHK_NORM_T(float, float);
  } else if (vec) {
    SHK_NORM_T(bf16, bf16);
  } else if (dtype == kF32) {
    add_rmsnorm_kernel<float><<<n, kNormThreads, 0, s>>>(
        resid, static_cast<const float*>(delta), weight, eps, static_cast<float*>(out), rows,
        hidden, write_resid);
  } else {
    add_rmsnorm_kernel<bf16><<<n, kNormThreads, 0, s>>>(
        resid, static_cast<const bf16*>(delta), weight, eps, static_cast<bf16*>(out), rows, hidden,
        write_resid);
  }
#undef SHK_NORM_T
#undef SHK_NORM
  SHK_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

extern "C" int shk_act_mul(const void* gu, void* out, int dtype, int n, int inter, int act, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "act_mul: unknown dtype %d", dtype);
  SHK_REQUIRE(act == 1 || act == 2, "act_mul: unknown activation %d", act);
  SHK_REQUIRE(n >= 0 && inter > 0, "act_mul: bad sizes n=%d inter=%d", n, inter);
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "act_mul: at most 65535 rows a call, got %d", n);
  SHK_REQUIRE(gu && out, "act_mul: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((inter + 255) / 256, n);
  if (dtype == kF32)
    act_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gu),
                                                static_cast<float*>(out), inter, act);
  else
    act_mul_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(gu),
                                               static_cast<bf16*>(out), inter, act);
  SHK_LAUNCH_CHECK("act_mul");
  return 0;
}
