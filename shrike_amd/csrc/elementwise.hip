// Embedding lookup, residual add + RMSNorm, SiLU-multiply.
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
// One workgroup per row.  The row is read once into registers when it fits
// (hidden <= 256 * kMaxPerThread), otherwise it is re-read from resid.

constexpr int kNormThreads = 256;

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

// ---------------------------------------------------------------- SiLU * up

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
  const size_t row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= inter) return;
  const float g = to_float(gu[row * 2 * inter + j]);
  const float u = to_float(gu[row * 2 * inter + inter + j]);
  const float s = g / (1.f + expf(-g));
  out[row * inter + j] = from_float<T>(s * u);
}

}  // namespace shk

using namespace shk;

extern "C" const char* shk_last_error(void) { return g_error; }
extern "C" int shk_version(void) { return 1; }

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
                               int write_resid, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "add_rmsnorm: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && hidden > 0, "add_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
  SHK_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be > 0");
  if (n == 0) return 0;
  SHK_REQUIRE(resid && weight && out, "add_rmsnorm: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32)
    add_rmsnorm_kernel<float><<<n, kNormThreads, 0, s>>>(
        resid, static_cast<const float*>(delta), weight, eps, static_cast<float*>(out), rows,
        hidden, write_resid);
  else
    add_rmsnorm_kernel<bf16><<<n, kNormThreads, 0, s>>>(
        resid, static_cast<const bf16*>(delta), weight, eps, static_cast<bf16*>(out), rows, hidden,
        write_resid);
  SHK_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

extern "C" int shk_silu_mul(const void* gu, void* out, int dtype, int n, int inter, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "silu_mul: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && inter > 0, "silu_mul: bad sizes n=%d inter=%d", n, inter);
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "silu_mul: at most 65535 rows a call, got %d", n);
  SHK_REQUIRE(gu && out, "silu_mul: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((inter + 255) / 256, n);
  if (dtype == kF32)
    silu_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gu),
                                                static_cast<float*>(out), inter);
  else
    silu_mul_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(gu),
                                               static_cast<bf16*>(out), inter);
  SHK_LAUNCH_CHECK("silu_mul");
  return 0;
}
