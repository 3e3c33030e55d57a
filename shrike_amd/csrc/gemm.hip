// out[n, m] = a[n, k] @ w[m, k]^T + bias: the matrix products of the model
// (projections, feed-forward, output matrix).
//
// gemm_tiled_kernel is the general kernel: every size, float32 or bfloat16
// storage, float32 fused-multiply-add accumulation in ascending k for every
// output element.  It is the whole of the float32 path (no matrix mode of
// reduced precision is involved) and the fallback of the bfloat16 path.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kTM = 64;  // rows of a (tokens) per workgroup
constexpr int kTN = 64;  // rows of w (output features) per workgroup
constexpr int kTK = 16;  // depth of one staged slice

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
    gemm_tiled_kernel(const TI* __restrict__ a, const TI* __restrict__ w,
                      const float* __restrict__ bias, TO* __restrict__ out, int n, int m, int k,
                      int lda, int ldo, int accumulate) {
  __shared__ float as[kTK][kTM + 4];
  __shared__ float ws[kTK][kTN + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int row0 = blockIdx.y * kTM, col0 = blockIdx.x * kTN;

  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += kTK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = threadIdx.x + i * 256;  // 0..1023 over [64 rows][16 k]
      const int r = idx / kTK, kk = idx % kTK;
      const int gr = row0 + r, gc = col0 + r, gk = k0 + kk;
      as[kk][r] = (gr < n && gk < k) ? to_float(a[static_cast<size_t>(gr) * lda + gk]) : 0.f;
      ws[kk][r] = (gc < m && gk < k) ? to_float(w[static_cast<size_t>(gc) * k + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gr = row0 + ty * 4 + i;
    if (gr >= n) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gc = col0 + tx * 4 + j;
      if (gc >= m) continue;
      float v = acc[i][j];
      if (bias) v += bias[gc];
      TO* dst = out + static_cast<size_t>(gr) * ldo + gc;
      if (accumulate) v += to_float(*dst);
      *dst = from_float<TO>(v);
    }
  }
}

template <typename TI, typename TO>
static int launch_tiled(const void* a, const void* w, const float* bias, void* out, int n, int m,
                        int k, int lda, int ldo, int accumulate, hipStream_t s) {
  dim3 grid((m + kTN - 1) / kTN, (n + kTM - 1) / kTM);
  gemm_tiled_kernel<TI, TO><<<grid, 256, 0, s>>>(static_cast<const TI*>(a),
                                                 static_cast<const TI*>(w), bias,
                                                 static_cast<TO*>(out), n, m, k, lda, ldo,
                                                 accumulate);
  return 0;
}

}  // namespace shk

using namespace shk;

extern "C" int shk_gemm(const void* a, const void* w, const float* bias, void* out, int n, int m,
                        int k, int lda, int ldo, int in_dtype, int out_dtype, int accumulate,
                        void* stream) {
  SHK_REQUIRE(in_dtype == kF32 || in_dtype == kBF16, "gemm: unknown in_dtype %d", in_dtype);
  SHK_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "gemm: unknown out_dtype %d", out_dtype);
  SHK_REQUIRE(n >= 0 && m > 0 && k > 0, "gemm: bad sizes n=%d m=%d k=%d", n, m, k);
  SHK_REQUIRE(lda >= k && ldo >= m, "gemm: row strides lda=%d ldo=%d too small for k=%d m=%d", lda,
              ldo, k, m);
  SHK_REQUIRE(!accumulate || out_dtype == kF32, "gemm: accumulate needs a float32 output");
  SHK_REQUIRE(!(in_dtype == kF32 && out_dtype == kBF16),
              "gemm: float32 inputs with a bfloat16 output are not built");
  if (n == 0) return 0;
  SHK_REQUIRE(a && w && out, "gemm: null pointer");
  SHK_REQUIRE((n + kTM - 1) / kTM <= 65535, "gemm: too many rows (%d)", n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == kF32)
    launch_tiled<float, float>(a, w, bias, out, n, m, k, lda, ldo, accumulate, s);
  else if (out_dtype == kF32)
    launch_tiled<bf16, float>(a, w, bias, out, n, m, k, lda, ldo, accumulate, s);
  else
    launch_tiled<bf16, bf16>(a, w, bias, out, n, m, k, lda, ldo, accumulate, s);
  SHK_LAUNCH_CHECK("gemm");
  return 0;
}
