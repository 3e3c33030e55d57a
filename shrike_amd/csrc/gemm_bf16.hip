// bfloat16 matrix products on the MFMA units, over weights that were re-laid
// at load time into the operand layout of v_mfma_f32_16x16x32_bf16.
//
// Tiled weight layout ("wt"): the [m, k] matrix is padded with zeros to
// [mb*16, kt*32] and cut into tiles of 16 rows x 32 columns.  Tile (b, t) is
// 1 KiB: lane l of a wavefront owns 16 bytes, the 8 values
// w[b*16 + l%16][t*32 + (l/16)*8 .. +8].  Tiles are stored [mb][kt][64 lanes],
// so the operand of one MFMA is one fully coalesced 1 KiB load and a block of
// 16 rows streams as one contiguous region.
//
// gemm_skinny_kernel: for few tokens (decode).  One workgroup of 4 wavefronts
// per block of 16 weight rows; the wavefronts take the k-tiles round-robin and
// their partial sums are added in a fixed order through LDS.  The weights are
// read exactly once from HBM; accumulation is float32.
#include "api.h"
#include "common.h"

namespace shk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

union Frag {
  uint4 u;
  bf16x8 v;
  uint16_t h[8];
};

// Eight consecutive activations a[token][kk .. kk+8) as an MFMA operand; zero
// beyond the matrix.  `vec` says rows are 16-byte aligned and k % 8 == 0.
__device__ __forceinline__ Frag load_act(const bf16* __restrict__ a, int lda, int n, int k,
                                         int token, int kk, bool vec) {
  Frag f;
  f.u = make_uint4(0, 0, 0, 0);
  if (token < n && kk < k) {
    const bf16* p = a + static_cast<size_t>(token) * lda + kk;
    if (vec) {
      f.u = *reinterpret_cast<const uint4*>(p);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (kk + e < k) f.h[e] = p[e].bits;
    }
  }
  return f;
}

constexpr int kSkinnyWaves = 4;
constexpr int kSkinnyUnroll = 8;

template <int NB>
__global__ void __launch_bounds__(kSkinnyWaves* kWave)
    gemm_skinny_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                       const uint4* __restrict__ wt, int ktiles, int m,
                       const float* __restrict__ bias, void* __restrict__ out, int ldo,
                       int out_f32, int accumulate, int vec) {
  __shared__ float red[kSkinnyWaves][NB][kWave][4];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int mb = blockIdx.x;
  const int j = lane % 16, kg = lane / 16;
  const uint4* wrow = wt + static_cast<size_t>(mb) * ktiles * kWave + lane;

  f32x4 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // k-tiles wave, wave + 4, ...; kSkinnyUnroll of them in flight at a time
  int t = wave;
  for (; t + (kSkinnyUnroll - 1) * kSkinnyWaves < ktiles; t += kSkinnyUnroll * kSkinnyWaves) {
    Frag w[kSkinnyUnroll];
#pragma unroll
    for (int u = 0; u < kSkinnyUnroll; ++u)
      w[u].u = wrow[static_cast<size_t>(t + u * kSkinnyWaves) * kWave];
#pragma unroll
    for (int u = 0; u < kSkinnyUnroll; ++u) {
      const int kk = (t + u * kSkinnyWaves) * 32 + kg * 8;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const Frag x = load_act(a, lda, n, k, b * 16 + j, kk, vec);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u].v, x.v, acc[b], 0, 0, 0);
      }
    }
  }
  for (; t < ktiles; t += kSkinnyWaves) {
    Frag w;
    w.u = wrow[static_cast<size_t>(t) * kWave];
    const int kk = t * 32 + kg * 8;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const Frag x = load_act(a, lda, n, k, b * 16 + j, kk, vec);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, x.v, acc[b], 0, 0, 0);
    }
  }

#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][b][lane][r] = acc[b][r];
  __syncthreads();

  // Lane (j, kg) of accumulator b holds rows kg*4 + r of the block for token b*16 + j.
  // Wavefront w finishes the token blocks b = w, w + 4, ...
  for (int b = wave; b < NB; b += kSkinnyWaves) {
    const int token = b * 16 + j;
    if (token >= n) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = mb * 16 + kg * 4 + r;
      if (row >= m) continue;
      float v = red[0][b][lane][r];
#pragma unroll
      for (int w = 1; w < kSkinnyWaves; ++w) v += red[w][b][lane][r];
      if (bias) v += bias[row];
      const size_t idx = static_cast<size_t>(token) * ldo + row;
      if (out_f32) {
        float* o = static_cast<float*>(out);
        o[idx] = accumulate ? o[idx] + v : v;
      } else {
        static_cast<bf16*>(out)[idx] = from_float<bf16>(v);
      }
    }
  }
}

// gemm_big_kernel: for many tokens (prompt portions).  A workgroup of 4
// wavefronts computes 128 weight rows x 128 tokens; each wavefront a 64 x 64
// quadrant as 4 x 4 MFMA tiles.  Per stage of 64 columns of k, the weights'
// tiles (already in operand layout) and the activations (re-laid on the way)
// are staged in LDS "fragment-major": the 16 bytes of lane l of a fragment sit
// at l * 16, so every LDS access is a conflict-free 128-bit access.  Stages are
// double-buffered: the loads of stage t+1 are in flight while stage t is
// multiplied.

constexpr int kBigM = 128;   // weight rows per workgroup
constexpr int kBigN = 128;   // tokens per workgroup
constexpr int kBigK = 64;    // k per stage (two MFMA steps)
constexpr int kBigFrags = (kBigM / 16) * (kBigK / 32);  // fragments per operand per stage: 16

__global__ void __launch_bounds__(256)
    gemm_big_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                    const uint4* __restrict__ wt, int ktiles, int m,
                    const float* __restrict__ bias, void* __restrict__ out, int ldo, int out_f32,
                    int accumulate, int vec) {
  // [buffer][operand: 0 weights, 1 activations][fragment][lane]
  __shared__ uint4 stage[2][2][kBigFrags][kWave];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / 2, wn = wave % 2;  // quadrant of the wavefront
  const int mb0 = blockIdx.x * (kBigM / 16);   // first block of 16 weight rows
  const int tok0 = blockIdx.y * kBigN;
  const int mblocks = (m + 15) / 16;
  const int nstages = (ktiles + 1) / 2;

  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int jn = 0; jn < 4; ++jn) acc[i][jn] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Each thread moves 4 fragments-lanes per operand per stage: fragment f = tid/64 + 4*i
  // (f = rb * 2 + ks: block of 16 rows rb, MFMA step ks), lane = tid % 64.
  uint4 wreg[4], areg[4];
  auto load_stage = [&](int st) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int f = wave + 4 * i, rb = f / 2, ks = f % 2;
      const int kt = st * 2 + ks;
      const int mb = mb0 + rb;
      wreg[i] = make_uint4(0, 0, 0, 0);
      if (mb < mblocks && kt < ktiles)
        wreg[i] = wt[(static_cast<size_t>(mb) * ktiles + kt) * kWave + lane];
      const int token = tok0 + rb * 16 + lane % 16;
      areg[i] = load_act(a, lda, n, k, token, kt * 32 + (lane / 16) * 8, vec).u;
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int f = wave + 4 * i;
      stage[buf][0][f][lane] = wreg[i];
      stage[buf][1][f][lane] = areg[i];
    }
  };

  load_stage(0);
  store_stage(0);
  __syncthreads();
  for (int st = 0; st < nstages; ++st) {
    const int buf = st & 1;
    if (st + 1 < nstages) load_stage(st + 1);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      Frag wf[4], af[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) wf[i].u = stage[buf][0][(wm * 4 + i) * 2 + ks][lane];
#pragma unroll
      for (int jn = 0; jn < 4; ++jn) af[jn].u = stage[buf][1][(wn * 4 + jn) * 2 + ks][lane];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jn = 0; jn < 4; ++jn)
          acc[i][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, af[jn].v, acc[i][jn], 0, 0, 0);
    }
    if (st + 1 < nstages) store_stage(buf ^ 1);
    __syncthreads();
  }

  // lane (j, kg) of tile (i, jn): token tok0 + (wn*4 + jn)*16 + j, rows (mb0 + wm*4 + i)*16 + kg*4 + r
  const int j = lane % 16, kg = lane / 16;
#pragma unroll
  for (int jn = 0; jn < 4; ++jn) {
    const int token = tok0 + (wn * 4 + jn) * 16 + j;
    if (token >= n) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row0 = (mb0 + wm * 4 + i) * 16 + kg * 4;
      if (row0 >= m) continue;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] = acc[i][jn][r];
        if (bias && row0 + r < m) v[r] += bias[row0 + r];
      }
      const size_t idx = static_cast<size_t>(token) * ldo + row0;
      if (out_f32) {
        float* o = static_cast<float*>(out) + idx;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (row0 + r < m) o[r] = accumulate ? o[r] + v[r] : v[r];
      } else {
        bf16* o = static_cast<bf16*>(out) + idx;
        if (row0 + 3 < m && (ldo & 3) == 0) {
          uint2 packed;
          packed.x = bf16_bits(v[0]) | (static_cast<uint32_t>(bf16_bits(v[1])) << 16);
          packed.y = bf16_bits(v[2]) | (static_cast<uint32_t>(bf16_bits(v[3])) << 16);
          *reinterpret_cast<uint2*>(o) = packed;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (row0 + r < m) o[r] = from_float<bf16>(v[r]);
        }
      }
    }
  }
}

}  // namespace shk

using namespace shk;

// Re-lays a row-major bfloat16 [m, k] matrix into the tiled layout.
__global__ void retile_kernel(const bf16* __restrict__ w, int m, int k, uint4* __restrict__ wt,
                              int ktiles) {
  const int mb = blockIdx.y, t = blockIdx.x, lane = threadIdx.x;
  const int row = mb * 16 + lane % 16, col = t * 32 + (lane / 16) * 8;
  Frag f;
  f.u = make_uint4(0, 0, 0, 0);
  if (row < m) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (col + e < k) f.h[e] = w[static_cast<size_t>(row) * k + col + e].bits;
  }
  wt[(static_cast<size_t>(mb) * ktiles + t) * kWave + lane] = f.u;
}

extern "C" int shk_retile_weight(const void* w, int m, int k, void* wt, void* stream) {
  SHK_REQUIRE(m > 0 && k > 0 && w && wt, "retile_weight: bad arguments m=%d k=%d", m, k);
  const int mb = (m + 15) / 16, kt = (k + 31) / 32;
  // grid.y is limited to 65535 blocks: 1,048,560 rows
  SHK_REQUIRE(mb <= 65535, "retile_weight: too many rows (%d)", m);
  retile_kernel<<<dim3(kt, mb), kWave, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const bf16*>(w), m, k, static_cast<uint4*>(wt), kt);
  SHK_LAUNCH_CHECK("retile_weight");
  return 0;
}

extern "C" int shk_gemm_bf16_tiled_weight(const void* a, const void* wt, const float* bias,
                                          void* out, int n, int m, int k, int lda, int ldo,
                                          int out_dtype, int accumulate, void* stream) {
  SHK_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "gemm_bf16: unknown out_dtype %d",
              out_dtype);
  SHK_REQUIRE(n >= 0 && m > 0 && k > 0, "gemm_bf16: bad sizes n=%d m=%d k=%d", n, m, k);
  SHK_REQUIRE(lda >= k && ldo >= m, "gemm_bf16: row strides lda=%d ldo=%d too small", lda, ldo);
  SHK_REQUIRE(!accumulate || out_dtype == kF32, "gemm_bf16: accumulate needs a float32 output");
  if (n == 0) return 0;
  SHK_REQUIRE(a && wt && out, "gemm_bf16: null pointer");
  const int mb = (m + 15) / 16, kt = (k + 31) / 32;
  const int vec = (k % 8 == 0 && lda % 8 == 0 && (reinterpret_cast<uintptr_t>(a) % 16) == 0);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bf16* ap = static_cast<const bf16*>(a);
  const uint4* wp = static_cast<const uint4*>(wt);
  const int of = out_dtype == kF32;
  if (n > 64) {
    SHK_REQUIRE(reinterpret_cast<uintptr_t>(out) % 8 == 0, "gemm_bf16: out is not 8-byte aligned");
    dim3 grid((m + kBigM - 1) / kBigM, (n + kBigN - 1) / kBigN);
    SHK_REQUIRE(grid.y <= 65535, "gemm_bf16: too many rows (%d)", n);
    gemm_big_kernel<<<grid, 256, 0, s>>>(ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate,
                                         vec);
    SHK_LAUNCH_CHECK("gemm_bf16");
    return 0;
  }
#define SHK_SKINNY(NB)                                                                        \
  gemm_skinny_kernel<NB><<<mb, kSkinnyWaves * kWave, 0, s>>>(ap, lda, n, k, wp, kt, m, bias, \
                                                             out, ldo, of, accumulate, vec)
  if (n <= 16)
    SHK_SKINNY(1);
  else if (n <= 32)
    SHK_SKINNY(2);
  else if (n <= 48)
    SHK_SKINNY(3);
  else
    SHK_SKINNY(4);
#undef SHK_SKINNY
  SHK_LAUNCH_CHECK("gemm_bf16");
  return 0;
}
