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
// gemm_skinny_kernel: for few tokens (decode).  One workgroup of 4, 8 or 16
// wavefronts per block of 16 weight rows; the wavefronts take the k-tiles
// round-robin and their partial sums are added in a fixed order through LDS.
// The weights are read exactly once from HBM; accumulation is float32.
#include <cstdlib>

#include "api.h"
#include "common.h"

namespace shk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
// 16 bytes as the compiler's own vector type: copies of it are loads and stores,
// where copies of HIP's uint4 struct can end up as memcpy through scratch memory
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

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

constexpr int kSkinnyBatch = 2;  // k-tiles a wavefront has in flight per buffer

// One batch of operands: kSkinnyBatch weight tiles and the matching activations.
// (RB = 2 for the gated variant: the tiles of a gate block and of its up block.)
template <int NB, int RB>
struct SkinnyBatch {
  Frag w[kSkinnyBatch][RB];
  Frag x[kSkinnyBatch][NB];
  uint32_t keep[kSkinnyBatch];  // all ones, or zero where x[u] lies beyond the matrix
};

__device__ __forceinline__ float silu(float g) { return g / (1.f + __expf(-g)); }

// The activation of a gated product's gate: kActSilu, or the tanh form of GELU,
// 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) = g / (1 + exp(-2 u)).  Gated
// kernels get the code in the argument that other products use for `accumulate`
// (a gated product never accumulates).
constexpr int kActSilu = 1, kActGeluTanh = 2;
__device__ __forceinline__ float gate_act(float g, int act) {
  if (act == kActGeluTanh) {
    const float u = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return g / (1.f + __expf(-2.f * u));
  }
  return silu(g);
}

template <int NB, int RB>
__device__ __forceinline__ void skinny_load(SkinnyBatch<NB, RB>& b, const uint4* __restrict__ wrow,
                                            const bf16* __restrict__ a, int lda, int n, int k,
                                            int ktiles, int t, int step, int j, int kg, bool vec,
                                            int blocks) {
#pragma unroll
  for (int u = 0; u < kSkinnyBatch; ++u) {
    const int tt = t + u * step;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      b.w[u][rb].u = make_uint4(0, 0, 0, 0);
      // weights are read once: a non-temporal load keeps them from displacing
      // the activations in the caches
      if (tt < ktiles && rb < blocks) {
        const uint4* p = wrow + (static_cast<size_t>(rb) * ktiles + tt) * kWave;
        b.w[u][rb].u.x = __builtin_nontemporal_load(&p->x);
        b.w[u][rb].u.y = __builtin_nontemporal_load(&p->y);
        b.w[u][rb].u.z = __builtin_nontemporal_load(&p->z);
        b.w[u][rb].u.w = __builtin_nontemporal_load(&p->w);
      }
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      b.x[u][nb] = load_act(a, lda, n, k, nb * 16 + j, tt * 32 + kg * 8, vec);
  }
}

// The same batch without a branch, for 16-byte aligned rows with k % 8 == 0
// (the usual case): every address is clamped into the matrices and what lies
// beyond them is zeroed afterwards.  A load under a condition would make the
// compiler wait, at every use of an operand, for all loads in flight, the next
// batch's included.  arow[nb]: the lane's activation row (token nb*16 + j,
// clamped to the last token), at column kg*8 when k >= 32.
template <int NB, int RB>
__device__ __forceinline__ void skinny_load_aligned(SkinnyBatch<NB, RB>& b,
                                                    const uint4* __restrict__ wrow,
                                                    const bf16* const (&arow)[NB], int k,
                                                    int ktiles, int t, int step, int kg,
                                                    int blocks) {
#pragma unroll
  for (int u = 0; u < kSkinnyBatch; ++u) {
    const int tt = t + u * step;
    const int ttc = tt < ktiles ? tt : ktiles - 1;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      // a block beyond the matrix reads block 0 again; its rows are never written
      const int rbc = rb < blocks ? rb : 0;
      const uint4* p = wrow + (static_cast<size_t>(rbc) * ktiles + ttc) * kWave;
      b.w[u][rb].u.x = __builtin_nontemporal_load(&p->x);
      b.w[u][rb].u.y = __builtin_nontemporal_load(&p->y);
      b.w[u][rb].u.z = __builtin_nontemporal_load(&p->z);
      b.w[u][rb].u.w = __builtin_nontemporal_load(&p->w);
    }
    const int col = tt * 32 + kg * 8;
    const bool inside = col < k;  // false for every tile at or beyond ktiles as well
    b.keep[u] = inside ? ~0u : 0u;  // applied when the operand is used, not while it travels
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      b.x[u][nb].u = *reinterpret_cast<const uint4*>(arow[nb] + (inside ? col : 0));
    }
  }
}

// WAVES wavefronts per workgroup share one block of 16 weight rows and take
// its k-tiles round-robin (wavefront w: tiles w, w + WAVES, ...), so the
// workgroup reads contiguous stretches of the block.  Each wavefront keeps two
// batches of tiles in registers: the next batch is in flight while the current
// one is multiplied.  The host picks WAVES so that about 4096 wavefronts or
// more are in flight whatever the number of rows.
//
// MODE kGated: the weight holds a gated feed-forward's two matrices interleaved
// by blocks of 16 rows (block 2b: rows 16b.. of the gate matrix, block 2b+1: the
// same rows of the up matrix).  A workgroup multiplies both blocks and writes
// silu(gate) * up: out[token][16b + row], `m` being the width of that output.
// MODE kPair: a workgroup owns two consecutive blocks of rows, so that every
// activation it loads feeds two multiplications.
constexpr int kSingle = 0, kGated = 1, kPair = 2;

template <int NB, int WAVES, int MODE>
__global__ void __launch_bounds__(WAVES* kWave)
    gemm_skinny_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                       const uint4* __restrict__ wt, int ktiles, int m,
                       const float* __restrict__ bias, void* __restrict__ out, int ldo,
                       int out_f32, int accumulate, int vec, int ksplit) {
  constexpr bool GATED = MODE == kGated;
  constexpr int RB = MODE == kSingle ? 1 : 2;
  __shared__ float red[WAVES][RB][NB][kWave][4];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int mb = blockIdx.x;  // block of 16 output rows (kPair: of 32)
  const int z = blockIdx.y;   // which share of k (ksplit workgroups per block)
  const int j = lane % 16, kg = lane / 16;
  const uint4* wrow = wt + static_cast<size_t>(mb) * RB * ktiles * kWave + lane;
  // weight blocks of 16 rows that exist for this workgroup (the last pair may be half)
  const int blocks = MODE == kPair ? ((m + 15) / 16 - mb * 2 >= 2 ? 2 : 1) : RB;

  f32x4 acc[RB][NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[rb][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // k-tile t belongs to wavefront (t % (WAVES * ksplit)) of the block's ksplit workgroups
  const int lanes_k = WAVES * ksplit;  // wavefronts that share the block's k-tiles
  const int kStride = kSkinnyBatch * lanes_k;
  const int t0 = z * WAVES + wave;
  auto multiply = [&](const SkinnyBatch<NB, RB>& bt, bool masked) {
#pragma unroll
    for (int u = 0; u < kSkinnyBatch; ++u)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        Frag x = bt.x[u][b];
        if (masked) {
          const uint32_t keep = bt.keep[u];
          x.u = make_uint4(x.u.x & keep, x.u.y & keep, x.u.z & keep, x.u.w & keep);
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
          acc[rb][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bt.w[u][rb].v, x.v, acc[rb][b], 0,
                                                               0, 0);
      }
  };
  // Two batches of tiles in registers: one is in flight while the other is multiplied.
  SkinnyBatch<NB, RB> ping, pong;
  if (vec) {
    const bf16* arow[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const int token = nb * 16 + j < n ? nb * 16 + j : n - 1;
      arow[nb] = a + static_cast<size_t>(token) * lda;
    }
    auto load = [&](SkinnyBatch<NB, RB>& bt, int t) {
      skinny_load_aligned<NB, RB>(bt, wrow, arow, k, ktiles, t, lanes_k, kg, blocks);
      // the loads go out here, before the other batch's multiplications, not among them
      __builtin_amdgcn_sched_barrier(0);
    };
    // every step of the loop issues one batch of loads and multiplies the other
    int t = t0;
    load(ping, t);
    for (; t + 2 * kStride < ktiles; t += 2 * kStride) {
      load(pong, t + kStride);
      multiply(ping, true);
      load(ping, t + 2 * kStride);
      multiply(pong, true);
    }
    if (t + kStride < ktiles) {
      load(pong, t + kStride);
      multiply(ping, true);
      multiply(pong, true);
    } else {
      multiply(ping, true);
    }
  } else {
    skinny_load<NB, RB>(ping, wrow, a, lda, n, k, ktiles, t0, lanes_k, j, kg, false, blocks);
    for (int t = t0; t < ktiles; t += kStride) {
      if (t + kStride < ktiles)
        skinny_load<NB, RB>(pong, wrow, a, lda, n, k, ktiles, t + kStride, lanes_k, j, kg, false,
                            blocks);
      multiply(ping, false);
      ping = pong;
    }
  }

#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][rb][b][lane][r] = acc[rb][b][r];
  __syncthreads();

  // Element e of the block's 16 x (16 * NB) outputs: accumulator b = e / 256,
  // lane (e % 256) / 4, register r = e % 4.  Lane (j, kg) holds rows kg*4 + r
  // for token b*16 + j.  The wavefronts' partial sums are added in wavefront order.
  constexpr int kOutBlocks = MODE == kPair ? 2 : 1;  // blocks of output rows per workgroup
  for (int e = threadIdx.x; e < kOutBlocks * NB * 256; e += WAVES * kWave) {
    const int ob = e / (NB * 256), b = (e / 256) % NB, ln = (e % 256) / 4, r = e % 4;
    const int token = b * 16 + ln % 16;
    const int row = (mb * kOutBlocks + ob) * 16 + (ln / 16) * 4 + r;
    if (token >= n || row >= m) continue;
    float v = red[0][ob][b][ln][r], up = 0.f;
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][ob][b][ln][r];
    if (ksplit > 1) {
      // this workgroup's share of k: a float32 partial sum, [ksplit][n][m], that the
      // kernel which reads the product adds up in order
      static_cast<float*>(out)[(static_cast<size_t>(z) * n + token) * ldo + row] = v;
      continue;
    }
    if (GATED) {
      up = red[0][RB - 1][b][ln][r];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) up += red[w][RB - 1][b][ln][r];
    }
    if (GATED) v = gate_act(v, accumulate) * up;
    if (bias) v += bias[row];
    const size_t idx = static_cast<size_t>(token) * ldo + row;
    if (out_f32) {
      float* o = static_cast<float*>(out);
      o[idx] = (accumulate && !GATED) ? o[idx] + v : v;
    } else {
      static_cast<bf16*>(out)[idx] = from_float<bf16>(v);
    }
  }
}

// gemm_mid_kernel: for 17 to 64 tokens.  The skinny kernel would fetch the
// activations once per block of 16 weight rows, which at this many tokens is
// several times the weight traffic.  Here a workgroup of WAVES wavefronts owns
// WAVES blocks of weight rows (one per wavefront; a gate and an up block when
// GATED) and walks k in stages of 128: the stage's activations are staged once
// in LDS in operand layout and shared by all wavefronts, while each wavefront
// streams its own weight tiles straight into registers (nobody else needs
// them).  Both are double-buffered.  ksplit > 1 shares k among workgroups,
// which leave float32 partial sums [ksplit][n][m] for the reading kernel.
constexpr int kMidTiles = 4;  // k-tiles per stage

template <int NB, int WAVES, bool GATED>
__global__ void __launch_bounds__(WAVES* kWave)
    gemm_mid_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                    const uint4* __restrict__ wt, int ktiles, int m,
                    const float* __restrict__ bias, void* __restrict__ out, int ldo, int out_f32,
                    int accumulate, int vec, int ksplit) {
  constexpr int RB = GATED ? 2 : 1;
  __shared__ uint4 act[2][NB][kMidTiles][kWave];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int j = lane % 16, kg = lane / 16;
  const int ob = blockIdx.x * WAVES + wave;  // block of 16 output rows of this wavefront
  const int oblocks = (m + 15) / 16;
  const bool have_rows = ob < oblocks;
  const uint4* wrow = wt + static_cast<size_t>(have_rows ? ob : 0) * RB * ktiles * kWave + lane;

  const int nstages = (ktiles + kMidTiles - 1) / kMidTiles;
  const int per = (nstages + ksplit - 1) / ksplit;
  const int st_begin = blockIdx.y * per;
  const int st_end = st_begin + per < nstages ? st_begin + per : nstages;

  f32x4 acc[RB][NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[rb][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  constexpr int kItems = NB * kMidTiles * kWave;           // activation fragments-lanes per stage
  constexpr int kPerThread = (kItems + WAVES * kWave - 1) / (WAVES * kWave);
  Frag wcur[RB][kMidTiles], wnext[RB][kMidTiles];
  uint4 areg[kPerThread];

  auto load_weights = [&](Frag (&w)[RB][kMidTiles], int st) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int t = 0; t < kMidTiles; ++t) {
        const int tt = st * kMidTiles + t;
        w[rb][t].u = make_uint4(0, 0, 0, 0);
        if (have_rows && tt < ktiles) {
          const uint4* p = wrow + (static_cast<size_t>(rb) * ktiles + tt) * kWave;
          w[rb][t].u.x = __builtin_nontemporal_load(&p->x);
          w[rb][t].u.y = __builtin_nontemporal_load(&p->y);
          w[rb][t].u.z = __builtin_nontemporal_load(&p->z);
          w[rb][t].u.w = __builtin_nontemporal_load(&p->w);
        }
      }
  };
  auto load_acts = [&](int st) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int item = tid + i * WAVES * kWave;  // (b * kMidTiles + t) * 64 + lane
      areg[i] = make_uint4(0, 0, 0, 0);
      if (item < kItems) {
        const int ln = item % kWave, f = item / kWave, t = f % kMidTiles, b = f / kMidTiles;
        areg[i] = load_act(a, lda, n, k, b * 16 + ln % 16, (st * kMidTiles + t) * 32 + (ln / 16) * 8,
                           vec).u;
      }
    }
  };
  auto store_acts = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int item = tid + i * WAVES * kWave;
      if (item < kItems) (&act[buf][0][0][0])[item] = areg[i];
    }
  };

  if (st_begin < st_end) {
    load_weights(wcur, st_begin);
    load_acts(st_begin);
    store_acts(0);
  }
  __syncthreads();
  for (int st = st_begin; st < st_end; ++st) {
    const int buf = (st - st_begin) & 1;
    const bool more = st + 1 < st_end;
    if (more) {
      load_weights(wnext, st + 1);
      load_acts(st + 1);
    }
#pragma unroll
    for (int t = 0; t < kMidTiles; ++t)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        Frag x;
        x.u = act[buf][b][t][lane];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
          acc[rb][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wcur[rb][t].v, x.v, acc[rb][b], 0, 0, 0);
      }
    if (more) store_acts(buf ^ 1);
    __syncthreads();
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int t = 0; t < kMidTiles; ++t) wcur[rb][t] = wnext[rb][t];
  }
  if (!have_rows) return;

  // lane (j, kg) of accumulator b: token b*16 + j, rows ob*16 + kg*4 + r
  const int row0 = ob * 16 + kg * 4;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int token = b * 16 + j;
    if (token >= n || row0 >= m) continue;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = GATED ? gate_act(acc[0][b][r], accumulate) * acc[RB - 1][b][r] : acc[0][b][r];
      if (bias && row0 + r < m) v[r] += bias[row0 + r];
    }
    if (ksplit > 1) {
      float* o = static_cast<float*>(out) + (static_cast<size_t>(blockIdx.y) * n + token) * ldo + row0;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (row0 + r < m) o[r] = v[r];
      continue;
    }
    const size_t idx = static_cast<size_t>(token) * ldo + row0;
    if (out_f32) {
      float* o = static_cast<float*>(out) + idx;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (row0 + r < m) o[r] = (accumulate && !GATED) ? o[r] + v[r] : v[r];
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

// What a wavefront of the large kernels does with its WM x WN accumulator tiles:
// lane (j, kg) of tile (i, jn) holds token tok_first + jn*16 + j, rows
// (block_first + i)*16 + kg*4 + r.  Gated: weight blocks come in (gate, up) pairs
// that make one block of output rows.  share: which float32 partial sum [share][n][m].
template <int WM, int WN, bool GATED>
__device__ __forceinline__ void big_store(const f32x4 (&acc)[WM][WN], int lane, int tok_first,
                                          int block_first, int n, int m,
                                          const float* __restrict__ bias, void* __restrict__ out,
                                          int ldo, int out_f32, int accumulate, int share) {
  const int j = lane % 16, kg = lane / 16;
  // the lane's bias values, fetched once for all its tokens
  float add[GATED ? 1 : WM][4];
  if (!GATED) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = (block_first + i) * 16 + kg * 4 + r;
        add[i][r] = (bias && row < m) ? bias[row] : 0.f;
      }
  }
#pragma unroll
  for (int jn = 0; jn < WN; ++jn) {
    const int token = tok_first + jn * 16 + j;
    if (token >= n) continue;
#pragma unroll
    for (int i = 0; i < WM; i += (GATED ? 2 : 1)) {
      // gated: weight blocks come in (gate, up) pairs that make one block of output rows
      const int row0 = (GATED ? (block_first + i) / 2 : block_first + i) * 16 + kg * 4;
      if (row0 >= m) continue;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] = GATED ? gate_act(acc[i][jn][r], accumulate) * acc[i + (GATED ? 1 : 0)][jn][r]
                     : acc[i][jn][r] + add[GATED ? 0 : i][r];
      }
      const size_t idx = (static_cast<size_t>(share) * n + token) * ldo + row0;
      if (out_f32) {
        float* o = static_cast<float*>(out) + idx;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (row0 + r < m) o[r] = (accumulate && !GATED) ? o[r] + v[r] : v[r];
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

// gemm_big_kernel: for many tokens (prompt portions).  A workgroup of 4 or 8
// wavefronts computes a tile of weight rows x tokens, each wavefront a part of
// it as WM x WN MFMA tiles.  Per stage of k, the weights' tiles (already in
// operand layout) and the activations (re-laid on the way) are staged in LDS
// "fragment-major": the 16 bytes of lane l of a fragment sit at l * 16, so every
// LDS access is a conflict-free 128-bit access.  Two LDS buffers alternate, and
// the loads of the next two stages are in flight (in registers) while a stage is
// multiplied.

constexpr int kDies = 8;        // accelerator dies (XCDs), each with an L2 of its own
constexpr int kDieUnits = 32;  // compute units per die

// The tile of a workgroup of the large kernels; false: none (the grid is padded).
__device__ __forceinline__ bool big_tile(int tiles_x, int tiles_y, int by_die, int& tile_x, int& tile_y) {
  // Which tile: workgroups are handed to the chip's eight dies (each with its own
  // L2) in turn, workgroup p to die p % 8.  The tiles are therefore dealt out in
  // blocks of 32 (up to 8 token tiles of 32 / that many weight tiles) and block B goes to
  // die B % 8, whose 32 compute units then work on tiles that share their
  // operands: the die's L2 serves most of their loads.
  // With fewer tiles (by_die == 2 * dx) the grid of tiles is cut into dx x 8/dx
  // rectangles, one for each die, where the numbers of tiles allow that; else
  // (by_die == 0) the tiles are taken in plain order.
  tile_x = blockIdx.x % tiles_x, tile_y = blockIdx.x / tiles_x;
  if (by_die > 1) {
    const int die = blockIdx.x % kDies, turn = blockIdx.x / kDies;
    const int dx = by_die / 2, wide = tiles_x / dx, high = tiles_y / (kDies / dx);
    tile_x = (die % dx) * wide + turn % wide;
    tile_y = (die / dx) * high + turn / wide;
  } else if (by_die) {
    const int die = blockIdx.x % kDies, turn = blockIdx.x / kDies;
    const int block_y = tiles_y < 8 ? tiles_y : 8, block_x = kDieUnits / block_y;
    const int blocks_x = (tiles_x + block_x - 1) / block_x;
    const int block = (turn / kDieUnits) * kDies + die, within = turn % kDieUnits;
    tile_x = (block % blocks_x) * block_x + within / block_y;
    tile_y = (block / blocks_x) * block_y + within % block_y;
    if (within >= block_x * block_y) return false;
  }
  return tile_x < tiles_x && tile_y < tiles_y;
}

// GM x GN wavefronts per workgroup, each with WM x WN MFMA tiles (16 x 16): the
// workgroup covers 16*GM*WM weight rows x 16*GN*WN tokens.  KS: MFMA steps (32 of
// k) per stage.  The stages live in dynamic LDS, [buffer][fragment][lane].
template <int GM, int GN, int WM, int WN, int KS, bool GATED>
__global__ void __launch_bounds__(GM* GN* kWave)
    __attribute__((amdgpu_waves_per_eu(GM* GN >= 8 || WM * WN <= 16 ? 2 : 1)))
    gemm_big_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                    const uint4* __restrict__ wt, int ktiles, int m,
                    const float* __restrict__ bias, void* __restrict__ out, int ldo, int out_f32,
                    int accumulate, int vec, int ksplit, int tiles_x, int tiles_y, int by_die) {
  constexpr int kWaves = GM * GN;
  constexpr int kWFrags = GM * WM * KS, kAFrags = GN * WN * KS;  // fragments per stage
  constexpr int kFrags = kWFrags + kAFrags;
  extern __shared__ uint4 stage_mem[];
  auto stage = [&](int buf, int frag) -> uint4* { return stage_mem + (buf * kFrags + frag) * kWave; };
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / GN, wn = wave % GN;  // place of the wavefront in the workgroup's tile
  int tile_x, tile_y;
  if (!big_tile(tiles_x, tiles_y, by_die, tile_x, tile_y)) return;
  const int mb0 = tile_x * (GM * WM);  // first block of 16 weight rows
  const int tok0 = tile_y * (16 * GN * WN);
  // blocks of 16 weight rows; a gated weight has two per 16 output rows
  const int mblocks = (GATED ? 2 : 1) * ((m + 15) / 16);
  // blockIdx.y: which share of the k stages (ksplit workgroups per tile leave float32
  // partial sums [ksplit][n][m] that the reading kernel adds up)
  const int all_stages = (ktiles + KS - 1) / KS;
  const int per_split = (all_stages + ksplit - 1) / ksplit;
  const int st_first = blockIdx.y * per_split;
  const int nstages = st_first + per_split < all_stages ? st_first + per_split : all_stages;

  f32x4 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int jn = 0; jn < WN; ++jn) acc[i][jn] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Fragment f of an operand is (block of 16 rows f / KS, MFMA step f % KS); wavefront w
  // moves fragments w, w + kWaves, ...
  constexpr int kWPer = (kWFrags + kWaves - 1) / kWaves, kAPer = (kAFrags + kWaves - 1) / kWaves;
  uint4 wreg[kWPer], areg[kAPer];
  auto load_stage = [&](int st) {
#pragma unroll
    for (int i = 0; i < kWPer; ++i) {
      const int f = wave + kWaves * i, rb = f / KS, kt = st * KS + f % KS;
      wreg[i] = make_uint4(0, 0, 0, 0);
      if (f < kWFrags && mb0 + rb < mblocks && kt < ktiles)
        wreg[i] = wt[(static_cast<size_t>(mb0 + rb) * ktiles + kt) * kWave + lane];
    }
#pragma unroll
    for (int i = 0; i < kAPer; ++i) {
      const int f = wave + kWaves * i, rb = f / KS, kt = st * KS + f % KS;
      areg[i] = make_uint4(0, 0, 0, 0);
      if (f < kAFrags)
        areg[i] = load_act(a, lda, n, k, tok0 + rb * 16 + lane % 16, kt * 32 + (lane / 16) * 8, vec).u;
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kWPer; ++i)
      if (wave + kWaves * i < kWFrags) stage(buf, wave + kWaves * i)[lane] = wreg[i];
#pragma unroll
    for (int i = 0; i < kAPer; ++i)
      if (wave + kWaves * i < kAFrags) stage(buf, kWFrags + wave + kWaves * i)[lane] = areg[i];
  };

  // every fragment of the stage is requested from LDS before the first multiplication,
  // so that the later reads travel under the earlier multiplications
  auto multiply = [&](int buf) {
    u32x4 af[KS][WN], wf[KS][WM];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int jn = 0; jn < WN; ++jn)
        af[ks][jn] = *reinterpret_cast<const u32x4*>(stage(buf, kWFrags + (wn * WN + jn) * KS + ks) + lane);
#pragma unroll
      for (int i = 0; i < WM; ++i)
        wf[ks][i] = *reinterpret_cast<const u32x4*>(stage(buf, (wm * WM + i) * KS + ks) + lane);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int jn = 0; jn < WN; ++jn)
          acc[i][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, wf[ks][i]), __builtin_bit_cast(bf16x8, af[ks][jn]),
              acc[i][jn], 0, 0, 0);
  };

  if (vec && kWFrags % kWaves == 0 && kAFrags % kWaves == 0) {
    // Aligned rows: every load is unconditional, its address clamped into the
    // matrices (what an activation row holds past k meets the zeros that pad the
    // weight tiles), and the loads of two stages are in flight while a stage is
    // multiplied.
    const uint4* wsrc[kWPer];
    const bf16* asrc[kAPer];
#pragma unroll
    for (int i = 0; i < kWPer; ++i) {
      const int rb = (wave + kWaves * i) / KS;
      const int block = mb0 + rb < mblocks ? mb0 + rb : mblocks - 1;
      wsrc[i] = wt + static_cast<size_t>(block) * ktiles * kWave + lane;
    }
#pragma unroll
    for (int i = 0; i < kAPer; ++i) {
      const int rb = (wave + kWaves * i) / KS;
      const int token = tok0 + rb * 16 + lane % 16;
      asrc[i] = a + static_cast<size_t>(token < n ? token : n - 1) * lda + (lane / 16) * 8;
    }
    // Two named sets of registers, not an array of two: an array indexed by the
    // loop's step would live in scratch memory.
    u32x4 even_w[kWPer], even_x[kAPer], odd_w[kWPer], odd_x[kAPer];
    auto fetch = [&](u32x4 (&hw)[kWPer], u32x4 (&hx)[kAPer], int st) {
#pragma unroll
      for (int i = 0; i < kAPer; ++i) {
        const int col = (st * KS + (wave + kWaves * i) % KS) * 32;  // + (lane / 16) * 8 in asrc
        hx[i] = *reinterpret_cast<const u32x4*>(asrc[i] + (col + (lane / 16) * 8 < k ? col : 0));
      }
#pragma unroll
      for (int i = 0; i < kWPer; ++i) {
        const int kt = st * KS + (wave + kWaves * i) % KS;
        hw[i] = *reinterpret_cast<const u32x4*>(wsrc[i] + static_cast<size_t>(kt < ktiles ? kt : 0) * kWave);
      }
      __builtin_amdgcn_sched_barrier(0);  // the loads go out before the multiplications
    };
    auto put = [&](const u32x4 (&hw)[kWPer], const u32x4 (&hx)[kAPer], int st, int buf) {
#pragma unroll
      for (int i = 0; i < kWPer; ++i)
        *reinterpret_cast<u32x4*>(stage(buf, wave + kWaves * i) + lane) = hw[i];
#pragma unroll
      for (int i = 0; i < kAPer; ++i) {
        // a k-tile past the last one (the stage is not full) must contribute nothing
        const uint32_t keep = st * KS + (wave + kWaves * i) % KS < ktiles ? ~0u : 0u;
        *reinterpret_cast<u32x4*>(stage(buf, kWFrags + wave + kWaves * i) + lane) = hx[i] & keep;
      }
    };
    // stage st is multiplied from LDS buffer st % 2 while the loads of stages
    // st + 1 (issued a step ago) and st + 2 (issued now) are in flight
    fetch(even_w, even_x, st_first);
    fetch(odd_w, odd_x, st_first + 1);
    put(even_w, even_x, st_first, 0);
    __syncthreads();
    // The loop's body has no branch: with one, the compiler moves loads behind it,
    // next to their use, and nothing is in flight any more.
    int st = st_first;
    for (; st + 2 < nstages; st += 2) {
      fetch(even_w, even_x, st + 2);
      multiply(0);
      put(odd_w, odd_x, st + 1, 1);
      __syncthreads();
      fetch(odd_w, odd_x, st + 3);
      multiply(1);
      put(even_w, even_x, st + 2, 0);
      __syncthreads();
    }
    if (st < nstages) multiply(0);
    if (st + 1 < nstages) {
      put(odd_w, odd_x, st + 1, 1);
      __syncthreads();
      multiply(1);
    }
  } else {
    load_stage(st_first);
    store_stage(0);
    __syncthreads();
    for (int st = st_first; st < nstages; ++st) {
      const int buf = (st - st_first) & 1;
      if (st + 1 < nstages) load_stage(st + 1);
      multiply(buf);
      if (st + 1 < nstages) store_stage(buf ^ 1);
      __syncthreads();
    }
  }

  big_store<WM, WN, GATED>(acc, lane, tok0 + wn * WN * 16, mb0 + wm * WM, n, m, bias, out, ldo, out_f32,
                           accumulate, blockIdx.y);
}

// gemm_big_lds_kernel: the same tiles, for aligned activations and whole stages
// of k, with the operands loaded from global memory straight into LDS
// (global_load_lds_dwordx4: lane l's 16 bytes land at l * 16 of the fragment, the
// layout above) instead of through registers.  Four stage buffers (three for the
// largest stages); the loads of the next two stages (one) are in flight while a
// stage is multiplied, and one barrier
// per stage both publishes a stage and frees the buffer of the stage before.
// The compiler cannot see when another wavefront's load has landed: every
// wavefront waits for its own loads of the stage (s_waitcnt vmcnt, counting the
// loads issued since) before the barrier.  Each buffer is an LDS array of its
// own, so that the compiler's own bookkeeping tells the buffers apart and adds
// no wait for loads into another one.
#define SHK_LOAD_TO_LDS(gptr, lptr)                                                        \
  __builtin_amdgcn_global_load_lds(                                                       \
      reinterpret_cast<const __attribute__((address_space(1))) void*>(                    \
          reinterpret_cast<uintptr_t>(gptr)),                                             \
      (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters at their maxima)
#define SHK_WAIT_LOADS(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14))

template <int GM, int GN, int WM, int WN, int KS, bool GATED>
__global__ void __launch_bounds__(GM* GN* kWave) __attribute__((amdgpu_waves_per_eu(GM * GN >= 16 ? 4 : 2)))
    gemm_big_lds_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                        const uint4* __restrict__ wt, int ktiles, int m,
                        const float* __restrict__ bias, void* __restrict__ out, int ldo,
                        int out_f32, int accumulate, int ksplit, int tiles_x, int tiles_y,
                        int by_die) {
  constexpr int kWaves = GM * GN;
  constexpr int kWFrags = GM * WM * KS, kAFrags = GN * WN * KS, kFrags = kWFrags + kAFrags;
  constexpr int kWPer = kWFrags / kWaves, kAPer = kAFrags / kWaves;
  constexpr int kLoads = kWPer + kAPer;  // per wavefront and stage
  static_assert(kWFrags % kWaves == 0 && kAFrags % kWaves == 0, "fragments must divide among the wavefronts");
  // four stage buffers where they fit into the 160 KiB of LDS, else three
  constexpr int NS = 4 * kFrags * kWave * 16 <= 160 * 1024 ? 4 : 3;
  static_assert(NS * kFrags * kWave * 16 <= 160 * 1024, "three stages must fit in LDS");
  __shared__ u32x4 stage0[kFrags][kWave], stage1[kFrags][kWave], stage2[kFrags][kWave],
      stage3[NS == 4 ? kFrags : 1][kWave];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / GN, wn = wave % GN;
  int tile_x, tile_y;
  if (!big_tile(tiles_x, tiles_y, by_die, tile_x, tile_y)) return;
  const int mb0 = tile_x * (GM * WM);
  const int tok0 = tile_y * (16 * GN * WN);
  const int mblocks = (GATED ? 2 : 1) * ((m + 15) / 16);
  const int all_stages = ktiles / KS;  // the host sends only whole stages here
  const int per_split = (all_stages + ksplit - 1) / ksplit;
  const int st_first = blockIdx.y * per_split;
  const int nstages = st_first + per_split < all_stages ? st_first + per_split : all_stages;

  f32x4 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int jn = 0; jn < WN; ++jn) acc[i][jn] = f32x4{0.f, 0.f, 0.f, 0.f};

  // what this wavefront loads: fragments wave, wave + kWaves, ... of either operand,
  // from rows clamped into the matrices (their products are never stored)
  const uint4* wsrc[kWPer];
  const bf16* asrc[kAPer];
#pragma unroll
  for (int i = 0; i < kWPer; ++i) {
    const int rb = (wave + kWaves * i) / KS;
    const int block = mb0 + rb < mblocks ? mb0 + rb : mblocks - 1;
    wsrc[i] = wt + static_cast<size_t>(block) * ktiles * kWave + lane;
  }
  // Activations, 1 KiB per load.  With stages of 64 of k (KS == 2) a load takes 8
  // tokens x 128 bytes, lane l the 16 bytes at (token l % 8, chunk l / 8): whole cache
  // lines, where a fragment of 16 tokens x 64 bytes uses half of each line it touches
  // and asks the L2 twice as often.  Unit u holds tokens (u / 2) * 16 + (u % 2) * 8 ...
  // in lane order; lane (j, kg) of the operand of step ks finds its 16 bytes in unit
  // 2 * block + j / 8 at place j % 8 + 8 * (kg + 4 * ks): groups of 8 lanes read 128
  // contiguous bytes, without bank conflicts.
  constexpr bool kUnits = KS == 2;
#pragma unroll
  for (int i = 0; i < kAPer; ++i) {
    const int f = wave + kWaves * i;
    const int token = kUnits ? tok0 + (f / 2) * 16 + (f % 2) * 8 + lane % 8 : tok0 + (f / KS) * 16 + lane % 16;
    asrc[i] = a + static_cast<size_t>(token < n ? token : n - 1) * lda + (kUnits ? lane / 8 : lane / 16) * 8;
  }
  const int xunit = (lane % 16) / 8, xplace = lane % 8 + 8 * (lane / 16);
  auto load = [&](u32x4 (&buf)[kFrags][kWave], int st) {
    const int stage = st < all_stages ? st : 0;  // past the end: any stage, never multiplied
#pragma unroll
    for (int i = 0; i < kAPer; ++i) {
      // (+ the lane's chunk, which is in asrc)
      const int col = kUnits ? stage * 64 : (stage * KS + (wave + kWaves * i) % KS) * 32;
      SHK_LOAD_TO_LDS(asrc[i] + (col + (kUnits ? lane / 8 : lane / 16) * 8 < k ? col : 0),
                      &buf[kWFrags + wave + kWaves * i][0]);
    }
#pragma unroll
    for (int i = 0; i < kWPer; ++i) {
      const int kt = stage * KS + (wave + kWaves * i) % KS;
      SHK_LOAD_TO_LDS(wsrc[i] + static_cast<size_t>(kt) * kWave, &buf[wave + kWaves * i][0]);
    }
  };
  auto multiply = [&](const u32x4 (&buf)[kFrags][kWave]) {
    u32x4 af[KS][WN], wf[KS][WM];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int jn = 0; jn < WN; ++jn)
        af[ks][jn] = kUnits ? buf[kWFrags + (wn * WN + jn) * 2 + xunit][xplace + 32 * ks]
                            : buf[kWFrags + (wn * WN + jn) * KS + ks][lane];
#pragma unroll
      for (int i = 0; i < WM; ++i) wf[ks][i] = buf[(wm * WM + i) * KS + ks][lane];
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int jn = 0; jn < WN; ++jn)
          acc[i][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, wf[ks][i]), __builtin_bit_cast(bf16x8, af[ks][jn]),
              acc[i][jn], 0, 0, 0);
  };
  // The stage in `now` has landed for every wavefront once each has waited for its
  // own loads (the younger stages may stay in flight) and met the others; after the
  // barrier nobody reads the stage before any more, so its buffer takes new loads.
#define SHK_LDS_STEP(now, refill, st_refill)  \
  SHK_WAIT_LOADS((NS - 2) * kLoads);          \
  asm volatile("" ::: "memory");              \
  __builtin_amdgcn_s_barrier();               \
  asm volatile("" ::: "memory");              \
  load(refill, st_refill);                    \
  __builtin_amdgcn_sched_barrier(0);          \
  multiply(now);
  int st = st_first;
  if constexpr (NS == 4) {
    load(stage0, st_first);
    load(stage1, st_first + 1);
    load(stage2, st_first + 2);
    for (; st + 3 < nstages; st += 4) {
      SHK_LDS_STEP(stage0, stage3, st + 3)
      SHK_LDS_STEP(stage1, stage0, st + 4)
      SHK_LDS_STEP(stage2, stage1, st + 5)
      SHK_LDS_STEP(stage3, stage2, st + 6)
    }
    if (st < nstages) { SHK_LDS_STEP(stage0, stage3, st + 3) }
    if (st + 1 < nstages) { SHK_LDS_STEP(stage1, stage0, st + 4) }
    if (st + 2 < nstages) { SHK_LDS_STEP(stage2, stage1, st + 5) }
  } else {
    load(stage0, st_first);
    load(stage1, st_first + 1);
    for (; st + 2 < nstages; st += 3) {
      SHK_LDS_STEP(stage0, stage2, st + 2)
      SHK_LDS_STEP(stage1, stage0, st + 3)
      SHK_LDS_STEP(stage2, stage1, st + 4)
    }
    if (st < nstages) { SHK_LDS_STEP(stage0, stage2, st + 2) }
    if (st + 1 < nstages) { SHK_LDS_STEP(stage1, stage0, st + 3) }
  }
#undef SHK_LDS_STEP
  SHK_WAIT_LOADS(0);  // no load may arrive in LDS that the workgroup has given back

  big_store<WM, WN, GATED>(acc, lane, tok0 + wn * WN * 16, mb0 + wm * WM, n, m, bias, out, ldo, out_f32,
                           accumulate, blockIdx.y);
}


// gemm_stream_kernel: for 17 to 64 tokens whose rows are 16-byte aligned with
// k % 8 == 0.  Such a product is bound by the stream of weights, like the skinny
// one, but its activations (up to 64 x k) are too many to fetch once per block of
// weight rows.  What was measured on the chip shapes this kernel: a wavefront
// pulls about 5 GB/s from memory however many loads it keeps in flight, and a
// compute unit about 50 GB/s, so the stream needs 8 or more wavefronts on every
// compute unit and the same work on each.  Hence one block of 16 weight rows per
// wavefront (a gate block and its up block go to neighbouring wavefronts, which
// combine their sums through LDS at the end), and workgroups of `waves` = 4 to 16
// wavefronts, a number the host picks so that the launch is one workgroup for
// each compute unit (or a whole number of rounds of them).
//
// k is walked in stages of kStreamTiles tiles.  Each wavefront streams its own
// weight tiles straight into registers with non-temporal loads (nobody else needs
// them); the stage's activations go from global memory straight into LDS in
// units of whole cache lines, once for the workgroup: its NB * kStreamTiles units
// are dealt out to the wavefronts, APER fetches each (where waves * APER exceeds
// the units, some are fetched twice, into the same place).  Three stage buffers
// and three sets of weight registers: while stage s is multiplied, the loads of
// stages s + 1 and s + 2 are in flight, and one barrier per stage both publishes
// a stage and frees the buffer of the stage before.  No load sits under a
// condition: addresses are clamped into the matrices, tokens beyond n fill
// output columns that are never written, columns beyond k meet the zeros that
// pad the weight tiles, and tiles beyond the last one are not multiplied (only
// the last stage of k can have such).  ksplit > 1 shares the stages among
// workgroups, which leave float32 partial sums [ksplit][n][m] for the reading
// kernel.
constexpr int kStreamTiles = 4;

template <int NB, int APER, bool GATED>
__global__ void __launch_bounds__(16 * kWave)
    gemm_stream_kernel(const bf16* __restrict__ a, int lda, int n, int k,
                       const uint4* __restrict__ wt, int ktiles, int m,
                       const float* __restrict__ bias, void* __restrict__ out, int ldo,
                       int out_f32, int accumulate, int ksplit) {
  constexpr int KT = kStreamTiles;
  constexpr int kFrags = NB * KT;      // activation fragments per stage
  constexpr int kLoads = APER + KT;    // loads per wavefront and stage
  static_assert(2 * kLoads <= 63, "the load counter holds 63");
  __shared__ u32x4 stage0[kFrags][kWave], stage1[kFrags][kWave], stage2[kFrags][kWave];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int waves = blockDim.x / kWave;
  const int j = lane % 16, kg = lane / 16;
  // blocks of 16 weight rows; a gated weight has a gate and an up block per 16 output rows
  const int wblocks = (GATED ? 2 : 1) * ((m + 15) / 16);
  const int wb = blockIdx.x * waves + wave;  // this wavefront's block
  const bool have_rows = wb < wblocks;
  // a wavefront without rows streams the last block's weights; its sums are dropped
  const u32x4* wrow = reinterpret_cast<const u32x4*>(wt) +
                      static_cast<size_t>(have_rows ? wb : wblocks - 1) * ktiles * kWave + lane;

  const int all_stages = (ktiles + KT - 1) / KT;
  const int per = (all_stages + ksplit - 1) / ksplit;
  const int st_first = blockIdx.y * per;
  const int st_end = st_first + per < all_stages ? st_first + per : all_stages;
  // the share's whole stages; the last stage of k may hold fewer than KT tiles
  const int tail_tiles = (st_end == all_stages && ktiles % KT && st_first < st_end) ? ktiles % KT : 0;
  const int full_end = tail_tiles ? st_end - 1 : st_end;

  f32x4 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // What a wavefront fetches of the stage's activations, 1 KiB at a time: unit f is
  // (token block f / KT, pair of tiles (f % KT) / 2, half of the block's tokens
  // f % 2): 8 tokens x 128 bytes, lane l taking the 16 bytes at (token l % 8,
  // chunk l / 8) - whole cache lines, where a fragment of 16 tokens x 64 bytes
  // would use half of each line it touches.  In LDS the unit lies in lane order;
  // lane (j, kg) of the operand of tile t finds its 16 bytes in unit (j / 8) at
  // place j % 8 + 8 * (kg + 4 * (t % 2)): groups of 8 lanes read 128 contiguous
  // bytes, without bank conflicts.  Beyond the last unit the first ones are
  // fetched again.
  static_assert(KT % 2 == 0, "tiles are fetched in pairs");
  const bf16* asrc[APER];
  int afrag[APER];
#pragma unroll
  for (int i = 0; i < APER; ++i) {
    int f = wave + waves * i;
    f = f < kFrags ? f : f % kFrags;
    afrag[i] = f;
    const int token = (f / KT) * 16 + (f % 2) * 8 + lane % 8;
    asrc[i] = a + static_cast<size_t>(token < n ? token : n - 1) * lda + (lane / 8) * 8;
  }
  auto fetch = [&](u32x4 (&buf)[kFrags][kWave], u32x4 (&w)[KT], int st) {
    // past the share's end: some stage that exists, never multiplied
    int stage = st < all_stages ? st : all_stages - 1;
    stage = stage < 0 ? 0 : stage;
#pragma unroll
    for (int i = 0; i < APER; ++i) {
      const int col = (stage * KT + ((afrag[i] % KT) / 2) * 2) * 32;  // + (lane / 8) * 8 in asrc
      SHK_LOAD_TO_LDS(asrc[i] + (col + (lane / 8) * 8 < k ? col : 0), &buf[afrag[i]][0]);
    }
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int tt = stage * KT + t;
      w[t] = __builtin_nontemporal_load(wrow + static_cast<size_t>(tt < ktiles ? tt : ktiles - 1) * kWave);
    }
  };
  const int xunit = j / 8, xplace = j % 8 + 8 * kg;  // where this lane's operands lie
  auto multiply = [&](const u32x4 (&buf)[kFrags][kWave], const u32x4 (&w)[KT], int tiles) {
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      if (t < tiles) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, w[t]),
              __builtin_bit_cast(bf16x8, buf[b * KT + (t / 2) * 2 + xunit][xplace + 32 * (t % 2)]), acc[b],
              0, 0, 0);
      }
    }
  };
  u32x4 w0[KT], w1[KT], w2[KT];
  // Stage `now` has landed for every wavefront once each has waited for its own
  // loads of it (the next stage's may stay in flight) and met the others; after
  // the barrier nobody reads the stage before any more, so its buffer and its
  // registers take the loads of the stage after next.
#define SHK_STREAM_STEP(buf_now, w_now, buf_fill, w_fill, st_fill, tiles) \
  SHK_WAIT_LOADS(kLoads);                                                  \
  asm volatile("" ::: "memory");                                           \
  __builtin_amdgcn_s_barrier();                                            \
  asm volatile("" ::: "memory");                                           \
  fetch(buf_fill, w_fill, st_fill);                                        \
  __builtin_amdgcn_sched_barrier(0);                                       \
  multiply(buf_now, w_now, tiles);
  fetch(stage0, w0, st_first);
  fetch(stage1, w1, st_first + 1);
  int st = st_first;
  for (; st + 3 <= full_end; st += 3) {
    SHK_STREAM_STEP(stage0, w0, stage2, w2, st + 2, KT)
    SHK_STREAM_STEP(stage1, w1, stage0, w0, st + 3, KT)
    SHK_STREAM_STEP(stage2, w2, stage1, w1, st + 4, KT)
  }
  // up to two whole stages are left, and then the one that is not whole
  const int left = full_end - st;
  if (left >= 1) { SHK_STREAM_STEP(stage0, w0, stage2, w2, st + 2, KT) }
  if (left >= 2) { SHK_STREAM_STEP(stage1, w1, stage0, w0, st + 3, KT) }
  if (tail_tiles) {
    if (left == 0) { SHK_STREAM_STEP(stage0, w0, stage2, w2, st + 2, tail_tiles) }
    if (left == 1) { SHK_STREAM_STEP(stage1, w1, stage0, w0, st + 3, tail_tiles) }
    if (left == 2) { SHK_STREAM_STEP(stage2, w2, stage1, w1, st + 4, tail_tiles) }
  }
#undef SHK_STREAM_STEP
  SHK_WAIT_LOADS(0);  // no load may arrive in LDS that the workgroup has given back

  int ob = wb;  // block of 16 output rows
  if (GATED) {
    // the wavefront of an up block hands its sums to its neighbour with the gate
    // block, through the first stage buffer: room for the sums of kFrags / NB
    // pairs at a time
    f32x4* hand = reinterpret_cast<f32x4*>(&stage0[0][0]);
    constexpr int kPairsPerPass = kFrags / NB;
    const int pair = wave / 2;
    for (int first = 0; first < waves / 2; first += kPairsPerPass) {
      __syncthreads();  // the stage buffers, or the pass before, are read no more
      const bool mine = pair >= first && pair < first + kPairsPerPass;
      if (mine && (wave & 1)) {
#pragma unroll
        for (int b = 0; b < NB; ++b) hand[((pair - first) * NB + b) * kWave + lane] = acc[b];
      }
      __syncthreads();
      if (mine && !(wave & 1)) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          const f32x4 up = hand[((pair - first) * NB + b) * kWave + lane];
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[b][r] = gate_act(acc[b][r], accumulate) * up[r];
        }
      }
    }
    if (wave & 1) return;
    ob = wb / 2;
  }
  if (!have_rows) return;

  // lane (j, kg) of accumulator b: token b*16 + j, rows ob*16 + kg*4 + r
  const int row0 = ob * 16 + kg * 4;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int token = b * 16 + j;
    if (token >= n || row0 >= m) continue;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = acc[b][r];
      if (bias && row0 + r < m) v[r] += bias[row0 + r];
    }
    if (ksplit > 1) {
      float* o = static_cast<float*>(out) + (static_cast<size_t>(blockIdx.y) * n + token) * ldo + row0;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (row0 + r < m) o[r] = v[r];
      continue;
    }
    const size_t idx = static_cast<size_t>(token) * ldo + row0;
    if (out_f32) {
      float* o = static_cast<float*>(out) + idx;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (row0 + r < m) o[r] = (accumulate && !GATED) ? o[r] + v[r] : v[r];
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

// mfma_alone_kernel: the matrix instruction by itself, a 64 x 64 x 32 block per
// wavefront and iteration from operands that stay in registers.  What it reaches is
// the ceiling of every product kernel on this chip: with random operands the power
// limit holds the clock well below the one that the published peak assumes, with
// zeros it does not.
__global__ void __launch_bounds__(4 * kWave)
    mfma_alone_kernel(const u32x4* __restrict__ operands, float* __restrict__ out, int iters) {
  const int tid = threadIdx.x;
  u32x4 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(tid + 64 * i) % 4096];
    b[i] = operands[(tid * 3 + 64 * i + 7) % 4096];
  }
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[i]),
                                                             __builtin_bit_cast(bf16x8, b[j]), acc[i][j], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) sum += acc[i][j][0] + acc[i][j][3];
  out[blockIdx.x * blockDim.x + tid] = sum;
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

// Interleaves the tiled layouts of a gate and an up matrix ([m, k] each) by
// blocks of 16 rows: wt[2b] = gate block b, wt[2b + 1] = up block b.
__global__ void interleave_blocks_kernel(const uint4* __restrict__ gate, const uint4* __restrict__ up,
                                         uint4* __restrict__ wt, size_t block_vecs) {
  const size_t b = blockIdx.y;
  for (size_t i = blockIdx.x * blockDim.x + threadIdx.x; i < block_vecs;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    wt[(2 * b) * block_vecs + i] = gate[b * block_vecs + i];
    wt[(2 * b + 1) * block_vecs + i] = up[b * block_vecs + i];
  }
}

extern "C" int shk_interleave_gate_up(const void* gate_t, const void* up_t, int m, int k, void* wt,
                                      void* stream) {
  SHK_REQUIRE(m > 0 && k > 0 && gate_t && up_t && wt, "interleave_gate_up: bad arguments");
  const int mb = (m + 15) / 16, kt = (k + 31) / 32;
  SHK_REQUIRE(mb <= 65535, "interleave_gate_up: too many rows (%d)", m);
  const size_t block_vecs = static_cast<size_t>(kt) * kWave;
  interleave_blocks_kernel<<<dim3(8, mb), 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint4*>(gate_t), static_cast<const uint4*>(up_t), static_cast<uint4*>(wt),
      block_vecs);
  SHK_LAUNCH_CHECK("interleave_gate_up");
  return 0;
}

// Workgroups per block of 16 weight rows that a product with at most 64 rows
// should be split into along k so that the chip is full (about 8192 wavefronts
// with 4 k-tiles or more each): 1 for matrices with many row blocks.
template <int GM, int GN, int WM, int WN, int KS>
static void launch_big(hipStream_t s, const bf16* ap, int lda, int n, int k, const uint4* wp, int kt,
                       int m, const float* bias, void* out, int ldo, int of, int accumulate, int vec,
                       int gated, int wblocks, int ksplit) {
  constexpr int lds = 2 * (GM * WM + GN * WN) * KS * kWave * 16;
  const int tiles_x = (wblocks + GM * WM - 1) / (GM * WM), tiles_y = (n + 16 * GN * WN - 1) / (16 * GN * WN);
  // one-dimensional, in whole rounds of the eight dies' blocks of 32 tiles (see the kernel)
  const int block_y = tiles_y < 8 ? tiles_y : 8, block_x = kDieUnits / block_y;
  const long long blocks = static_cast<long long>((tiles_x + block_x - 1) / block_x) *
                           ((tiles_y + block_y - 1) / block_y);
  // worth it from four rounds of workgroups on: below that, whole dies would stay idle
  int by_die = static_cast<long long>(tiles_x) * tiles_y >= 4 * kDies * kDieUnits;
  if (!by_die) {
    // one rectangle of tiles per die, cut so that a die's tiles share the most
    // operands (the fewest rows of weights and activations to read per die)
    long long least = 0;
    for (int dx = 1; dx <= kDies; dx *= 2) {
      const int dy = kDies / dx;
      if (tiles_x % dx || tiles_y % dy) continue;
      const long long rows = static_cast<long long>(tiles_x / dx) * (16 * GM * WM) +
                             static_cast<long long>(tiles_y / dy) * (16 * GN * WN);
      if (!least || rows < least) least = rows, by_die = 2 * dx;
    }
  }
  dim3 grid(by_die == 1 ? static_cast<unsigned>((blocks + kDies - 1) / kDies * kDies * kDieUnits)
                   : static_cast<unsigned>(tiles_x * tiles_y),
            ksplit);
  // The kernel that loads straight into LDS, for workgroups that have a compute unit
  // to themselves anyway (its three or four stage buffers leave no room for a
  // second) and at least 128 tokens (with 64 it measured 3 % slower).
  if constexpr (GM * GN >= 8 && GN * WN >= 8 &&
                3 * (GM * WM + GN * WN) * KS * kWave * 16 <= 160 * 1024) {
    if (vec && kt % KS == 0) {
      if (gated)
        gemm_big_lds_kernel<GM, GN, WM, WN, KS, true><<<grid, GM * GN * kWave, 0, s>>>(
            ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, ksplit, tiles_x, tiles_y, by_die);
      else
        gemm_big_lds_kernel<GM, GN, WM, WN, KS, false><<<grid, GM * GN * kWave, 0, s>>>(
            ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, ksplit, tiles_x, tiles_y, by_die);
      return;
    }
  }
  if (gated) {
    auto kernel = gemm_big_kernel<GM, GN, WM, WN, KS, true>;
    if (lds > 65536)
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    kernel<<<grid, GM * GN * kWave, lds, s>>>(ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate,
                                              vec, ksplit, tiles_x, tiles_y, by_die);
  } else {
    auto kernel = gemm_big_kernel<GM, GN, WM, WN, KS, false>;
    if (lds > 65536)
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    kernel<<<grid, GM * GN * kWave, lds, s>>>(ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate,
                                              vec, ksplit, tiles_x, tiles_y, by_die);
  }
}

// Estimated time in microseconds of a product of many tokens with workgroup tiles
// of `shape` (0: 256 weight rows x 256 tokens, 1: 256 x 128, 2: 128 x 128) and
// `split` shares of k: rounds of workgroups over the chip's 256 compute units
// times the time of one workgroup, at the rates measured for each shape
// (TFLOP/s per compute unit: 4.75, 4.0, and for the smallest tile 3.0 with the
// compute unit to itself or 1.5 for each of two), plus what a kernel costs
// anyway, plus writing and reading the float32 parts of a split product at
// 3 TB/s (at 4 TB/s the estimate took shares that lost with their reader: the
// 14B down matrix at 4,096 tokens 701 us in two shares against 553 whole, the 14B
// QKV matrix at 768 tokens 100 us in three against 87, the 7B QKV matrix at 512
// tokens 54 in three against 51).  It reproduces the measured times of the 7B
// and 14B matrices at 512 tokens within 10 %.
static double big_estimate(int shape, int split, int n, int wblocks, int m, int k) {
  const int rows = shape == 2 ? 128 : 256, tokens = shape == 0 ? 256 : 128;
  const long long tiles =
      static_cast<long long>((wblocks * 16 + rows - 1) / rows) * ((n + tokens - 1) / tokens);
  const long long workgroups = tiles * split;
  double rounds, rate;
  if (shape == 2) {
    rounds = workgroups <= 256 ? 1.0 : static_cast<double>((workgroups + 511) / 512);
    rate = workgroups <= 256 ? 3.0 : 1.5;
  } else {
    rounds = static_cast<double>((workgroups + 255) / 256);
    rate = shape == 0 ? 4.75 : 4.0;
  }
  const double share = static_cast<double>(k) / split;
  double us = rounds * 2.0 * rows * tokens * share / (rate * 1e6) + 5.0;
  // (tokens counted in whole tiles of 128: the choice is then the same for every
  // number of tokens that a captured decode step of 128 or 256 rows may stand for)
  if (split > 1) us += 2.0 * split * ((n + 127) / 128 * 128.0) * m * 4.0 / 3e6;
  return us;
}

// The shape that big_estimate() prefers for a given number of shares.
static int big_shape(int split, int n, int wblocks, int m, int k) {
  int best = 0;
  for (int shape = 1; shape < 3; ++shape)
    if (big_estimate(shape, split, n, wblocks, m, k) < big_estimate(best, split, n, wblocks, m, k))
      best = shape;
  return best;
}

extern "C" int shk_gemm_bf16_splits(int n, int m, int k);

// 256 x 256 tiles that do not make whole rounds of the 256 compute units (296 of them:
// two rounds, the second nearly empty) are better run as two products: the row tiles
// that make whole rounds, then the remaining rows with the tile shape that suits them.
// Returns how many blocks of 16 weight rows the first product takes, or 0 where the
// estimate does not expect 7 % less time than from `shape` alone (the 14B gate/up matrix
// at 2,048 tokens, 864 tiles, is expected to gain 9 % and measured 12 %: 520 us against 588).
static int big_main_blocks(int shape, int n, int wblocks, int m, int k, int gated) {
  const int tiles_x = (wblocks + 15) / 16, tiles_y = (n + 255) / 256;
  const long long total = static_cast<long long>(tiles_x) * tiles_y;
  const int main_x = static_cast<int>(total / 256 * 256 / tiles_y);
  if (total <= 256 || main_x <= 0 || main_x >= tiles_x) return 0;
  const int main_blocks = main_x * 16, rest_blocks = wblocks - main_blocks;
  const int main_rows = main_blocks * 16 / (gated ? 2 : 1), rest_rows = m - main_rows;
  const int rest_shape = big_shape(1, n, rest_blocks, rest_rows, k);
  const double whole = big_estimate(shape, 1, n, wblocks, m, k);
  const double parts = big_estimate(0, 1, n, main_blocks, main_rows, k) +
                       big_estimate(rest_shape, 1, n, rest_blocks, rest_rows, k);
  return parts < 0.93 * whole ? main_blocks : 0;
}

// Products that a call with these sizes is made of (1, or 2: see big_main_blocks).
extern "C" int shk_gemm_bf16_parts(int n, int m, int k, int gated) {
  if (n <= 64 || shk_gemm_bf16_splits(n, m, k) > 1) return 1;
  const int wblocks = (gated ? 2 : 1) * ((m + 15) / 16);
  return big_main_blocks(big_shape(1, n, wblocks, m, k), n, wblocks, m, k, gated) ? 2 : 1;
}

extern "C" int shk_gemm_bf16_splits(int n, int m, int k) {
  const int mblocks = (m + 15) / 16, ktiles = (k + 31) / 32;
  if (n > 64) {
    // many tokens: the number of shares, each of at least 8 stages of 64, that
    // big_estimate() expects to be fastest with the tile shape that suits it
    int most = ktiles / 16;
    if (most > 16) most = 16;
    int best = 1;
    double least = big_estimate(big_shape(1, n, mblocks, m, k), 1, n, mblocks, m, k);
    for (int split = 2; split <= most; ++split) {
      const double us = big_estimate(big_shape(split, n, mblocks, m, k), split, n, mblocks, m, k);
      if (us < 0.97 * least) least = us, best = split;  // more shares only for a clear gain
    }
    return best;
  }
  if (mblocks >= 512) return 1;
  // up to 16 tokens: workgroups of 4 wavefronts share a block's k-tiles; more tokens:
  // every wavefront walks a block's k in stages of 4 tiles: about 2048 wavefronts
  // fill the chip, but a share below 28 tiles is mostly start and end, and the
  // reading kernel pays for every share (measured with 64 tokens, product and
  // norm together: 3584 x 3584 16 us with 4 shares against 20 with 8; 3584 x
  // 18944 37 us with 8 against 40 with 4)
  int split, most;
  if (n <= 16) {
    split = 8192 / (mblocks * 4), most = ktiles / 16;
    if (split > 16) split = 16;
    // A matrix of less than 96 MiB is read sooner than its kernel starts and ends: what
    // counts is how long the busiest compute unit's workgroups walk and what every share
    // costs by itself and in the kernel that adds the shares up.  Workgroups on one compute
    // unit take turns at its intake, so a launch takes about (workgroups per compute unit,
    // rounded up) x (k-tiles per share) x 0.057 us, and a share about 0.45 us.  Measured
    // with 8 tokens, product + reading norm: 3584 x 3584 in 2 shares 10.1 us, in 3 11.4,
    // in 4 11.0, in 7 11.8 (224, 336, 448, 784 workgroups on 256 compute units); 4608 x
    // 3584 in 2 13.8, in 3 12.4, in 4 13.6, in 7 12.9; 5120 x 5120 in 3 14.9, in 6 16.4;
    // 7168 x 5120 whole 17.6, in 4 19.5.
    if (static_cast<long long>(mblocks) * ktiles <= 96 * 1024) {
      const int groups = mblocks >= 128 ? (mblocks + 1) / 2 : mblocks;  // (pairs of row blocks)
      const int top = most < 1 ? 1 : (most > 16 ? 16 : most);
      int best = 1;
      double least = 0.0;
      for (int shares = 1; shares <= top; ++shares) {
        const int turns = (groups * shares + kDies * kDieUnits - 1) / (kDies * kDieUnits);
        const double us = turns * ((ktiles + shares - 1) / shares) * 0.057 + shares * 0.45;
        if (shares == 1 || us < least) least = us, best = shares;
      }
      return best;
    }
  } else {
    split = 2048 / mblocks, most = ktiles / 28;
    if (split > 8) split = 8;
    // a small matrix (896 x 896 has 56 blocks: 14 workgroups) is a matter of how long one
    // wavefront walks, not of what its shares cost: shares down to two stages of four tiles
    // (with 64 tokens 896 x 896 takes 6 us in 3 shares against 10.5 whole)
    const int with_most = split < most ? split : most;
    if (mblocks * (with_most > 1 ? with_most : 1) < 512) most = ktiles / 8;
  }
  if (split > most) split = most;
  return split > 1 ? split : 1;
}

extern "C" int shk_gemm_bf16_tiled_weight(const void* a, const void* wt, const float* bias,
                                          void* out, int n, int m, int k, int lda, int ldo,
                                          int out_dtype, int accumulate, int gated, int ksplit,
                                          void* stream) {
  SHK_REQUIRE(gated >= 0 && gated <= kActGeluTanh, "gemm_bf16: unknown gate activation %d", gated);
  SHK_REQUIRE(!gated || (!accumulate && !bias), "gemm_bf16: a gated product takes no bias and does not accumulate");
  SHK_REQUIRE(ksplit >= 1 && ksplit <= 64, "gemm_bf16: ksplit %d is outside 1..64", ksplit);
  SHK_REQUIRE(ksplit == 1 || (!gated && !accumulate && !bias && out_dtype == kF32 && ldo == m),
              "gemm_bf16: a product split along k writes plain float32 partial sums [ksplit][n][m]");
  SHK_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "gemm_bf16: unknown out_dtype %d",
              out_dtype);
  SHK_REQUIRE(n >= 0 && m > 0 && k > 0, "gemm_bf16: bad sizes n=%d m=%d k=%d", n, m, k);
  SHK_REQUIRE(lda >= k && ldo >= m, "gemm_bf16: row strides lda=%d ldo=%d too small", lda, ldo);
  SHK_REQUIRE(!accumulate || out_dtype == kF32, "gemm_bf16: accumulate needs a float32 output");
  if (n == 0) return 0;
  if (gated) accumulate = gated;  // the gated kernels read the activation from this argument
  SHK_REQUIRE(a && wt && out, "gemm_bf16: null pointer");
  const int mb = (m + 15) / 16, kt = (k + 31) / 32;
  const int vec = (k % 8 == 0 && lda % 8 == 0 && (reinterpret_cast<uintptr_t>(a) % 16) == 0);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bf16* ap = static_cast<const bf16*>(a);
  const uint4* wp = static_cast<const uint4*>(wt);
  const int of = out_dtype == kF32;
  if (n > 64) {
    SHK_REQUIRE(reinterpret_cast<uintptr_t>(out) % 8 == 0, "gemm_bf16: out is not 8-byte aligned");
    const int wblocks = (gated ? 2 : 1) * mb;  // blocks of 16 weight rows
    // Tile of the workgroup: 256 x 256, 256 x 128 or 128 x 128 (weight rows x
    // tokens), whichever big_estimate() expects to finish first.
    const int shape = big_shape(ksplit, n, wblocks, m, k);
    int main_blocks = 0;
    if (ksplit == 1) main_blocks = big_main_blocks(shape, n, wblocks, m, k, gated);
    if (main_blocks) {
      const int rest_blocks = wblocks - main_blocks;
      const int main_rows = main_blocks * 16 / (gated ? 2 : 1), rest_rows = m - main_rows;
      const int rest_shape = big_shape(1, n, rest_blocks, rest_rows, k);
      launch_big<4, 4, 4, 4, 1>(s, ap, lda, n, k, wp, kt, main_rows, bias, out, ldo, of, accumulate,
                                vec, gated, main_blocks, 1);
      const uint4* rest_w = wp + static_cast<size_t>(main_blocks) * kt * kWave;
      const float* rest_bias = bias ? bias + main_rows : nullptr;
      void* rest_out = of ? static_cast<void*>(static_cast<float*>(out) + main_rows)
                          : static_cast<void*>(static_cast<bf16*>(out) + main_rows);
      if (rest_shape == 0)
        launch_big<4, 4, 4, 4, 1>(s, ap, lda, n, k, rest_w, kt, rest_rows, rest_bias, rest_out, ldo,
                                  of, accumulate, vec, gated, rest_blocks, 1);
      else if (rest_shape == 1)
        launch_big<4, 4, 4, 2, 2>(s, ap, lda, n, k, rest_w, kt, rest_rows, rest_bias, rest_out, ldo,
                                  of, accumulate, vec, gated, rest_blocks, 1);
      else if (static_cast<long long>((rest_blocks + 7) / 8) * ((n + 127) / 128) <= 256)
        launch_big<4, 2, 2, 4, 2>(s, ap, lda, n, k, rest_w, kt, rest_rows, rest_bias, rest_out, ldo,
                                  of, accumulate, vec, gated, rest_blocks, 1);
      else
        launch_big<2, 2, 4, 4, 2>(s, ap, lda, n, k, rest_w, kt, rest_rows, rest_bias, rest_out, ldo,
                                  of, accumulate, vec, gated, rest_blocks, 1);
      SHK_LAUNCH_CHECK("gemm_bf16");
      return 0;
    }
    if (shape == 0)
      launch_big<4, 4, 4, 4, 1>(s, ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec,
                                gated, wblocks, ksplit);
    else if (shape == 1)
      launch_big<4, 4, 4, 2, 2>(s, ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec,
                                gated, wblocks, ksplit);
    else if (static_cast<long long>((wblocks + 7) / 8) * ((n + 127) / 128) * ksplit <= 256)
      // every workgroup has a compute unit to itself: eight wavefronts, loads straight into LDS
      launch_big<4, 2, 2, 4, 2>(s, ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec,
                                gated, wblocks, ksplit);
    else  // four wavefronts and two LDS buffers: two workgroups fit on a compute unit
      launch_big<2, 2, 4, 4, 2>(s, ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec,
                                gated, wblocks, ksplit);
    SHK_LAUNCH_CHECK("gemm_bf16");
    return 0;
  }
  if (n > 16 && vec) {
    // 17 to 64 tokens, aligned rows: every wavefront streams the weights of its own
    // block of rows, the activations are shared through LDS.  Wavefronts per
    // workgroup: so many that the launch is one workgroup for each of the 256
    // compute units, or a whole number of rounds of them where 16 per workgroup
    // do not suffice (an even number for gated weights: gate and up side by side).
    const int wblocks = (gated ? 2 : 1) * mb;
    const long long tasks = static_cast<long long>(wblocks) * ksplit;
    // (more than a round's worth: workgroups of 8, two of which share a compute unit
    // and fill each other's pauses)
    int waves = tasks > 256 * 16 ? 8 : static_cast<int>((tasks + 255) / 256);
    waves = waves < 4 ? 4 : waves;
    if (gated) waves += waves & 1;
    const int nb = n <= 32 ? 2 : 4;
    const int aper = (nb * kStreamTiles + waves - 1) / waves;  // 1 to 4
    dim3 sgrid((wblocks + waves - 1) / waves, ksplit);
#define SHK_STREAM(NB, APER)                                                         \
  do {                                                                               \
    if (gated)                                                                       \
      gemm_stream_kernel<NB, APER, true><<<sgrid, waves * kWave, 0, s>>>(            \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, ksplit);         \
    else                                                                             \
      gemm_stream_kernel<NB, APER, false><<<sgrid, waves * kWave, 0, s>>>(           \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, ksplit);         \
  } while (0)
    if (nb == 2) {
      if (aper == 1) SHK_STREAM(2, 1); else SHK_STREAM(2, 2);
    } else {
      if (aper == 1) SHK_STREAM(4, 1);
      else if (aper == 2) SHK_STREAM(4, 2);
      else if (aper == 3) SHK_STREAM(4, 3);
      else SHK_STREAM(4, 4);
    }
#undef SHK_STREAM
    SHK_LAUNCH_CHECK("gemm_bf16");
    return 0;
  }
  if (n > 32 && mb < 4096) {
    // 33 to 64 tokens: the LDS-staged kernel with tiles of 256 weight rows x 64
    // tokens beats the kernel below where it has at least half the chip's
    // compute units to fill and a long walk along k for each workgroup (the
    // 7B down and gate/up matrices at 64 tokens: 36 us against 46, 61 against 65)
    const int wblocks = (gated ? 2 : 1) * mb;
    const int workgroups = ((wblocks + 15) / 16) * ksplit;
    const int stages = (kt / ksplit + 1) / 2;
    if (workgroups >= 128 && stages >= 16) {
      SHK_REQUIRE(reinterpret_cast<uintptr_t>(out) % 8 == 0, "gemm_bf16: out is not 8-byte aligned");
      launch_big<4, 2, 4, 2, 2>(s, ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec,
                                gated, wblocks, ksplit);
      SHK_LAUNCH_CHECK("gemm_bf16");
      return 0;
    }
  }
  if (n > 16) {
    // blocks of output rows per workgroup: 8 where that still leaves enough workgroups
    const int mid_waves = (mb >= 4096) ? 8 : 4;
    dim3 mgrid((mb + mid_waves - 1) / mid_waves, ksplit);
#define SHK_MID_W(NB, W)                                                                    \
  do {                                                                                      \
    if (gated)                                                                              \
      gemm_mid_kernel<NB, W, true><<<mgrid, W * kWave, 0, s>>>(                             \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec, ksplit);           \
    else                                                                                    \
      gemm_mid_kernel<NB, W, false><<<mgrid, W * kWave, 0, s>>>(                            \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec, ksplit);           \
  } while (0)
#define SHK_MID(NB)          \
  do {                       \
    if (mid_waves == 8)      \
      SHK_MID_W(NB, 8);      \
    else                     \
      SHK_MID_W(NB, 4);      \
  } while (0)
    // always four token blocks: the narrower instantiations measured slower, and the
    // multiplications for absent tokens cost nothing next to the weight traffic
    SHK_MID(4);
#undef SHK_MID
#undef SHK_MID_W
    SHK_LAUNCH_CHECK("gemm_bf16");
    return 0;
  }
  // wavefronts per workgroup: matrices with few row blocks get more of them
  const int waves = (mb >= 512 || ksplit > 1) ? ((mb >= 512) ? 8 : 4) : 16;
  const int max_waves = 16;
  // two row blocks per workgroup share their activation loads, where the matrix has
  // enough blocks to fill the chip with half as many workgroups
  const bool pair = !gated && mb >= 128;
  dim3 sgrid(pair ? (mb + 1) / 2 : mb, ksplit);
#define SHK_SKINNY_W(NB, W)                                                                     \
  do {                                                                                          \
    if (gated)                                                                                  \
      gemm_skinny_kernel<NB, W, kGated><<<sgrid, W * kWave, 0, s>>>(                            \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec, ksplit);               \
    else if (pair)                                                                              \
      gemm_skinny_kernel<NB, W, kPair><<<sgrid, W * kWave, 0, s>>>(                             \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec, ksplit);               \
    else                                                                                        \
      gemm_skinny_kernel<NB, W, kSingle><<<sgrid, W * kWave, 0, s>>>(                           \
          ap, lda, n, k, wp, kt, m, bias, out, ldo, of, accumulate, vec, ksplit);               \
  } while (0)
#define SHK_SKINNY(NB)                       \
  do {                                       \
    if (waves == 4)                          \
      SHK_SKINNY_W(NB, 4);                   \
    else if (waves == 8 || max_waves == 8)   \
      SHK_SKINNY_W(NB, 8);                   \
    else                                     \
      SHK_SKINNY_W(NB, 16);                  \
  } while (0)
  SHK_SKINNY(1);
#undef SHK_SKINNY
#undef SHK_SKINNY_W
  SHK_LAUNCH_CHECK("gemm_bf16");
  return 0;
}

// The matrix units alone: workgroups x 4 wavefronts, each iters times a 64 x 64 x 32
// block (2 * 64 * 64 * 32 flop) from operands (64 KiB of bfloat16) held in registers;
// out takes workgroups * 256 floats.  For measuring what the chip's matrix units give
// on operands of a given kind; no product of the engine calls it.
extern "C" int shk_mfma_alone(const void* operands, float* out, int workgroups, int iters, void* stream) {
  SHK_REQUIRE(operands && out && workgroups > 0 && iters > 0, "mfma_alone: bad arguments");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(operands) % 16 == 0, "mfma_alone: operands are not 16-byte aligned");
  mfma_alone_kernel<<<workgroups, 4 * kWave, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const u32x4*>(operands), out, iters);
  SHK_LAUNCH_CHECK("mfma_alone");
  return 0;
}
