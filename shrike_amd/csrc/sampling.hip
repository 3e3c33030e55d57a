// Choosing the next token from float32 logits: argmax (lowest index among equal
// maxima) and temperature / top-p sampling.
//
// Sampling follows the reference's rule (shrike/engine/sampler.py:20-30):
// weights softmax(logits / T); ordered by descending weight, an entry is kept
// while the weight before it is below top_p (the largest is always kept); one
// entry is drawn in proportion to the kept weights.  Nothing is sorted here:
// the smallest kept weight tau is the largest value x whose upper mass
// sum{w >= x} still reaches top_p, found by a 31-step search over the bits of
// x; entries equal to tau are kept lowest index first, as many as the rule
// admits.  The draw walks the kept entries in index order with the caller's
// uniform number, so a row's result depends only on its logits and its number.
#include <mutex>

#include "api.h"
#include "common.h"

namespace shk {

constexpr int kSampleThreads = 1024;

struct MaxIdx {
  float v;
  int i;
};

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ MaxIdx block_argmax(const float* __restrict__ x, int n, MaxIdx* scratch) {
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = x[i];
    if (v > best.v) best = MaxIdx{v, i};  // ascending i per thread: first maximum wins
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    MaxIdx o{__shfl_xor(best.v, off, kWave), __shfl_xor(best.i, off, kWave)};
    best = better(best, o);
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = best;
  __syncthreads();
  MaxIdx total = scratch[0];
  for (int w = 1; w < nwaves; ++w) total = better(total, scratch[w]);
  if (total.i == 0x7fffffff) total.i = 0;  // a row of NaN or -inf
  return total;
}

__global__ void __launch_bounds__(kSampleThreads)
    argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, int vocab, int ld) {
  __shared__ MaxIdx scratch[16];
  const MaxIdx best = block_argmax(logits + static_cast<size_t>(blockIdx.x) * ld, vocab, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = best.i;
}

// Two stages for wide rows: every chunk of kArgmaxChunk values gets a workgroup
// that leaves its best (value, index); a second kernel picks among the chunks,
// lowest index first among equals.
constexpr int kArgmaxChunk = 4096;
constexpr int kArgmaxThreads = 256;

__global__ void __launch_bounds__(kArgmaxThreads)
    argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ best_value,
                         int32_t* __restrict__ best_index, int vocab, int ld, int chunks) {
  __shared__ MaxIdx scratch[16];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int begin = chunk * kArgmaxChunk;
  const int count = vocab - begin < kArgmaxChunk ? vocab - begin : kArgmaxChunk;
  MaxIdx best = block_argmax(logits + static_cast<size_t>(row) * ld + begin, count, scratch);
  if (threadIdx.x == 0) {
    best_value[row * chunks + chunk] = best.v;
    best_index[row * chunks + chunk] = begin + best.i;
  }
}

__global__ void __launch_bounds__(kArgmaxThreads)
    argmax_pick_kernel(const float* __restrict__ best_value, const int32_t* __restrict__ best_index,
                       int32_t* __restrict__ out, int chunks) {
  __shared__ MaxIdx scratch[16];
  const int row = blockIdx.x;
  // chunks are in index order, so the first maximum among them has the lowest index
  const MaxIdx best = block_argmax(best_value + static_cast<size_t>(row) * chunks, chunks, scratch);
  if (threadIdx.x == 0) out[row] = best_index[row * chunks + best.i];
}

// Exclusive prefix sums over the threads of the workgroup (thread order), and the total.
__device__ void block_exclusive_scan(float v, float* buf, float* before, float* total) {
  __syncthreads();
  buf[threadIdx.x] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int i = 0; i < static_cast<int>(blockDim.x); ++i) {
      const float x = buf[i];
      buf[i] = run;
      run += x;
    }
    buf[blockDim.x] = run;
  }
  __syncthreads();
  *before = buf[threadIdx.x];
  *total = buf[blockDim.x];
}

__global__ void __launch_bounds__(kSampleThreads)
    sample_kernel(const float* __restrict__ logits, int32_t* __restrict__ out,
                  const float* __restrict__ temperature, const float* __restrict__ top_p,
                  const float* __restrict__ uniforms, float* __restrict__ scratch_all, int vocab,
                  int ld) {
  __shared__ MaxIdx mscratch[16];
  __shared__ float fscratch[16];
  __shared__ float scan[kSampleThreads + 1];
  __shared__ int chosen;

  const int r = blockIdx.x;
  const float* x = logits + static_cast<size_t>(r) * ld;
  float* w = scratch_all + static_cast<size_t>(r) * vocab;
  const MaxIdx best = block_argmax(x, vocab, mscratch);
  const float temp = temperature[r];
  if (!(temp > 0.f)) {
    if (threadIdx.x == 0) out[r] = best.i;
    return;
  }

  // weights w_i = exp((x_i - max) / T); Z their sum
  float z = 0.f;
  for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
    const float e = expf((x[i] - best.v) / temp);
    w[i] = e;
    z += e;
  }
  z = block_sum(z, fscratch);

  // tau: largest x with sum{w >= x} >= top_p * Z
  const float p = top_p[r];
  const float need = p * z;
  uint32_t tau_bits = 0;
  if (p < 1.f) {
    for (int bit = 30; bit >= 0; --bit) {
      const uint32_t cand = tau_bits | (1u << bit);
      float mass = 0.f;
      for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
        const float e = w[i];
        if (__float_as_uint(e) >= cand) mass += e;
      }
      mass = block_sum(mass, fscratch);
      if (mass >= need) tau_bits = cand;
    }
  }
  const float tau = __uint_as_float(tau_bits);

  // how many entries equal to tau the rule admits: those with above + c * tau < need
  float above = 0.f, ties = 0.f;
  for (int i = threadIdx.x; i < vocab; i += kSampleThreads) {
    const float e = w[i];
    if (e > tau) above += e;
    if (e == tau) ties += 1.f;
  }
  above = block_sum(above, fscratch);
  ties = block_sum(ties, fscratch);
  float admit = ties;
  if (p < 1.f && tau > 0.f) admit = fminf(fmaxf(ceilf((need - above) / tau), 1.f), ties);

  // walk in index order: each thread owns a contiguous chunk
  const int chunk = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int begin = threadIdx.x * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;
  float my_ties = 0.f;
  for (int i = begin; i < end; ++i)
    if (w[i] == tau) my_ties += 1.f;
  float ties_before, ties_total;
  block_exclusive_scan(my_ties, scan, &ties_before, &ties_total);
  float my_mass = 0.f;
  {
    float seen = ties_before;
    for (int i = begin; i < end; ++i) {
      const float e = w[i];
      if (e > tau) {
        my_mass += e;
      } else if (e == tau) {
        if (seen < admit) my_mass += e;
        seen += 1.f;
      }
    }
  }
  float mass_before, mass_total;
  block_exclusive_scan(my_mass, scan, &mass_before, &mass_total);
  const float target = uniforms[r] * mass_total;

  if (threadIdx.x == 0) chosen = 0x7fffffff;
  __syncthreads();
  if (mass_before <= target && my_mass > 0.f) {
    float run = mass_before, seen = ties_before;
    for (int i = begin; i < end; ++i) {
      const float e = w[i];
      bool kept = e > tau;
      if (e == tau) {
        kept = seen < admit;
        seen += 1.f;
      }
      if (!kept) continue;
      run += e;
      if (run > target) {
        atomicMin(&chosen, i);
        break;
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) out[r] = (chosen == 0x7fffffff) ? best.i : chosen;
}

}  // namespace shk

using namespace shk;

extern "C" int shk_argmax_scratch_floats(int rows, int vocab) {
  const int chunks = (vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  return chunks > 1 ? 2 * rows * chunks : 0;
}

extern "C" int shk_argmax(const float* logits, int32_t* out, int rows, int vocab, int ld,
                          float* scratch, void* stream) {
  SHK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "argmax: bad sizes rows=%d vocab=%d ld=%d",
              rows, vocab, ld);
  if (rows == 0) return 0;
  SHK_REQUIRE(logits && out, "argmax: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  if (chunks == 1) {
    argmax_kernel<<<rows, kSampleThreads, 0, s>>>(logits, out, vocab, ld);
    SHK_LAUNCH_CHECK("argmax");
    return 0;
  }
  SHK_REQUIRE(scratch, "argmax: rows of %d values need the scratch buffer", vocab);
  SHK_REQUIRE(rows <= 65535, "argmax: at most 65535 rows a call, got %d", rows);
  float* best_value = scratch;
  int32_t* best_index = reinterpret_cast<int32_t*>(scratch + static_cast<size_t>(rows) * chunks);
  argmax_chunks_kernel<<<dim3(chunks, rows), kArgmaxThreads, 0, s>>>(logits, best_value, best_index,
                                                                     vocab, ld, chunks);
  SHK_LAUNCH_CHECK("argmax");
  argmax_pick_kernel<<<rows, kArgmaxThreads, 0, s>>>(best_value, best_index, out, chunks);
  SHK_LAUNCH_CHECK("argmax");
  return 0;
}

// ------------------------------------------------------ argmax without a workspace
// The chunk results of the two-stage argmax in memory that the library itself
// holds: one array per GPU, there from the moment the code object is loaded until
// the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels get the device address it returns.
constexpr int kStaticScratchFloats = 1 << 16;  // 256 KiB: 2 * rows * chunks floats at most
static __device__ __align__(256) float scratch[kStaticScratchFloats];

constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
static float* scratch_of_device[kMaxDevices];  // device address of `scratch` on each GPU

// Address of the current device's copy of `scratch`, looked up once per device.
static int static_scratch(float** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  SHK_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  SHK_REQUIRE(device >= 0 && device < kMaxDevices, "argmax_static: device %d is beyond %d", device,
              kMaxDevices);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_of_device[device] == nullptr) {
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    SHK_REQUIRE(e == hipSuccess && addr != nullptr,
                "argmax_static: hipGetSymbolAddress failed on device %d: %s", device,
                hipGetErrorString(e));
    scratch_of_device[device] = static_cast<float*>(addr);
  }
  *ptr = scratch_of_device[device];
  return 0;
}

extern "C" int shk_argmax_static_max_floats(void) { return kStaticScratchFloats; }

extern "C" int shk_argmax_static(const float* logits, int32_t* out, int rows, int vocab, int ld,
                                 void* stream) {
  SHK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab,
              "argmax_static: bad sizes rows=%d vocab=%d ld=%d", rows, vocab, ld);
  const long long need = shk_argmax_scratch_floats(1, vocab) * static_cast<long long>(rows);
  SHK_REQUIRE(need <= kStaticScratchFloats,
              "argmax_static: %d rows of %d values need %lld floats of scratch, the library's own "
              "array holds %d (use shk_argmax with a workspace)",
              rows, vocab, need, kStaticScratchFloats);
  float* ptr = nullptr;
  if (int rc = static_scratch(&ptr)) return rc;
  // every chunk result that the second kernel reads is written by the first one in
  // this call: nothing has to be cleared, whatever an earlier call left behind
  return shk_argmax(logits, out, rows, vocab, ld, ptr, stream);
}

extern "C" int shk_sample(const float* logits, int32_t* out, const float* temperature,
                          const float* top_p, const float* uniforms, float* scratch, int rows,
                          int vocab, int ld, void* stream) {
  SHK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%d",
              rows, vocab, ld);
  if (rows == 0) return 0;
  SHK_REQUIRE(logits && out && temperature && top_p && uniforms && scratch, "sample: null pointer");
  sample_kernel<<<rows, kSampleThreads, 0, static_cast<hipStream_t>(stream)>>>(
      logits, out, temperature, top_p, uniforms, scratch, vocab, ld);
  SHK_LAUNCH_CHECK("sample");
  return 0;
}
