// Choosing the next token from float32 logits: argmax (lowest index among equal
// maxima) and temperature / top-p sampling.
//
// Sampling follows the reference's rule (shrike/engine/sampler.py:20-30):
// weights softmax(logits / T); ordered by descending weight, an entry is kept
// while the weight before it is below top_p (the largest is always kept); one
// entry is drawn in proportion to the kept weights.  Nothing is sorted here:
// the smallest kept weight tau is the largest value x whose upper mass
// sum{w >= x} still reaches top_p, found by a search over the bits of x;
// entries equal to tau are kept lowest index first, as many as the rule
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

// ------------------------------------------------------ temperature / top-p
// A row of 152,064 logits is too long for one workgroup to walk a few dozen
// times (that takes 0.3 to 1.8 ms a step, with the batch), so a row is cut into
// chunks of 4096 like the wide argmax, every pass over the logits is a launch of
// chunks x rows workgroups, and short single-workgroup kernels between them
// decide.  Weights are integers, floor(exp((x - max) / T) * 2^40): sums of
// integers do not depend on their order, so every comparison below comes out the
// same however the work is cut (and weights below 2^-40 of the largest count as
// nothing).  The passes:
//   chunks   largest logit of every chunk (argmax_chunks_kernel);
//   weigh    the chunk's weights by class of magnitude (eight classes per factor
//            of two), summed per class;
//   boundary the class in which the upper mass reaches need = top_p * total;
//   collect  where the weights of that class lie, in index order;
//   threshold  tau, the smallest kept weight: the largest x whose upper mass
//            sum{w >= x} reaches need, found eight bits at a time among the
//            collected weights alone (in LDS if there are at most 8192); how many
//            of the weights equal to tau the rule admits (lowest index first);
//            and with that every chunk's kept mass and number of such weights;
//   draw     the chunk, then the entry, at which the kept mass in index order
//            passes uniform * kept mass; rows of temperature 0 get their argmax.
// Rows without a nucleus (top_p >= 1) keep everything: tau = 0.  When the caller
// says that no row has one, boundary, collect and threshold are not launched.

constexpr int kChunkThreads = 256;
constexpr int kPerThread = kArgmaxChunk / kChunkThreads;  // consecutive logits of a thread
constexpr int kChunkLds = kArgmaxChunk + kArgmaxChunk / kPerThread;  // a spare word per thread: no bank conflicts
constexpr int kBins = 320;            // classes of weights (weight_class() gives 0..304)
constexpr int kBoundaryInLds = 8192;  // collected weights that the threshold search keeps in LDS
constexpr int kMaxChunks = 1024;      // a row of at most 4,194,304 logits
constexpr int kThresholdThreads = 1024;
using u64 = unsigned long long;

struct RowState {
  u64 need;      // top_p * total, rounded up
  u64 above;     // mass of the classes above the boundary class
  u64 tau;       // smallest kept weight
  uint32_t admit;  // how many weights equal to tau are kept
  int boundary;    // the class that holds tau; -1: the row keeps everything
};

__device__ __forceinline__ u64 weight_of(float x, float mx, float temp) {
  const float scaled = expf((x - mx) / temp) * 1099511627776.f;  // 2^40
  return scaled >= 1.f ? __float2ull_rz(scaled) : 0ull;  // NaN, -inf and tiny: nothing
}

// Classes in the order of the weights: the value itself below 16, then the
// position of the highest bit and the three bits after it.
__device__ __forceinline__ int weight_class(u64 q) {
  if (q < 16) return static_cast<int>(q);
  const int hb = 63 - __clzll(q);
  const int cls = (hb - 3) * 8 + static_cast<int>((q >> (hb - 3)) & 7) + 8;
  return cls < kBins ? cls : kBins - 1;  // (weights reach 2^40, class 304)
}

// The smallest weight of a class, and how many low bits the class leaves open.
__device__ __forceinline__ u64 class_base(int cls, int* open_bits) {
  if (cls < 16) {
    *open_bits = 0;
    return static_cast<u64>(cls);
  }
  const int hb = (cls - 8) / 8 + 3;
  *open_bits = hb - 3;
  return static_cast<u64>(8 + (cls - 8) % 8) << (hb - 3);
}

__device__ __forceinline__ u64 wave_sum_u64(u64 v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Sum over the workgroup; every thread gets it.  `scratch` holds 16 values.
__device__ __forceinline__ u64 block_sum_u64(u64 v, u64* scratch) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum_u64(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  u64 total = 0;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

// Exclusive prefix sums in thread order, and the total.  `scratch` holds 17 values.
__device__ __forceinline__ void block_scan_u64(u64 v, u64* scratch, u64* before, u64* total) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  u64 incl = v;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const u64 o = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += o;
  }
  __syncthreads();
  if (lane == kWave - 1) scratch[wave] = incl;
  __syncthreads();
  u64 base = 0, all = 0;
  for (int w = 0; w < nwaves; ++w) {
    if (w < wave) base += scratch[w];
    all += scratch[w];
  }
  *before = base + incl - v;
  *total = all;
}

// The largest logit of the row, from the chunks' maxima.  `scratch` holds 16 floats.
__device__ __forceinline__ float row_maximum(const float* __restrict__ best_value, int row, int chunks,
                                             float* scratch) {
  float mx = -INFINITY;
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) mx = fmaxf(mx, best_value[row * chunks + c]);
  return block_max(mx, scratch);
}

// A chunk's logits: fetched 256 neighbours at a time and handed to their owners
// through LDS; thread t owns logits 16 t .. 16 t + 15 of the chunk.  Beyond the
// row's end: -inf, whose weight is nothing.
__device__ __forceinline__ void load_chunk(const float* __restrict__ row, int begin, int vocab, float* lds,
                                           float (&x)[kPerThread]) {
  __syncthreads();  // whoever read lds before is done
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const int i = k * kChunkThreads + threadIdx.x;
    lds[i + i / kPerThread] = begin + i < vocab ? row[begin + i] : -INFINITY;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) x[k] = lds[threadIdx.x * (kPerThread + 1) + k];
}

// What the passes leave for each other, per row and chunk, in the caller's scratch.
struct SampleScratch {
  float* best_value;    // [rows][chunks]
  int32_t* best_index;  // [rows][chunks]
  RowState* state;      // [rows]
  u64* kept_mass;       // [rows][chunks]
  uint32_t* ties;       // [rows][chunks] weights equal to tau
  uint32_t* collected;  // [rows][chunks] entries of `where`
  u64* class_mass;      // [rows][chunks][kBins]
  u64* heavier;         // [rows][chunks] mass of the classes above the boundary class
  int32_t* where;       // [rows][chunks][kArgmaxChunk] indices of the boundary class's weights
};

static size_t sample_scratch_words(int rows, int chunks, SampleScratch* s, float* base) {
  const size_t rc = static_cast<size_t>(rows) * chunks;
  size_t at = 0;
  const auto take = [&](size_t words) {
    const size_t here = at;
    at += (words + 3) / 4 * 4;  // every array starts 16-byte aligned
    return here;
  };
  const size_t a = take(rc), b = take(rc), c = take(static_cast<size_t>(rows) * sizeof(RowState) / 4),
               d = take(2 * rc), e = take(rc), f = take(rc), g = take(2 * rc * kBins), i = take(2 * rc),
               h = take(rc * kArgmaxChunk);
  if (s) {
    s->best_value = base + a;
    s->best_index = reinterpret_cast<int32_t*>(base + b);
    s->state = reinterpret_cast<RowState*>(base + c);
    s->kept_mass = reinterpret_cast<u64*>(base + d);
    s->ties = reinterpret_cast<uint32_t*>(base + e);
    s->collected = reinterpret_cast<uint32_t*>(base + f);
    s->class_mass = reinterpret_cast<u64*>(base + g);
    s->heavier = reinterpret_cast<u64*>(base + i);
    s->where = reinterpret_cast<int32_t*>(base + h);
  }
  return at;
}

template <bool NUCLEUS>
__global__ void __launch_bounds__(kChunkThreads)
    sample_weigh_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                        SampleScratch s, int vocab, int ld, int chunks) {
  __shared__ float lds[kChunkLds];
  __shared__ float fscratch[16];
  __shared__ u64 uscratch[16];
  __shared__ u64 mass[NUCLEUS ? kBins : 1];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float temp = temperature[row];
  if (!(temp > 0.f)) return;
  const float mx = row_maximum(s.best_value, row, chunks, fscratch);
  float x[kPerThread];
  load_chunk(logits + static_cast<size_t>(row) * ld, chunk * kArgmaxChunk, vocab, lds, x);
  if (NUCLEUS) {
    for (int b = threadIdx.x; b < kBins; b += kChunkThreads) mass[b] = 0;
    __syncthreads();
  }
  u64 sum = 0;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const u64 q = weight_of(x[k], mx, temp);
    sum += q;
    if (NUCLEUS && q) atomicAdd(&mass[weight_class(q)], q);  // integers: any order gives the same sums
  }
  const size_t rc = static_cast<size_t>(row) * chunks + chunk;
  if (NUCLEUS) {
    __syncthreads();
    for (int b = threadIdx.x; b < kBins; b += kChunkThreads) s.class_mass[rc * kBins + b] = mass[b];
  } else {
    sum = block_sum_u64(sum, uscratch);
    if (threadIdx.x == 0) {
      s.kept_mass[rc] = sum;  // everything is kept
      s.ties[rc] = 0;
    }
  }
}

__global__ void __launch_bounds__(kBins)
    sample_boundary_kernel(const float* __restrict__ temperature, const float* __restrict__ top_p,
                           SampleScratch s, int chunks) {
  __shared__ u64 uscratch[17];
  __shared__ float fscratch[16];
  const int row = blockIdx.x;
  if (!(temperature[row] > 0.f)) return;
  // thread t takes class kBins - 1 - t: the prefix sums in thread order are the masses above a class
  const int cls = kBins - 1 - static_cast<int>(threadIdx.x);
  u64 mass = 0;
  const u64* of_chunk = s.class_mass + static_cast<size_t>(row) * chunks * kBins + cls;
  for (int c0 = 0; c0 < chunks; c0 += 8) {  // eight loads in flight
    u64 part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = c0 + u < chunks ? of_chunk[static_cast<size_t>(c0 + u) * kBins] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) mass += part[u];
  }
  u64 above, total;
  block_scan_u64(mass, uscratch, &above, &total);
  const float p = top_p[row];
  if (!(p < 1.f) || total == 0) {
    if (threadIdx.x == 0) s.state[row] = RowState{total, 0, 0, 0, -1};
    return;
  }
  const double exact = static_cast<double>(p) * static_cast<double>(total);
  u64 need = static_cast<u64>(ceil(exact));
  need = need < 1 ? 1 : (need > total ? total : need);
  // the heaviest class at which the upper mass reaches `need`
  const bool reached = above + mass >= need;
  const int boundary = static_cast<int>(block_max(reached ? static_cast<float>(cls) : -1.f, fscratch));
  if (cls == boundary) s.state[row] = RowState{need, above, 0, 0, boundary};
}

__global__ void __launch_bounds__(kChunkThreads)
    sample_collect_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                          SampleScratch s, int vocab, int ld, int chunks) {
  __shared__ float lds[kChunkLds];
  __shared__ float fscratch[16];
  __shared__ u64 uscratch[17];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float temp = temperature[row];
  if (!(temp > 0.f)) return;
  const size_t rc = static_cast<size_t>(row) * chunks + chunk;
  const int boundary = s.state[row].boundary;
  // the chunk's mass in the classes above the boundary class: kept whatever tau turns out to be
  u64 above = 0;
  for (int b = boundary + 1 + threadIdx.x; b < kBins; b += kChunkThreads) above += s.class_mass[rc * kBins + b];
  above = block_sum_u64(above, uscratch);
  if (boundary < 0) {  // the row keeps everything
    if (threadIdx.x == 0) s.kept_mass[rc] = above, s.ties[rc] = 0, s.collected[rc] = 0;
    return;
  }
  if (threadIdx.x == 0) s.heavier[rc] = above;
  const float mx = row_maximum(s.best_value, row, chunks, fscratch);
  float x[kPerThread];
  const int begin = chunk * kArgmaxChunk;
  load_chunk(logits + static_cast<size_t>(row) * ld, begin, vocab, lds, x);
  uint32_t flags = 0;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const u64 q = weight_of(x[k], mx, temp);
    if (q && weight_class(q) == boundary) flags |= 1u << k;
  }
  u64 before, total;
  block_scan_u64(__popc(flags), uscratch, &before, &total);
  int32_t* dst = s.where + rc * kArgmaxChunk + before;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k)
    if (flags & (1u << k)) *dst++ = begin + threadIdx.x * kPerThread + k;
  if (threadIdx.x == 0) s.collected[rc] = static_cast<uint32_t>(total);
}

__global__ void __launch_bounds__(kThresholdThreads)
    sample_threshold_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                            SampleScratch s, int ld, int chunks) {
  __shared__ u64 held[kBoundaryInLds];
  __shared__ uint32_t first[kMaxChunks + 1];  // where a chunk's collected weights start
  __shared__ u64 digit_mass[2][256];
  __shared__ float fscratch[16];
  __shared__ u64 uscratch[17];
  const int row = blockIdx.x;
  const float temp = temperature[row];
  if (!(temp > 0.f)) return;
  const RowState st = s.state[row];
  if (st.boundary < 0) return;
  const float mx = row_maximum(s.best_value, row, chunks, fscratch);
  const float* x = logits + static_cast<size_t>(row) * ld;
  const size_t rc0 = static_cast<size_t>(row) * chunks;

  u64 before, total;
  block_scan_u64(static_cast<int>(threadIdx.x) < chunks ? s.collected[rc0 + threadIdx.x] : 0, uscratch, &before,
                 &total);
  if (static_cast<int>(threadIdx.x) < chunks) first[threadIdx.x] = static_cast<uint32_t>(before);
  if (threadIdx.x == 0) first[chunks] = static_cast<uint32_t>(total);
  __syncthreads();
  const int count = static_cast<int>(total);
  const bool in_lds = count <= kBoundaryInLds;

  // entry k of chunk c's collected weights (chunk by chunk they are in index order)
  const auto weight_at = [&](int c, int k) {
    return weight_of(x[s.where[(rc0 + c) * kArgmaxChunk + k]], mx, temp);
  };
  if (in_lds) {
    // all of them at once: entry j lies in the chunk c with first[c] <= j < first[c + 1]
    for (int j = threadIdx.x; j < count; j += kThresholdThreads) {
      int lo = 0, hi = chunks;  // first[lo] <= j < first[hi]
      while (hi - lo > 1) {
        const int mid = (lo + hi) / 2;
        if (first[mid] <= static_cast<uint32_t>(j)) lo = mid; else hi = mid;
      }
      held[j] = weight_at(lo, j - static_cast<int>(first[lo]));
    }
    __syncthreads();
  }
  // f(q) for every collected weight q, dealt out to the threads
  const auto for_all = [&](auto f) {
    if (in_lds) {
      for (int j = threadIdx.x; j < count; j += kThresholdThreads) f(held[j]);
    } else {
      for (int c = 0; c < chunks; ++c) {
        const int n = first[c + 1] - first[c];
        for (int k = threadIdx.x; k < n; k += kThresholdThreads) f(weight_at(c, k));
      }
    }
  };

  // tau's high bits are the class's; the open ones are found eight at a time: among the
  // weights that share the bits found so far, the mass by the next eight bits, and from
  // the top the digit at which the upper mass reaches `need`.  A weight is a float's 24
  // bits shifted: below those every weight has zeros, which need no search.
  int open_bits;
  u64 found = class_base(st.boundary, &open_bits) >> open_bits;  // the bits known so far
  u64 above = st.above;                                          // mass of the weights above them
  const int zero_bits = open_bits > 20 ? open_bits - 20 : 0;     // (4 bits are the class's, 20 more may differ)
  const int lane = threadIdx.x & (kWave - 1);
  for (int phase = 0; open_bits > zero_bits; ++phase) {
    const int width = open_bits - zero_bits < 8 ? open_bits - zero_bits : 8, shift = open_bits - width;
    u64* mass = digit_mass[phase & 1];
    if (threadIdx.x < 256) mass[threadIdx.x] = 0;
    __syncthreads();
    for_all([&](u64 q) {
      if ((q >> open_bits) == found) atomicAdd(&mass[(q >> shift) & ((1u << width) - 1)], q);
    });
    __syncthreads();
    // Every wavefront finds the digit by itself, from the same 256 sums: lane l takes the
    // digits 255 - 4 l down to 252 - 4 l, a prefix sum over the lanes gives the mass above
    // them, and the first lane (highest digits) in which the upper mass reaches `need` tells.
    u64 own[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) own[i] = mass[255 - (4 * lane + i)], sum += own[i];
    u64 upto = sum;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const u64 o = __shfl_up(upto, off, kWave);
      if (lane >= off) upto += o;
    }
    u64 run = upto - sum, run_at_hit = 0;
    int hit = -1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (hit < 0 && above + run + own[i] >= st.need) hit = i, run_at_hit = run;
      run += own[i];
    }
    const unsigned long long reached = __ballot(hit >= 0);
    const int teller = reached ? __ffsll(reached) - 1 : kWave - 1;  // (some lane always reaches it)
    const int digit = __shfl(hit >= 0 ? 255 - (4 * lane + hit) : 0, teller, kWave);
    above += __shfl(hit >= 0 ? run_at_hit : run, teller, kWave);
    found = (found << width) | static_cast<u64>(digit);
    open_bits = shift;
  }
  found <<= open_bits;  // the bits that are zero in every weight
  const u64 tau = found;  // `above` is now the mass of all weights above tau
  u64 equal = 0;
  for_all([&](u64 q) { equal += q == tau; });
  equal = block_sum_u64(equal, uscratch);
  // weights equal to tau are kept while the mass before them is below `need`
  u64 admit = (st.need - above + tau - 1) / tau;
  admit = admit < 1 ? 1 : (admit > equal ? equal : admit);
  if (threadIdx.x == 0) {
    s.state[row].tau = tau;
    s.state[row].admit = static_cast<uint32_t>(admit);
  }
  // every chunk's kept mass (without the weights equal to tau) and the number of those
  for (int c = threadIdx.x; c < chunks; c += kThresholdThreads) {
    u64 mass = s.heavier[rc0 + c];
    uint32_t ties = 0;
    const int n = first[c + 1] - first[c];
    for (int k = 0; k < n; ++k) {
      const u64 q = in_lds ? held[first[c] + k] : weight_at(c, k);
      if (q > tau) mass += q;
      ties += q == tau;
    }
    s.kept_mass[rc0 + c] = mass;
    s.ties[rc0 + c] = ties;
  }
}

__global__ void __launch_bounds__(kChunkThreads)
    sample_draw_kernel(const float* __restrict__ logits, int32_t* __restrict__ out,
                       const float* __restrict__ temperature, const float* __restrict__ uniforms,
                       SampleScratch s, int vocab, int ld, int chunks, int nucleus) {
  __shared__ float lds[kChunkLds];
  __shared__ MaxIdx mscratch[16];
  __shared__ float fscratch[16];
  __shared__ u64 uscratch[17];
  __shared__ u64 found[3];  // the chunk of the draw, the kept mass and the equal weights before it
  const int row = blockIdx.x;
  const size_t rc0 = static_cast<size_t>(row) * chunks;
  // the argmax (only where it is the answer): chunks are in index order, so the first
  // maximum among them has the lowest index
  const auto greedy = [&]() {
    const MaxIdx best = block_argmax(s.best_value + rc0, chunks, mscratch);
    return s.best_index[rc0 + best.i];
  };
  const float temp = temperature[row];
  if (!(temp > 0.f)) {
    const int token = greedy();
    if (threadIdx.x == 0) out[row] = token;
    return;
  }
  u64 tau = 0;
  uint32_t admit = 0;
  if (nucleus) {
    const RowState st = s.state[row];
    if (st.boundary >= 0) tau = st.tau, admit = st.admit;
  }
  // Chunk c keeps its heavier weights and those equal to tau that are still admitted.
  // A thread takes kOwn neighbouring chunks; prefix sums over the threads give the
  // equal weights and the kept mass before them.
  constexpr int kOwn = kMaxChunks / kChunkThreads;
  const int c0 = threadIdx.x * kOwn;
  uint32_t own_ties[kOwn];
  u64 ties_sum = 0;
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    own_ties[i] = c0 + i < chunks ? s.ties[rc0 + c0 + i] : 0;
    ties_sum += own_ties[i];
  }
  u64 seen, all_ties;
  block_scan_u64(ties_sum, uscratch, &seen, &all_ties);
  u64 own_mass[kOwn], seen_at[kOwn], mass_sum = 0;
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const u64 room = admit > seen ? admit - seen : 0;
    own_mass[i] = c0 + i < chunks ? s.kept_mass[rc0 + c0 + i] + (own_ties[i] < room ? own_ties[i] : room) * tau : 0;
    seen_at[i] = seen;
    seen += own_ties[i];
    mass_sum += own_mass[i];
  }
  u64 run, kept;
  block_scan_u64(mass_sum, uscratch, &run, &kept);
  if (kept == 0) {  // nothing has any weight (a row of NaN): the argmax's answer
    const int token = greedy();
    if (threadIdx.x == 0) out[row] = token;
    return;
  }
  u64 target = static_cast<u64>(static_cast<double>(uniforms[row]) * static_cast<double>(kept));
  target = target < kept ? target : kept - 1;
  if (run <= target && target < run + mass_sum) {  // one thread's chunks span the target
#pragma unroll
    for (int i = 0; i < kOwn; ++i) {
      if (target >= run && target < run + own_mass[i]) found[0] = c0 + i, found[1] = run, found[2] = seen_at[i];
      run += own_mass[i];
    }
  }
  __syncthreads();
  const int chunk = static_cast<int>(found[0]);
  const float mx = row_maximum(s.best_value, row, chunks, fscratch);
  float x[kPerThread];
  const int begin = chunk * kArgmaxChunk;
  load_chunk(logits + static_cast<size_t>(row) * ld, begin, vocab, lds, x);
  u64 q[kPerThread];
  u64 my_ties = 0;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    q[k] = weight_of(x[k], mx, temp);
    if (tau && q[k] == tau) my_ties += 1;
  }
  u64 ties_before, ties_total;
  block_scan_u64(my_ties, uscratch, &ties_before, &ties_total);
  ties_before += found[2];
  uint32_t keep = 0;
  u64 my_mass = 0;
  {
    u64 equal_before = ties_before;
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
      bool taken = q[k] > tau;
      if (tau && q[k] == tau) {
        taken = equal_before < admit;
        equal_before += 1;
      }
      if (taken) keep |= 1u << k, my_mass += q[k];
    }
  }
  u64 mass_before, mass_total;
  block_scan_u64(my_mass, uscratch, &mass_before, &mass_total);
  mass_before += found[1];
  // exactly one thread's kept weights span the target
  if (my_mass > 0 && mass_before <= target && target < mass_before + my_mass) {
    u64 passed = mass_before;
    int token = begin;  // (always replaced: the thread's kept mass spans the target)
    bool done = false;
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {  // the first kept entry at which the running mass passes the target
      if (!(keep & (1u << k)) || done) continue;
      passed += q[k];
      if (passed > target) {
        token = begin + threadIdx.x * kPerThread + k;
        done = true;
      }
    }
    out[row] = token;
  }
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

extern "C" long long shk_sample_scratch_floats(int rows, int vocab) {
  if (rows <= 0 || vocab <= 0) return 0;
  const int chunks = (vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  return static_cast<long long>(sample_scratch_words(rows, chunks, nullptr, nullptr));
}

extern "C" int shk_sample(const float* logits, int32_t* out, const float* temperature,
                          const float* top_p, const float* uniforms, float* scratch,
                          long long scratch_floats, int rows, int vocab, int ld, int nucleus,
                          void* stream) {
  SHK_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%d",
              rows, vocab, ld);
  if (rows == 0) return 0;
  SHK_REQUIRE(logits && out && temperature && top_p && uniforms && scratch, "sample: null pointer");
  SHK_REQUIRE(rows <= 65535, "sample: at most 65535 rows a call, got %d", rows);
  const int chunks = (vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  SHK_REQUIRE(chunks <= kMaxChunks, "sample: a row of %d logits is beyond %d", vocab,
              kMaxChunks * kArgmaxChunk);
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(scratch) % 16 == 0, "sample: scratch is not 16-byte aligned");
  SampleScratch s;
  const size_t words = sample_scratch_words(rows, chunks, &s, scratch);
  SHK_REQUIRE(scratch_floats >= static_cast<long long>(words),
              "sample: scratch holds %lld floats, %lld are needed (shk_sample_scratch_floats)",
              scratch_floats, static_cast<long long>(words));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 by_chunk(chunks, rows);
  argmax_chunks_kernel<<<by_chunk, kArgmaxThreads, 0, st>>>(logits, s.best_value, s.best_index, vocab,
                                                            ld, chunks);
  SHK_LAUNCH_CHECK("sample");
  if (nucleus) {
    sample_weigh_kernel<true><<<by_chunk, kChunkThreads, 0, st>>>(logits, temperature, s, vocab, ld, chunks);
    SHK_LAUNCH_CHECK("sample");
    sample_boundary_kernel<<<rows, kBins, 0, st>>>(temperature, top_p, s, chunks);
    SHK_LAUNCH_CHECK("sample");
    sample_collect_kernel<<<by_chunk, kChunkThreads, 0, st>>>(logits, temperature, s, vocab, ld, chunks);
    SHK_LAUNCH_CHECK("sample");
    sample_threshold_kernel<<<rows, kThresholdThreads, 0, st>>>(logits, temperature, s, ld, chunks);
    SHK_LAUNCH_CHECK("sample");
  } else {
    sample_weigh_kernel<false><<<by_chunk, kChunkThreads, 0, st>>>(logits, temperature, s, vocab, ld, chunks);
    SHK_LAUNCH_CHECK("sample");
  }
  sample_draw_kernel<<<rows, kChunkThreads, 0, st>>>(logits, out, temperature, uniforms, s, vocab, ld,
                                                     chunks, nucleus);
  SHK_LAUNCH_CHECK("sample");
  return 0;
}
