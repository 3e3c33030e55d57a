// Causal grouped-query attention over paged key/value caches.
//
// attention_generic_kernel: one workgroup per (query token, query head), for
// any head size up to 256, any page size, any number of heads and groups,
// float32 or bfloat16 storage.  Scores, softmax and the weighted sum of values
// are float32.  It walks the keys of the token's sequence in tiles of 256
// through the block table, with a running maximum and sum, so prompt portions
// and single decoded tokens take the same path and the same order of
// operations: a token's result does not depend on how the step was cut.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kAttnThreads = 256;
constexpr int kMaxHeadDim = 256;

template <typename T>
__global__ void __launch_bounds__(kAttnThreads)
    attention_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out,
                             int heads, int kv_heads, int head_dim,
                             const int32_t* __restrict__ positions,
                             const int32_t* __restrict__ token_seq,
                             const int32_t* __restrict__ tables, int table_stride,
                             const T* __restrict__ k_pool, const T* __restrict__ v_pool,
                             int page_size, int num_pages, int window, float scale) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float probs[kAttnThreads];
  __shared__ int32_t rows[kAttnThreads];  // key-cache row of each key of the tile, -1 if masked
  __shared__ float scratch[16];
  __shared__ float partial[kAttnThreads];

  const int head = blockIdx.x, t = blockIdx.y;
  const int kvh = head / (heads / kv_heads);
  const int pos = positions[t];
  const int32_t* table = tables + static_cast<size_t>(token_seq[t]) * table_stride;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  const T* qrow = q + static_cast<size_t>(t) * q_stride + head * head_dim;
  for (int d = threadIdx.x; d < head_dim; d += kAttnThreads) qs[d] = to_float(qrow[d]);
  __syncthreads();

  // PV ownership: thread (g, d) sums keys jj = g, g + groups, ... of a tile for element d.
  const int groups = kAttnThreads / head_dim;  // >= 1 because head_dim <= 256
  const int g = threadIdx.x / head_dim, d = threadIdx.x % head_dim;
  const bool pv_active = g < groups;

  float m_run = -INFINITY, l_run = 0.f, acc = 0.f;
  for (int j0 = lo; j0 <= pos; j0 += kAttnThreads) {
    const int j = j0 + threadIdx.x;
    float s = -INFINITY;
    int32_t row = -1;
    if (j <= pos) {
      const int page = table[j / page_size];
      if (page >= 0 && page < num_pages) {
        row = (page * kv_heads + kvh) * page_size + j % page_size;
        // keys are stored in slabs: [head_dim / slab][page_size][slab] per page and head
        const int slab = key_slab(head_dim);
        const T* kr = k_pool + static_cast<size_t>(page * kv_heads + kvh) * page_size * head_dim +
                      static_cast<size_t>(j % page_size) * slab;
        float dot = 0.f;
        for (int e0 = 0; e0 < head_dim; e0 += slab) {
          for (int e = 0; e < slab; ++e) dot = fmaf(qs[e0 + e], to_float(kr[e]), dot);
          kr += static_cast<size_t>(page_size) * slab;
        }
        s = dot * scale;
      }
    }
    const float m_new = fmaxf(m_run, block_max(s, scratch));
    const float p = (row >= 0) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m_run - m_new);  // 0 on the first tile (m_run = -inf)
    probs[threadIdx.x] = p;
    rows[threadIdx.x] = row;
    const float tile_sum = block_sum(p, scratch);  // has the barriers that publish probs/rows
    l_run = l_run * alpha + tile_sum;
    m_run = m_new;
    if (pv_active) {
      float a = 0.f;
      const int count = (pos - j0 + 1 < kAttnThreads) ? pos - j0 + 1 : kAttnThreads;
      for (int jj = g; jj < count; jj += groups) {
        const int32_t r = rows[jj];
        if (r < 0) continue;
        // values are stored [page][kv head][head_dim][page_size]
        const size_t v_at =
            (static_cast<size_t>(r / page_size) * head_dim + d) * page_size + r % page_size;
        a = fmaf(probs[jj], to_float(v_pool[v_at]), a);
      }
      acc = acc * alpha + a;
    }
    __syncthreads();  // probs/rows are rewritten by the next tile
  }

  partial[threadIdx.x] = pv_active ? acc : 0.f;
  __syncthreads();
  if (threadIdx.x < head_dim) {
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += partial[gg * head_dim + threadIdx.x];
    out[static_cast<size_t>(t) * heads * head_dim + head * head_dim + threadIdx.x] =
        from_float<T>(total / l_run);
  }
}

}  // namespace shk

using namespace shk;

extern "C" int shk_attention(const void* q, int q_stride, void* out, int dtype, int n, int heads,
                             int kv_heads, int head_dim, const int32_t* positions,
                             const int32_t* token_seq, const int32_t* tables, int table_stride,
                             int num_seqs, const void* k_pool, const void* v_pool, int page_size,
                             int num_pages, int window, float scale, void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "attention: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
              "attention: heads=%d must be a positive multiple of kv_heads=%d", heads, kv_heads);
  SHK_REQUIRE(head_dim > 0 && head_dim <= kMaxHeadDim,
              "attention: head_dim %d is outside 1..%d", head_dim, kMaxHeadDim);
  SHK_REQUIRE(q_stride >= heads * head_dim, "attention: q_stride %d < heads*head_dim %d", q_stride,
              heads * head_dim);
  SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0 && num_seqs > 0,
              "attention: bad cache sizes page_size=%d num_pages=%d table_stride=%d num_seqs=%d",
              page_size, num_pages, table_stride, num_seqs);
  SHK_REQUIRE(static_cast<int64_t>(num_pages) * kv_heads * page_size < (1LL << 31),
              "attention: cache pool has too many rows for 32-bit row indices");
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 65535, "attention: at most 65535 tokens a call, got %d", n);
  SHK_REQUIRE(q && out && positions && token_seq && tables && k_pool && v_pool,
              "attention: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(heads, n);
  if (dtype == kF32)
    attention_generic_kernel<float><<<grid, kAttnThreads, 0, s>>>(
        static_cast<const float*>(q), q_stride, static_cast<float*>(out), heads, kv_heads, head_dim,
        positions, token_seq, tables, table_stride, static_cast<const float*>(k_pool),
        static_cast<const float*>(v_pool), page_size, num_pages, window, scale);
  else
    attention_generic_kernel<bf16><<<grid, kAttnThreads, 0, s>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), heads, kv_heads, head_dim,
        positions, token_seq, tables, table_stride, static_cast<const bf16*>(k_pool),
        static_cast<const bf16*>(v_pool), page_size, num_pages, window, scale);
  SHK_LAUNCH_CHECK("attention");
  return 0;
}
