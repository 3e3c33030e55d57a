// Rotary position encoding of queries and keys fused with the write of keys
// and values into their cache pages.  One thread per element pair (queries and
// keys) or element (values); a workgroup first tabulates the cosines and sines
// of its token in LDS.  Angles are float32 products as in the reference.  The projections may arrive as the float32 partial sums of a
// product that was split along k; they are added here, in order, with the bias.
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kMaxHalf = 256;  // rot_dim / 2 <= 256
constexpr int kRopeThreads = 256;

template <typename T>
__global__ void __launch_bounds__(kRopeThreads)
    rope_kv_store_kernel(T* __restrict__ qkv, int n, int heads, int kv_heads, int head_dim,
                         int rot_dim, const float* __restrict__ inv_freq,
                         const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables,
                         int table_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
                         int page_size, int num_pages, int write_kv,
                         const float* __restrict__ parts, int splits,
                         const float* __restrict__ bias) {
  __shared__ float cs[kMaxHalf];
  __shared__ float sn[kMaxHalf];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot_dim / 2;
  const int width = (heads + 2 * kv_heads) * head_dim;
  T* row = qkv + static_cast<size_t>(t) * width;

  // What this thread moves: a rotated pair, an element behind the rotated part,
  // or an element of the values.  Its inputs are requested first, so that they
  // travel while the cosines and sines are tabulated.
  const int tail = head_dim - rot_dim;  // elements that are not rotated
  const int n_pairs = (heads + kv_heads) * half;
  const int n_tail = (heads + kv_heads) * tail;
  const int n_values = kv_heads * head_dim;
  const int item = blockIdx.y * kRopeThreads + threadIdx.x;
  enum { kPairItem, kTailItem, kValueItem, kNone } role = kNone;
  int h = 0, i = 0, col = 0;
  if (item < n_pairs) {
    role = kPairItem;
    h = item / half, i = item % half;
    col = h * head_dim + i;
  } else if (item < n_pairs + n_tail) {
    role = kTailItem;
    const int e = item - n_pairs;
    h = e / tail, i = rot_dim + e % tail;
    col = h * head_dim + i;
  } else if (item < n_pairs + n_tail + n_values) {
    role = kValueItem;
    i = item - n_pairs - n_tail;  // kv head * head_dim + element
    col = (heads + kv_heads) * head_dim + i;
  }
  // columns `col` and (for a pair) `col + half` of this token's projections; the
  // parts of a split product are added in order, eight of them in flight
  float x1 = 0.f, x2 = 0.f;
  if (role != kNone) {
    const bool two = role == kPairItem;
    if (splits == 0) {
      x1 = to_float(row[col]);
      if (two) x2 = to_float(row[col + half]);
    } else {
      const size_t split_stride = static_cast<size_t>(n) * width;
      const float* p = parts + static_cast<size_t>(t) * width + col;
      for (int z0 = 0; z0 < splits; z0 += 8) {
        float a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const bool have = z0 + u < splits;
          a[u] = have ? p[(z0 + u) * split_stride] : 0.f;
          b[u] = have && two ? p[(z0 + u) * split_stride + half] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          x1 += a[u];
          x2 += b[u];
        }
      }
      if (bias) {
        x1 += bias[col];
        if (two) x2 += bias[col + half];
      }
    }
  }

  int page = -1;
  if (write_kv) {
    page = tables[static_cast<size_t>(token_seq[t]) * table_stride + pos / page_size];
    // The host builds tables that cover every position of the step; a page id
    // outside the pool would be a host bug, and is never dereferenced.
    if (page < 0 || page >= num_pages) page = -1;
  }
  const int slot = pos % page_size;
  // keys [page][kv head] in slabs (key_offset); values transposed [page][kv head][head_dim][slot]
  const size_t page_base = static_cast<size_t>(page < 0 ? 0 : page) * kv_heads * page_size * head_dim;

  for (int f = threadIdx.x; f < half; f += kRopeThreads) {
    // The angle is the float32 product, as the reference forms it; it reaches
    // thousands of radians, so it is brought into [-pi, pi] in float64 (exact
    // to 1e-13) before the float32 sine and cosine.
    const float angle = static_cast<float>(pos) * inv_freq[f];
    const double a = static_cast<double>(angle);
    const double turns = rint(a * 0.15915494309189535);
    const float reduced = static_cast<float>(fma(turns, -6.283185307179586, a));
    float sv, cv;
    sincosf(reduced, &sv, &cv);
    cs[f] = cv;
    sn[f] = sv;
  }
  __syncthreads();

  if (role == kPairItem) {
    const float o1 = x1 * cs[i] - x2 * sn[i], o2 = x2 * cs[i] + x1 * sn[i];
    if (h < heads) {
      row[col] = from_float<T>(o1);
      row[col + half] = from_float<T>(o2);
    } else if (page >= 0) {
      T* dst = k_pool + page_base + static_cast<size_t>(h - heads) * page_size * head_dim;
      dst[key_offset(slot, i, page_size, head_dim)] = from_float<T>(o1);
      dst[key_offset(slot, i + half, page_size, head_dim)] = from_float<T>(o2);
    }
  } else if (role == kTailItem) {
    if (h < heads) {
      row[col] = from_float<T>(x1);
    } else if (page >= 0) {
      k_pool[page_base + static_cast<size_t>(h - heads) * page_size * head_dim +
             key_offset(slot, i, page_size, head_dim)] = from_float<T>(x1);
    }
  } else if (role == kValueItem) {
    if (page >= 0) v_pool[page_base + static_cast<size_t>(i) * page_size + slot] = from_float<T>(x1);
  }
}

// The same for bfloat16 rows that are rotated whole (rot_dim == head_dim, a
// multiple of 16): one workgroup per token, a thread moves 8 neighbouring
// elements at a time (16 bytes; a rotated pair is two such runs, head_dim / 2
// apart), so that queries and keys travel in whole vectors.  Values go to
// their transposed pages element by element.  Arithmetic as above.
constexpr int kVecItems = 4;  // runs (or pairs of runs) per thread at most
// from this many tokens on; fewer (decode steps) are a matter of latency, which the
// kernel above with its ten workgroups per token and eight parts in flight handles better
constexpr int kVecMinTokens = 65;

__global__ void __launch_bounds__(kRopeThreads)
    rope_kv_store_vec_kernel(bf16* __restrict__ qkv, int n, int heads, int kv_heads, int head_dim,
                             const float* __restrict__ inv_freq,
                             const int32_t* __restrict__ positions,
                             const int32_t* __restrict__ token_seq,
                             const int32_t* __restrict__ tables, int table_stride,
                             bf16* __restrict__ k_pool, bf16* __restrict__ v_pool, int page_size,
                             int num_pages, int write_kv, const float* __restrict__ parts, int splits,
                             const float* __restrict__ bias) {
  __shared__ float cs[kMaxHalf];
  __shared__ float sn[kMaxHalf];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = head_dim / 2;
  const int width = (heads + 2 * kv_heads) * head_dim;
  bf16* row = qkv + static_cast<size_t>(t) * width;
  const int per_head = half / 8;                      // pairs of runs in a rotated head
  const int n_pairs = (heads + kv_heads) * per_head;  // queries, then keys
  const int n_values = kv_heads * (head_dim / 8);
  const size_t split_stride = static_cast<size_t>(n) * width;

  // 8 elements from column `col` on: the row itself, or the sum of its parts and the bias
  auto fetch = [&](int col, float (&x)[8]) {
    if (splits == 0) {
      const uint4 raw = *reinterpret_cast<const uint4*>(row + col);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[2 * e] = __uint_as_float(w[e] << 16);
        x[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
      }
      return;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = 0.f;
    const float* p = parts + static_cast<size_t>(t) * width + col;
    for (int z0 = 0; z0 < splits; z0 += 4) {  // four parts in flight, added in order
      float4 lo[4], hi[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int z = z0 + u < splits ? z0 + u : splits - 1;
        lo[u] = *reinterpret_cast<const float4*>(p + z * split_stride);
        hi[u] = *reinterpret_cast<const float4*>(p + z * split_stride + 4);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool have = z0 + u < splits;  // (past the last part: the last one again, not added)
        x[0] += have ? lo[u].x : 0.f, x[1] += have ? lo[u].y : 0.f;
        x[2] += have ? lo[u].z : 0.f, x[3] += have ? lo[u].w : 0.f;
        x[4] += have ? hi[u].x : 0.f, x[5] += have ? hi[u].y : 0.f;
        x[6] += have ? hi[u].z : 0.f, x[7] += have ? hi[u].w : 0.f;
      }
    }
    if (bias) {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] += bias[col + e];
    }
  };
  auto pack = [](const float (&x)[8]) {
    uint4 out;
    out.x = bf16_bits(x[0]) | (static_cast<uint32_t>(bf16_bits(x[1])) << 16);
    out.y = bf16_bits(x[2]) | (static_cast<uint32_t>(bf16_bits(x[3])) << 16);
    out.z = bf16_bits(x[4]) | (static_cast<uint32_t>(bf16_bits(x[5])) << 16);
    out.w = bf16_bits(x[6]) | (static_cast<uint32_t>(bf16_bits(x[7])) << 16);
    return out;
  };

  // this thread's items, fetched before the table of cosines and sines is made
  float a[kVecItems][8], b[kVecItems][8];
#pragma unroll
  for (int u = 0; u < kVecItems; ++u) {
    const int item = threadIdx.x + u * kRopeThreads;
    if (item < n_pairs) {
      const int col = (item / per_head) * head_dim + (item % per_head) * 8;
      fetch(col, a[u]);
      fetch(col + half, b[u]);
    } else if (item < n_pairs + n_values) {
      fetch((heads + kv_heads) * head_dim + (item - n_pairs) * 8, a[u]);
    }
  }

  int page = -1;
  if (write_kv) {
    page = tables[static_cast<size_t>(token_seq[t]) * table_stride + pos / page_size];
    if (page < 0 || page >= num_pages) page = -1;  // a host bug; never dereferenced
  }
  const int slot = pos % page_size;
  const size_t page_base = static_cast<size_t>(page < 0 ? 0 : page) * kv_heads * page_size * head_dim;

  for (int f = threadIdx.x; f < half; f += kRopeThreads) {
    const float angle = static_cast<float>(pos) * inv_freq[f];
    const double wide = static_cast<double>(angle);
    const double turns = rint(wide * 0.15915494309189535);
    const float reduced = static_cast<float>(fma(turns, -6.283185307179586, wide));
    float sv, cv;
    sincosf(reduced, &sv, &cv);
    cs[f] = cv;
    sn[f] = sv;
  }
  __syncthreads();

#pragma unroll
  for (int u = 0; u < kVecItems; ++u) {
    const int item = threadIdx.x + u * kRopeThreads;
    if (item < n_pairs) {
      const int h = item / per_head, i = (item % per_head) * 8;
      float lo[8], hi[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        lo[e] = a[u][e] * cs[i + e] - b[u][e] * sn[i + e];
        hi[e] = b[u][e] * cs[i + e] + a[u][e] * sn[i + e];
      }
      if (h < heads) {
        *reinterpret_cast<uint4*>(row + h * head_dim + i) = pack(lo);
        *reinterpret_cast<uint4*>(row + h * head_dim + i + half) = pack(hi);
      } else if (page >= 0) {
        bf16* dst = k_pool + page_base + static_cast<size_t>(h - heads) * page_size * head_dim;
        *reinterpret_cast<uint4*>(dst + key_offset(slot, i, page_size, head_dim)) = pack(lo);
        *reinterpret_cast<uint4*>(dst + key_offset(slot, i + half, page_size, head_dim)) = pack(hi);
      }
    } else if (item < n_pairs + n_values && page >= 0) {
      const int d0 = (item - n_pairs) * 8;  // kv head * head_dim + element
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v_pool[page_base + static_cast<size_t>(d0 + e) * page_size + slot] = from_float<bf16>(a[u][e]);
    }
  }
}

}  // namespace shk

using namespace shk;

extern "C" int shk_rope_kv_store(void* qkv, int dtype, int n, int heads, int kv_heads,
                                 int head_dim, int rot_dim, const float* inv_freq,
                                 const int32_t* positions, const int32_t* token_seq,
                                 const int32_t* tables, int table_stride, void* k_pool,
                                 void* v_pool, int page_size, int num_pages, int write_kv,
                                 const float* parts, int splits, const float* bias,
                                 void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "rope_kv_store: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0,
              "rope_kv_store: bad sizes n=%d heads=%d kv_heads=%d head_dim=%d", n, heads, kv_heads,
              head_dim);
  SHK_REQUIRE(rot_dim >= 0 && rot_dim <= head_dim && rot_dim % 2 == 0,
              "rope_kv_store: rot_dim %d must be even and at most head_dim %d", rot_dim, head_dim);
  SHK_REQUIRE(rot_dim / 2 <= kMaxHalf, "rope_kv_store: rot_dim %d exceeds %d", rot_dim,
              2 * kMaxHalf);
  SHK_REQUIRE(splits >= 0 && (splits == 0 || parts), "rope_kv_store: partial sums without a pointer");
  if (n == 0) return 0;
  SHK_REQUIRE(n <= 2147483647 / ((heads + 2 * kv_heads) * head_dim),
              "rope_kv_store: too many tokens (%d)", n);
  SHK_REQUIRE(qkv && positions, "rope_kv_store: null pointer");
  SHK_REQUIRE(rot_dim == 0 || inv_freq, "rope_kv_store: rotation needs inv_freq");
  if (write_kv) {
    SHK_REQUIRE(token_seq && tables && k_pool && v_pool, "rope_kv_store: null cache pointer");
    SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0,
                "rope_kv_store: bad cache sizes page_size=%d num_pages=%d table_stride=%d",
                page_size, num_pages, table_stride);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // whole vectors where the layout allows: bfloat16, rows rotated whole, 16-byte alignment
  const int vec_items = (heads + kv_heads) * (head_dim / 16) + kv_heads * (head_dim / 8);
  if (dtype == kBF16 && rot_dim == head_dim && head_dim % 16 == 0 && n >= kVecMinTokens &&
      vec_items <= kVecItems * kRopeThreads && reinterpret_cast<uintptr_t>(qkv) % 16 == 0 &&
      (!write_kv || reinterpret_cast<uintptr_t>(k_pool) % 16 == 0) &&
      (!parts || reinterpret_cast<uintptr_t>(parts) % 16 == 0)) {
    rope_kv_store_vec_kernel<<<n, kRopeThreads, 0, s>>>(
        static_cast<bf16*>(qkv), n, heads, kv_heads, head_dim, inv_freq, positions, token_seq, tables,
        table_stride, static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool), page_size, num_pages,
        write_kv, parts, splits, bias);
    SHK_LAUNCH_CHECK("rope_kv_store");
    return 0;
  }
  const int items = (heads + kv_heads) * (head_dim - rot_dim / 2) + kv_heads * head_dim;
  dim3 grid(n, (items + kRopeThreads - 1) / kRopeThreads);
  SHK_REQUIRE(grid.y <= 65535, "rope_kv_store: too many elements per token");
  if (dtype == kF32)
    rope_kv_store_kernel<float><<<grid, kRopeThreads, 0, s>>>(
        static_cast<float*>(qkv), n, heads, kv_heads, head_dim, rot_dim, inv_freq, positions,
        token_seq, tables, table_stride, static_cast<float*>(k_pool), static_cast<float*>(v_pool),
        page_size, num_pages, write_kv, parts, splits, bias);
  else
    rope_kv_store_kernel<bf16><<<grid, kRopeThreads, 0, s>>>(
        static_cast<bf16*>(qkv), n, heads, kv_heads, head_dim, rot_dim, inv_freq, positions,
        token_seq, tables, table_stride, static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool),
        page_size, num_pages, write_kv, parts, splits, bias);
  SHK_LAUNCH_CHECK("rope_kv_store");
  return 0;
}
