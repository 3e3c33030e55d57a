// Rotary position encoding of queries and keys fused with the write of keys
// and values into their cache pages.  One workgroup per token.  Angles, sine
// and cosine are float32 (sincosf with full range reduction: positions reach
// thousands of radians at the highest frequency).
#include "api.h"
#include "common.h"

namespace shk {

constexpr int kMaxHalf = 256;  // rot_dim / 2 <= 256

template <typename T>
__global__ void __launch_bounds__(256)
    rope_kv_store_kernel(T* __restrict__ qkv, int heads, int kv_heads, int head_dim, int rot_dim,
                         const float* __restrict__ inv_freq, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ token_seq, const int32_t* __restrict__ tables,
                         int table_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
                         int page_size, int num_pages, int write_kv) {
  __shared__ float cs[kMaxHalf];
  __shared__ float sn[kMaxHalf];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot_dim / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float angle = static_cast<float>(pos) * inv_freq[i];
    float s, c;
    sincosf(angle, &s, &c);
    cs[i] = c;
    sn[i] = s;
  }
  __syncthreads();

  T* row = qkv + static_cast<size_t>(t) * (heads + 2 * kv_heads) * head_dim;
  size_t slot_row = 0;  // index of this token's [head_dim] row for kv head 0
  int page = 0;
  if (write_kv) {
    page = tables[static_cast<size_t>(token_seq[t]) * table_stride + pos / page_size];
    // The host builds tables that cover every position of the step; a page id
    // outside the pool would be a host bug, and is never dereferenced.
    if (page < 0 || page >= num_pages) write_kv = 0;
    slot_row = (static_cast<size_t>(page) * kv_heads) * page_size + pos % page_size;
  }
  const size_t head_rows = page_size;  // rows between consecutive kv heads of one page

  // queries: rotate in place
  for (int idx = threadIdx.x; idx < heads * half; idx += blockDim.x) {
    const int h = idx / half, i = idx % half;
    T* x = row + h * head_dim;
    const float x1 = to_float(x[i]), x2 = to_float(x[i + half]);
    x[i] = from_float<T>(x1 * cs[i] - x2 * sn[i]);
    x[i + half] = from_float<T>(x2 * cs[i] + x1 * sn[i]);
  }
  if (!write_kv) return;

  // keys: rotate into the page
  const T* krow = row + heads * head_dim;
  for (int idx = threadIdx.x; idx < kv_heads * half; idx += blockDim.x) {
    const int h = idx / half, i = idx % half;
    const T* x = krow + h * head_dim;
    T* dst = k_pool + (slot_row + h * head_rows) * head_dim;
    const float x1 = to_float(x[i]), x2 = to_float(x[i + half]);
    dst[i] = from_float<T>(x1 * cs[i] - x2 * sn[i]);
    dst[i + half] = from_float<T>(x2 * cs[i] + x1 * sn[i]);
  }
  const int tail = head_dim - rot_dim;  // elements that are not rotated
  for (int idx = threadIdx.x; idx < kv_heads * tail; idx += blockDim.x) {
    const int h = idx / tail, i = rot_dim + idx % tail;
    k_pool[(slot_row + h * head_rows) * head_dim + i] = krow[h * head_dim + i];
  }
  // values: stored transposed, [page][kv head][head_dim][page_size], so that the
  // keys of a page are contiguous for every element (the operand layout of P.V)
  const T* vrow = krow + kv_heads * head_dim;
  const size_t vbase = static_cast<size_t>(page) * kv_heads * head_dim * page_size + pos % page_size;
  for (int idx = threadIdx.x; idx < kv_heads * head_dim; idx += blockDim.x)
    v_pool[vbase + static_cast<size_t>(idx) * page_size] = vrow[idx];
}

}  // namespace shk

using namespace shk;

extern "C" int shk_rope_kv_store(void* qkv, int dtype, int n, int heads, int kv_heads,
                                 int head_dim, int rot_dim, const float* inv_freq,
                                 const int32_t* positions, const int32_t* token_seq,
                                 const int32_t* tables, int table_stride, void* k_pool,
                                 void* v_pool, int page_size, int num_pages, int write_kv,
                                 void* stream) {
  SHK_REQUIRE(dtype == kF32 || dtype == kBF16, "rope_kv_store: unknown dtype %d", dtype);
  SHK_REQUIRE(n >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0,
              "rope_kv_store: bad sizes n=%d heads=%d kv_heads=%d head_dim=%d", n, heads, kv_heads,
              head_dim);
  SHK_REQUIRE(rot_dim >= 0 && rot_dim <= head_dim && rot_dim % 2 == 0,
              "rope_kv_store: rot_dim %d must be even and at most head_dim %d", rot_dim, head_dim);
  SHK_REQUIRE(rot_dim / 2 <= kMaxHalf, "rope_kv_store: rot_dim %d exceeds %d", rot_dim,
              2 * kMaxHalf);
  if (n == 0) return 0;
  SHK_REQUIRE(qkv && positions, "rope_kv_store: null pointer");
  SHK_REQUIRE(rot_dim == 0 || inv_freq, "rope_kv_store: rotation needs inv_freq");
  if (write_kv) {
    SHK_REQUIRE(token_seq && tables && k_pool && v_pool, "rope_kv_store: null cache pointer");
    SHK_REQUIRE(page_size > 0 && num_pages > 0 && table_stride > 0,
                "rope_kv_store: bad cache sizes page_size=%d num_pages=%d table_stride=%d",
                page_size, num_pages, table_stride);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32)
    rope_kv_store_kernel<float><<<n, 256, 0, s>>>(
        static_cast<float*>(qkv), heads, kv_heads, head_dim, rot_dim, inv_freq, positions,
        token_seq, tables, table_stride, static_cast<float*>(k_pool), static_cast<float*>(v_pool),
        page_size, num_pages, write_kv);
  else
    rope_kv_store_kernel<bf16><<<n, 256, 0, s>>>(
        static_cast<bf16*>(qkv), heads, kv_heads, head_dim, rot_dim, inv_freq, positions,
        token_seq, tables, table_stride, static_cast<bf16*>(k_pool), static_cast<bf16*>(v_pool),
        page_size, num_pages, write_kv);
  SHK_LAUNCH_CHECK("rope_kv_store");
  return 0;
}
