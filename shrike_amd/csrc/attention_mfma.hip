// bfloat16 attention over the paged cache on the MFMA units (gfx950).
//
// One wavefront owns a tile of 16 "rows" that share a key/value head of one
// sequence: for a prompt portion the rows are 16 consecutive queries of one
// query head; for a decoded token they are the query heads of one group
// (padded to 16).  The wavefront walks its key range in chunks of 32 keys:
//
//   S = Q K^T      two 16x16 tiles, v_mfma_f32_16x16x32_bf16 over head_dim;
//                  K rows are read straight from the page ([slot][head_dim])
//   softmax        running maximum and sum per row in float32, exp in float32
//   O += P V       P goes through LDS into operand layout; V is stored
//                  transposed in the cache ([head_dim][slot]), so 8 keys of one
//                  element are one 16-byte load
//
// Decode splits a sequence's keys over several wavefronts; each writes an
// unnormalised partial (O, max, sum) and attention_merge_kernel combines them
// in a fixed order.  Head sizes: multiples of 32 up to 256; page sizes:
// multiples of 16; up to 16 query heads per key/value head.  Other shapes are
// served by the general kernel.
#include "api.h"
#include "common.h"

namespace shk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

union AFrag {
  uint4 u;
  bf16x8 v;
  uint16_t h[8];
};

// Maximum and sum over the 16 lanes that hold one row of a score tile (lanes
// 16*g .. 16*g+15, a DPP "row"): four data-parallel-primitive moves on the vector
// unit instead of four round trips through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]: lane ^ 1
  v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]: lane ^ 2
  v = fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror: the other quad of each 8 lanes
  v = fmaxf(v, dpp_move<0x140>(v));  // row_mirror: the other half of the 16 lanes
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  v += dpp_move<0x141>(v);
  v += dpp_move<0x140>(v);
  return v;
}

constexpr int kPStride = 40;  // bf16 elements per row of the P tile in LDS (32 + padding)

// A window of 64 entries of a sequence's block table held across the lanes of
// the wavefront (lane i: entry base + i), so that finding a key's page is a
// register exchange instead of a load that the key and value loads wait for.
struct PageWindow {
  int base;     // index of the first entry held
  int32_t mine;  // this lane's entry
};

__device__ __forceinline__ PageWindow load_pages(const int32_t* table, int first, int last) {
  // entries first .. first + 63, none beyond `last` (the last entry the keys reach)
  PageWindow w;
  w.base = first;
  const int i = first + static_cast<int>(threadIdx.x % kWave);
  w.mine = (i <= last) ? table[i] : 0;
  return w;
}

__device__ __forceinline__ int page_at(const PageWindow& w, int entry) {
  return __shfl(w.mine, entry - w.base, kWave);
}

struct TileArgs {
  const int32_t* table;  // block table of the sequence
  const bf16* k_pool;    // [pages][kv_heads][page_size][D]
  const bf16* v_pool;    // [pages][kv_heads][D][page_size]
  int page_size;
  int kv_heads;
  int kvh;
  float scale;
};

// The operands of one chunk of 32 keys: K rows for two score tiles and the
// transposed V columns for P.V.
template <int D>
struct Chunk {
  AFrag k[2][D / 32];
  AFrag v[D / 16];
};

// Issues every load of the chunk at key `kb`; tiles and key groups that no row
// reads (beyond pos_max, before lo_min) are not touched and read as zero.
template <int D>
__device__ __forceinline__ void load_chunk(Chunk<D>& c, const TileArgs& ta, const PageWindow& pw,
                                           int kb, int pos_max, int lo_min) {
  const int lane = threadIdx.x % kWave;
  const int j = lane % 16, kg = lane / 16;
  const int ps = ta.page_size;
  const size_t head_elems = static_cast<size_t>(ps) * D;  // one kv head of one page
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    const int key0 = kb + tt * 16;
    const bool live = key0 <= pos_max && key0 + 15 >= lo_min;
    const bf16* krow = nullptr;
    const int kpage = page_at(pw, (key0 <= pos_max ? key0 : pos_max) / ps);
    if (live) {
      const int page = kpage;
      krow = ta.k_pool + (static_cast<size_t>(page) * ta.kv_heads + ta.kvh) * head_elems +
             static_cast<size_t>(key0 % ps + j) * D + kg * 8;
    }
#pragma unroll
    for (int ds = 0; ds < D / 32; ++ds) {
      c.k[tt][ds].u = make_uint4(0, 0, 0, 0);
      if (live) c.k[tt][ds].u = *reinterpret_cast<const uint4*>(krow + ds * 32);
    }
  }
  // this lane supplies keys kb + 8*kg .. +8 of element db*16 + j
  const int g0 = kb + kg * 8;
  const bool live = g0 <= pos_max && g0 + 7 >= lo_min;
  const bf16* vcol = nullptr;
  const int vpage = page_at(pw, (g0 <= pos_max ? g0 : pos_max) / ps);
  if (live) {
    const int page = vpage;
    vcol = ta.v_pool + (static_cast<size_t>(page) * ta.kv_heads + ta.kvh) * head_elems +
           static_cast<size_t>(j) * ps + g0 % ps;
  }
#pragma unroll
  for (int db = 0; db < D / 16; ++db) {
    c.v[db].u = make_uint4(0, 0, 0, 0);
    if (live) c.v[db].u = *reinterpret_cast<const uint4*>(vcol + static_cast<size_t>(db) * 16 * ps);
  }
}

// Walks keys [key_begin, key_end) (key_begin a multiple of 32) for 16 rows.
// qf: the rows' queries as A operands.  row_pos / row_lo: for this lane's four
// accumulator rows (4*(lane/16) + r), the last and first key each may read.
// pos_max / lo_min: the same bounds over all 16 rows.  The next chunk's loads
// are in flight while the current chunk is computed.
template <int D>
__device__ __forceinline__ void attend_tile(const TileArgs& ta, const AFrag (&qf)[D / 32],
                                            const int (&row_pos)[4], const int (&row_lo)[4],
                                            int pos_max, int lo_min, int key_begin, int key_end,
                                            f32x4 (&o)[D / 16], float (&m)[4], float (&l)[4],
                                            uint16_t* p_lds) {
  const int lane = threadIdx.x % kWave;
  const int j = lane % 16, kg = lane / 16;

  const int ps = ta.page_size;
  const int last_entry = pos_max / ps;
  PageWindow pw = load_pages(ta.table, key_begin / ps, last_entry);
  Chunk<D> cur, nxt;
  if (key_begin < key_end) load_chunk<D>(cur, ta, pw, key_begin, pos_max, lo_min);
  for (int kb = key_begin; kb < key_end; kb += 32) {
    if (kb + 32 < key_end) {
      // the window must hold the entries of keys kb + 32 .. kb + 63
      if ((kb + 63) / ps >= pw.base + kWave) pw = load_pages(ta.table, (kb + 32) / ps, last_entry);
      load_chunk<D>(nxt, ta, pw, kb + 32, pos_max, lo_min);
    }

    // ---- S = Q K^T for two tiles of 16 keys
    f32x4 s[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ds = 0; ds < D / 32; ++ds)
        s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ds].v, cur.k[tt][ds].v, s[tt], 0, 0, 0);
    }

    // ---- mask, running maximum and sum (lane holds key kb + tt*16 + j for rows 4*kg + r)
    float p[2][4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sc[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const int key = kb + tt * 16 + j;
        const bool keep = key <= row_pos[r] && key >= row_lo[r];
        sc[tt] = keep ? s[tt][r] * ta.scale : -INFINITY;
      }
      const float mx = row16_max(fmaxf(sc[0], sc[1]));
      const float m_new = fmaxf(m[r], mx);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __expf(m[r] - m_safe);
      p[0][r] = __expf(sc[0] - m_safe);
      p[1][r] = __expf(sc[1] - m_safe);
      const float sum = row16_sum(p[0][r] + p[1][r]);
      l[r] = l[r] * alpha + sum;
      m[r] = m_new;
#pragma unroll
      for (int db = 0; db < D / 16; ++db) o[db][r] *= alpha;
    }

    // ---- P through LDS into A-operand layout: rows 16, keys 32
    __syncthreads();  // the previous chunk's reads are done (one wavefront per workgroup)
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        p_lds[(kg * 4 + r) * kPStride + tt * 16 + j] = bf16_bits(p[tt][r]);
    __syncthreads();
    AFrag pf;
    pf.u = *reinterpret_cast<const uint4*>(p_lds + j * kPStride + kg * 8);

    // ---- O += P V.  Keys outside [lo_min, pos_max] carry weight 0 but their
    // slots may hold anything: zero them so that 0 * x stays 0.
    const int g0 = kb + kg * 8;
    uint4 keep_bits = make_uint4(~0u, ~0u, ~0u, ~0u);
    if (g0 < lo_min || g0 + 7 > pos_max) {
      uint32_t w[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool a = g0 + 2 * e >= lo_min && g0 + 2 * e <= pos_max;
        const bool b = g0 + 2 * e + 1 >= lo_min && g0 + 2 * e + 1 <= pos_max;
        w[e] = (a ? 0x0000ffffu : 0u) | (b ? 0xffff0000u : 0u);
      }
      keep_bits = make_uint4(w[0], w[1], w[2], w[3]);
    }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      AFrag vf = cur.v[db];
      vf.u.x &= keep_bits.x;
      vf.u.y &= keep_bits.y;
      vf.u.z &= keep_bits.z;
      vf.u.w &= keep_bits.w;
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf.v, vf.v, o[db], 0, 0, 0);
    }
    cur = nxt;
  }
}

// ------------------------------------------------------------------- decode
// grid (kv_heads, sequences, splits), one wavefront per workgroup.

template <int D>
__global__ void __launch_bounds__(kWave)
    attention_decode_kernel(const bf16* __restrict__ q, int q_stride, int heads, int kv_heads,
                            const int32_t* __restrict__ positions,
                            const int32_t* __restrict__ tables, int table_stride,
                            const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
                            int page_size, int window, float scale, float* __restrict__ partial,
                            int nsplit) {
  __shared__ __attribute__((aligned(16))) uint16_t p_lds[16 * kPStride];
  const int kvh = blockIdx.x, seq = blockIdx.y, z = blockIdx.z;
  const int lane = threadIdx.x, j = lane % 16, kg = lane / 16;
  const int group = heads / kv_heads;
  // decode sequences come first in the step: token index == sequence index
  const int pos = positions[seq];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  // this split's keys: chunks of 32 from the chunk that holds `lo`
  const int first = lo & ~31;
  const int chunks = (pos - first) / 32 + 1;
  const int per = (chunks + nsplit - 1) / nsplit;
  const int key_begin = first + z * per * 32;
  int key_end = key_begin + per * 32;
  if (key_end > pos + 1) key_end = pos + 1;

  float m[4], l[4];
  f32x4 o[D / 16];
#pragma unroll
  for (int r = 0; r < 4; ++r) m[r] = -INFINITY, l[r] = 0.f;
#pragma unroll
  for (int db = 0; db < D / 16; ++db) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (key_begin <= pos) {
    AFrag qf[D / 32];
    const bf16* qrow = q + static_cast<size_t>(seq) * q_stride +
                       static_cast<size_t>(kvh * group + j) * D + kg * 8;
#pragma unroll
    for (int ds = 0; ds < D / 32; ++ds) {
      qf[ds].u = make_uint4(0, 0, 0, 0);
      if (j < group) qf[ds].u = *reinterpret_cast<const uint4*>(qrow + ds * 32);
    }
    const int row_pos[4] = {pos, pos, pos, pos};
    const int row_lo[4] = {lo, lo, lo, lo};
    TileArgs ta{tables + static_cast<size_t>(seq) * table_stride, k_pool, v_pool, page_size,
                kv_heads, kvh, scale};
    attend_tile<D>(ta, qf, row_pos, row_lo, pos, lo, key_begin, key_end, o, m, l, p_lds);
  }

  // partial[seq][head][split] = {O[D], max, sum}; lane holds element db*16 + j of rows 4*kg + r
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int hrow = kg * 4 + r;
    if (hrow >= group) continue;
    float* dst = partial + ((static_cast<size_t>(seq) * heads + kvh * group + hrow) * nsplit + z) *
                               (D + 2);
#pragma unroll
    for (int db = 0; db < D / 16; ++db) dst[db * 16 + j] = o[db][r];
    if (j == 0) {
      dst[D] = m[r];
      dst[D + 1] = l[r];
    }
  }
}

// out[seq][head][:] = sum_z exp(m_z - M) O_z / sum_z exp(m_z - M) l_z, splits in order.
constexpr int kMaxSplits = 64;

__global__ void attention_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out,
                                       int head_dim, int nsplit) {
  __shared__ float ms[kMaxSplits], ls[kMaxSplits];
  const size_t row = blockIdx.x;  // seq * heads + head
  const int stride = head_dim + 2;
  const float* src = partial + row * nsplit * stride;
  if (threadIdx.x < nsplit) {
    ms[threadIdx.x] = src[threadIdx.x * stride + head_dim];
    ls[threadIdx.x] = src[threadIdx.x * stride + head_dim + 1];
  }
  __syncthreads();
  float mx = -INFINITY;
  for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, ms[z]);
  float den = 0.f;
  for (int z = 0; z < nsplit; ++z) den += (ms[z] == -INFINITY ? 0.f : __expf(ms[z] - mx)) * ls[z];
  const float inv = 1.f / den;
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
    float num = 0.f;
#pragma unroll 8
    for (int z = 0; z < nsplit; ++z) {
      const float f = ms[z] == -INFINITY ? 0.f : __expf(ms[z] - mx);
      num += f * src[z * stride + d];
    }
    out[row * head_dim + d] = from_float<bf16>(num * inv);
  }
}

// ------------------------------------------------------------------ prefill
// grid (query tiles of 16 over all portions, heads), one wavefront per
// workgroup.  tile_seq / tile_q0: for each tile its sequence and the offset of
// its first query inside the sequence's portion.

template <int D>
__global__ void __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(2)))
    attention_prefill_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                             int heads, int kv_heads, const int32_t* __restrict__ cu_q,
                             const int32_t* __restrict__ ctx_lens,
                             const int32_t* __restrict__ tile_seq,
                             const int32_t* __restrict__ tile_q0,
                             const int32_t* __restrict__ tables, int table_stride,
                             const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
                             int page_size, int window, float scale) {
  __shared__ __attribute__((aligned(16))) uint16_t p_lds[16 * kPStride];
  // tiles are listed in token order; the last ones read the most keys, so they start first
  const int tile = gridDim.x - 1 - blockIdx.x, head = blockIdx.y;
  const int lane = threadIdx.x, j = lane % 16, kg = lane / 16;
  const int seq = tile_seq[tile], q0 = tile_q0[tile];
  const int tok0 = cu_q[seq], q_len = cu_q[seq + 1] - tok0;
  const int start = ctx_lens[seq] - q_len;  // position of the portion's first token
  const int kvh = head / (heads / kv_heads);
  const int rows = (q_len - q0 < 16) ? q_len - q0 : 16;

  AFrag qf[D / 32];
  const bf16* qrow = q + static_cast<size_t>(tok0 + q0 + j) * q_stride +
                     static_cast<size_t>(head) * D + kg * 8;
#pragma unroll
  for (int ds = 0; ds < D / 32; ++ds) {
    qf[ds].u = make_uint4(0, 0, 0, 0);
    if (j < rows) qf[ds].u = *reinterpret_cast<const uint4*>(qrow + ds * 32);
  }

  int row_pos[4], row_lo[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int qi = kg * 4 + r;
    row_pos[r] = (qi < rows) ? start + q0 + qi : -1;  // rows past the portion read nothing
    row_lo[r] = (window > 0 && row_pos[r] - window + 1 > 0) ? row_pos[r] - window + 1 : 0;
  }
  const int pos_min = start + q0, pos_max = start + q0 + rows - 1;
  const int lo_min = (window > 0 && pos_min - window + 1 > 0) ? pos_min - window + 1 : 0;

  float m[4], l[4];
  f32x4 o[D / 16];
#pragma unroll
  for (int r = 0; r < 4; ++r) m[r] = -INFINITY, l[r] = 0.f;
#pragma unroll
  for (int db = 0; db < D / 16; ++db) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  TileArgs ta{tables + static_cast<size_t>(seq) * table_stride, k_pool, v_pool, page_size,
              kv_heads, kvh, scale};
  attend_tile<D>(ta, qf, row_pos, row_lo, pos_max, lo_min, lo_min & ~31, pos_max + 1, o, m, l,
                 p_lds);

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int qi = kg * 4 + r;
    if (qi >= rows) continue;
    bf16* dst = out + static_cast<size_t>(tok0 + q0 + qi) * heads * D + static_cast<size_t>(head) * D;
    const float inv = 1.f / l[r];
#pragma unroll
    for (int db = 0; db < D / 16; ++db) dst[db * 16 + j] = from_float<bf16>(o[db][r] * inv);
  }
}

// ------------------------------------------------- prefill, keys shared in LDS
// A workgroup of 4 wavefronts serves every query head of one key/value head for
// a run of 16-query tiles of one sequence: the chunk of 32 keys is fetched once,
// staged in LDS in operand layout and read by all of them, instead of once per
// (head, tile).  A wavefront owns two "units" (query head, query tile); unit
// u < tiles * group is tile u / group, head u % group of the key/value head.
// grid (workgroup tiles, kv_heads); wg_seq / wg_q0 as tile_seq / tile_q0 above,
// in steps of 16 * tiles queries.

constexpr int kUnitsPerWave = 2;
constexpr int kSharedWaves = 4;

template <int D>
__global__ void __launch_bounds__(kSharedWaves* kWave) __attribute__((amdgpu_waves_per_eu(2)))
    attention_prefill_shared_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                                    int heads, int kv_heads, int tiles,
                                    const int32_t* __restrict__ cu_q,
                                    const int32_t* __restrict__ ctx_lens,
                                    const int32_t* __restrict__ wg_seq,
                                    const int32_t* __restrict__ wg_q0,
                                    const int32_t* __restrict__ tables, int table_stride,
                                    const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
                                    int page_size, int window, float scale) {
  constexpr int kKFrags = 2 * (D / 32), kVFrags = D / 16, kFrags = kKFrags + kVFrags;
  constexpr int kPerThread = kFrags / kSharedWaves;  // fragments each wavefront stages
  __shared__ uint4 kv[2][kFrags][kWave];
  __shared__ __attribute__((aligned(16))) uint16_t p_all[kSharedWaves][16 * kPStride];

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int j = lane % 16, kg = lane / 16;
  // workgroups are listed in token order; the last ones read the most keys, so they start first
  const int wg = gridDim.x - 1 - blockIdx.x;
  const int seq = wg_seq[wg], q0 = wg_q0[wg], kvh = blockIdx.y;
  const int group = heads / kv_heads;
  const int tok0 = cu_q[seq], q_len = cu_q[seq + 1] - tok0;
  const int start = ctx_lens[seq] - q_len;  // position of the portion's first token
  const int q_end = (q0 + 16 * tiles < q_len) ? q0 + 16 * tiles : q_len;
  const int ps = page_size;
  const size_t head_elems = static_cast<size_t>(ps) * D;
  const int32_t* table = tables + static_cast<size_t>(seq) * table_stride;
  uint16_t* p_lds = p_all[wave];

  // bounds over the whole workgroup: what has to be staged
  const int pos_min = start + q0, pos_max = start + q_end - 1;
  const int lo_min = (window > 0 && pos_min - window + 1 > 0) ? pos_min - window + 1 : 0;
  const int key_begin = lo_min & ~31;

  // this wavefront's units
  AFrag qf[kUnitsPerWave][D / 32];
  int row_pos[kUnitsPerWave][4], row_lo[kUnitsPerWave][4];
  float m[kUnitsPerWave][4], l[kUnitsPerWave][4];
  f32x4 o[kUnitsPerWave][D / 16];
  int unit_head[kUnitsPerWave], unit_q0[kUnitsPerWave], unit_rows[kUnitsPerWave];
#pragma unroll
  for (int u = 0; u < kUnitsPerWave; ++u) {
    const int unit = wave * kUnitsPerWave + u;
    const bool valid = unit < tiles * group && q0 + (unit / group) * 16 < q_len;
    unit_head[u] = kvh * group + unit % group;
    unit_q0[u] = q0 + (unit / group) * 16;
    unit_rows[u] = !valid ? 0 : (q_len - unit_q0[u] < 16 ? q_len - unit_q0[u] : 16);
    const bf16* qrow = q + static_cast<size_t>(tok0 + unit_q0[u] + j) * q_stride +
                       static_cast<size_t>(unit_head[u]) * D + kg * 8;
#pragma unroll
    for (int ds = 0; ds < D / 32; ++ds) {
      qf[u][ds].u = make_uint4(0, 0, 0, 0);
      if (j < unit_rows[u]) qf[u][ds].u = *reinterpret_cast<const uint4*>(qrow + ds * 32);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int qi = kg * 4 + r;
      row_pos[u][r] = (qi < unit_rows[u]) ? start + unit_q0[u] + qi : -1;
      row_lo[u][r] = (window > 0 && row_pos[u][r] - window + 1 > 0) ? row_pos[u][r] - window + 1 : 0;
      m[u][r] = -INFINITY;
      l[u][r] = 0.f;
    }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) o[u][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // Staging: wavefront w fetches fragments w, w + 4, ...  Fragment f < kKFrags is
  // K tile f / (D/32), head_dim slice f % (D/32); the others are V blocks of 16 elements.
  uint4 regs[kPerThread];
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int f = wave + kSharedWaves * i;
      regs[i] = make_uint4(0, 0, 0, 0);
      if (f < kKFrags) {
        const int tt = f / (D / 32), ds = f % (D / 32);
        const int key0 = kb + tt * 16;
        if (key0 <= pos_max && key0 + 15 >= lo_min) {
          const int page = table[key0 / ps];
          regs[i] = *reinterpret_cast<const uint4*>(
              k_pool + (static_cast<size_t>(page) * kv_heads + kvh) * head_elems +
              static_cast<size_t>(key0 % ps + j) * D + ds * 32 + kg * 8);
        }
      } else {
        const int db = f - kKFrags;
        const int g0 = kb + kg * 8;
        if (g0 <= pos_max && g0 + 7 >= lo_min) {
          const int page = table[g0 / ps];
          uint4 v = *reinterpret_cast<const uint4*>(
              v_pool + (static_cast<size_t>(page) * kv_heads + kvh) * head_elems +
              static_cast<size_t>(db * 16 + j) * ps + g0 % ps);
          if (g0 < lo_min || g0 + 7 > pos_max) {
            // keys outside [lo_min, pos_max] carry weight 0 but may hold anything
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const bool a = g0 + 2 * e >= lo_min && g0 + 2 * e <= pos_max;
              const bool b = g0 + 2 * e + 1 >= lo_min && g0 + 2 * e + 1 <= pos_max;
              w[e] &= (a ? 0x0000ffffu : 0u) | (b ? 0xffff0000u : 0u);
            }
            v = make_uint4(w[0], w[1], w[2], w[3]);
          }
          regs[i] = v;
        }
      }
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) kv[buf][wave + kSharedWaves * i][lane] = regs[i];
  };

  fetch(key_begin);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int kb = key_begin; kb <= pos_max; kb += 32) {
    const bool more = kb + 32 <= pos_max;
    if (more) fetch(kb + 32);
#pragma unroll
    for (int u = 0; u < kUnitsPerWave; ++u) {
      // ---- S = Q K^T
      f32x4 s[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ds = 0; ds < D / 32; ++ds) {
          AFrag kf;
          kf.u = kv[buf][tt * (D / 32) + ds][lane];
          s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[u][ds].v, kf.v, s[tt], 0, 0, 0);
        }
      }
      // ---- mask, running maximum and sum
      float p[2][4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float sc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const int key = kb + tt * 16 + j;
          const bool keep = key <= row_pos[u][r] && key >= row_lo[u][r];
          sc[tt] = keep ? s[tt][r] * scale : -INFINITY;
        }
        const float mx = row16_max(fmaxf(sc[0], sc[1]));
        const float m_new = fmaxf(m[u][r], mx);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __expf(m[u][r] - m_safe);
        p[0][r] = __expf(sc[0] - m_safe);
        p[1][r] = __expf(sc[1] - m_safe);
        const float sum = row16_sum(p[0][r] + p[1][r]);
        l[u][r] = l[u][r] * alpha + sum;
        m[u][r] = m_new;
#pragma unroll
        for (int db = 0; db < D / 16; ++db) o[u][db][r] *= alpha;
      }
      // ---- P through this wavefront's LDS patch into A-operand layout.  Only this
      // wavefront touches the patch; the fences order its own writes and reads.
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          p_lds[(kg * 4 + r) * kPStride + tt * 16 + j] = bf16_bits(p[tt][r]);
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      AFrag pf;
      pf.u = *reinterpret_cast<const uint4*>(p_lds + j * kPStride + kg * 8);
      // ---- O += P V
#pragma unroll
      for (int db = 0; db < D / 16; ++db) {
        AFrag vf;
        vf.u = kv[buf][kKFrags + db][lane];
        o[u][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf.v, vf.v, o[u][db], 0, 0, 0);
      }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

#pragma unroll
  for (int u = 0; u < kUnitsPerWave; ++u)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int qi = kg * 4 + r;
      if (qi >= unit_rows[u]) continue;
      bf16* dst = out + static_cast<size_t>(tok0 + unit_q0[u] + qi) * heads * D +
                  static_cast<size_t>(unit_head[u]) * D;
      const float inv = 1.f / l[u][r];
#pragma unroll
      for (int db = 0; db < D / 16; ++db) dst[db * 16 + j] = from_float<bf16>(o[u][db][r] * inv);
    }
}

template <int D>
static void launch_decode(dim3 grid, hipStream_t s, const bf16* q, int q_stride, int heads,
                          int kv_heads, const int32_t* positions, const int32_t* tables,
                          int table_stride, const bf16* k_pool, const bf16* v_pool, int page_size,
                          int window, float scale, float* partial, int nsplit) {
  attention_decode_kernel<D><<<grid, kWave, 0, s>>>(q, q_stride, heads, kv_heads, positions, tables,
                                                    table_stride, k_pool, v_pool, page_size,
                                                    window, scale, partial, nsplit);
}

template <int D>
static void launch_prefill(dim3 grid, hipStream_t s, const bf16* q, int q_stride, bf16* out,
                           int heads, int kv_heads, const int32_t* cu_q, const int32_t* ctx_lens,
                           const int32_t* tile_seq, const int32_t* tile_q0, const int32_t* tables,
                           int table_stride, const bf16* k_pool, const bf16* v_pool, int page_size,
                           int window, float scale) {
  attention_prefill_kernel<D><<<grid, kWave, 0, s>>>(q, q_stride, out, heads, kv_heads, cu_q,
                                                     ctx_lens, tile_seq, tile_q0, tables,
                                                     table_stride, k_pool, v_pool, page_size,
                                                     window, scale);
}

template <int D>
static void launch_prefill_shared(dim3 grid, hipStream_t s, const bf16* q, int q_stride, bf16* out,
                                  int heads, int kv_heads, int tiles, const int32_t* cu_q,
                                  const int32_t* ctx_lens, const int32_t* wg_seq,
                                  const int32_t* wg_q0, const int32_t* tables, int table_stride,
                                  const bf16* k_pool, const bf16* v_pool, int page_size, int window,
                                  float scale) {
  attention_prefill_shared_kernel<D><<<grid, kSharedWaves * kWave, 0, s>>>(
      q, q_stride, out, heads, kv_heads, tiles, cu_q, ctx_lens, wg_seq, wg_q0, tables, table_stride,
      k_pool, v_pool, page_size, window, scale);
}

}  // namespace shk

using namespace shk;

#define SHK_DISPATCH_D(D, CALL)                                                         \
  switch (D) {                                                                          \
    case 32: CALL(32); break;                                                           \
    case 64: CALL(64); break;                                                           \
    case 96: CALL(96); break;                                                           \
    case 128: CALL(128); break;                                                         \
    case 160: CALL(160); break;                                                         \
    case 192: CALL(192); break;                                                         \
    case 224: CALL(224); break;                                                         \
    case 256: CALL(256); break;                                                         \
    default: break;                                                                     \
  }

static int check_mfma_shapes(const char* who, int heads, int kv_heads, int head_dim, int page_size,
                             int q_stride) {
  SHK_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
              "%s: heads=%d must be a positive multiple of kv_heads=%d", who, heads, kv_heads);
  SHK_REQUIRE(head_dim % 32 == 0 && head_dim >= 32 && head_dim <= 256,
              "%s: head_dim %d is not a multiple of 32 in 32..256", who, head_dim);
  SHK_REQUIRE(page_size > 0 && page_size % 16 == 0, "%s: page_size %d is not a multiple of 16", who,
              page_size);
  SHK_REQUIRE(q_stride % 8 == 0, "%s: q_stride %d is not a multiple of 8", who, q_stride);
  return 0;
}

extern "C" int shk_attention_supports_mfma(int heads, int kv_heads, int head_dim, int page_size,
                                           int q_stride) {
  return heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads / kv_heads <= 16 &&
         head_dim % 32 == 0 && head_dim >= 32 && head_dim <= 256 && page_size > 0 &&
         page_size % 16 == 0 && q_stride % 8 == 0;
}

extern "C" int shk_attention_decode_bf16(const void* q, int q_stride, void* out, int num_seqs,
                                         int heads, int kv_heads, int head_dim,
                                         const int32_t* positions, const int32_t* tables,
                                         int table_stride, const void* k_pool, const void* v_pool,
                                         int page_size, int window, float scale, float* partial,
                                         int nsplit, void* stream) {
  if (check_mfma_shapes("attention_decode", heads, kv_heads, head_dim, page_size, q_stride)) return 1;
  SHK_REQUIRE(heads / kv_heads <= 16, "attention_decode: at most 16 query heads per key/value head");
  SHK_REQUIRE(num_seqs >= 0 && num_seqs <= 65535 && nsplit >= 1 && nsplit <= kMaxSplits,
              "attention_decode: bad sizes num_seqs=%d nsplit=%d (at most %d splits)", num_seqs,
              nsplit, kMaxSplits);
  if (num_seqs == 0) return 0;
  SHK_REQUIRE(q && out && positions && tables && k_pool && v_pool && partial && table_stride > 0,
              "attention_decode: null pointer");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0, "attention_decode: q is not 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(kv_heads, num_seqs, nsplit);
#define CALL(D)                                                                              \
  launch_decode<D>(grid, s, static_cast<const bf16*>(q), q_stride, heads, kv_heads, positions, \
                   tables, table_stride, static_cast<const bf16*>(k_pool),                   \
                   static_cast<const bf16*>(v_pool), page_size, window, scale, partial, nsplit)
  SHK_DISPATCH_D(head_dim, CALL)
#undef CALL
  SHK_LAUNCH_CHECK("attention_decode");
  attention_merge_kernel<<<num_seqs * heads, head_dim <= 64 ? 64 : 128, 0, s>>>(
      partial, static_cast<bf16*>(out), head_dim, nsplit);
  SHK_LAUNCH_CHECK("attention_merge");
  return 0;
}

// Query tiles of 16 that one workgroup of the shared-key prefill kernel serves for
// a given number of query heads per key/value head; 0: the shape is not served.
extern "C" int shk_attention_prefill_shared_tiles(int heads, int kv_heads, int head_dim) {
  const int group = heads / kv_heads;
  if (group < 1 || group > kUnitsPerWave * kSharedWaves || head_dim > 128) return 0;
  return (kUnitsPerWave * kSharedWaves) / group;
}

extern "C" int shk_attention_prefill_shared_bf16(const void* q, int q_stride, void* out,
                                                 int num_wgs, int heads, int kv_heads,
                                                 int head_dim, const int32_t* cu_q,
                                                 const int32_t* ctx_lens, const int32_t* wg_seq,
                                                 const int32_t* wg_q0, const int32_t* tables,
                                                 int table_stride, const void* k_pool,
                                                 const void* v_pool, int page_size, int window,
                                                 float scale, void* stream) {
  if (check_mfma_shapes("attention_prefill_shared", heads, kv_heads, head_dim, page_size, q_stride))
    return 1;
  const int tiles = shk_attention_prefill_shared_tiles(heads, kv_heads, head_dim);
  SHK_REQUIRE(tiles > 0, "attention_prefill_shared: %d query heads per key/value head or head_dim %d "
              "is not served", heads / kv_heads, head_dim);
  SHK_REQUIRE(num_wgs >= 0 && kv_heads <= 65535, "attention_prefill_shared: bad sizes");
  if (num_wgs == 0) return 0;
  SHK_REQUIRE(q && out && cu_q && ctx_lens && wg_seq && wg_q0 && tables && k_pool && v_pool &&
                  table_stride > 0,
              "attention_prefill_shared: null pointer");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0,
              "attention_prefill_shared: q is not 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(num_wgs, kv_heads);
#define CALL(D)                                                                                \
  launch_prefill_shared<D>(grid, s, static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), \
                           heads, kv_heads, tiles, cu_q, ctx_lens, wg_seq, wg_q0, tables,      \
                           table_stride, static_cast<const bf16*>(k_pool),                     \
                           static_cast<const bf16*>(v_pool), page_size, window, scale)
  switch (head_dim) {
    case 32: CALL(32); break;
    case 64: CALL(64); break;
    case 96: CALL(96); break;
    case 128: CALL(128); break;
    default: break;
  }
#undef CALL
  SHK_LAUNCH_CHECK("attention_prefill_shared");
  return 0;
}

extern "C" int shk_attention_prefill_bf16(const void* q, int q_stride, void* out, int num_tiles,
                                          int heads, int kv_heads, int head_dim,
                                          const int32_t* cu_q, const int32_t* ctx_lens,
                                          const int32_t* tile_seq, const int32_t* tile_q0,
                                          const int32_t* tables, int table_stride,
                                          const void* k_pool, const void* v_pool, int page_size,
                                          int window, float scale, void* stream) {
  if (check_mfma_shapes("attention_prefill", heads, kv_heads, head_dim, page_size, q_stride)) return 1;
  SHK_REQUIRE(num_tiles >= 0 && heads <= 65535, "attention_prefill: bad sizes");
  if (num_tiles == 0) return 0;
  SHK_REQUIRE(q && out && cu_q && ctx_lens && tile_seq && tile_q0 && tables && k_pool && v_pool &&
                  table_stride > 0,
              "attention_prefill: null pointer");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0, "attention_prefill: q is not 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(num_tiles, heads);
#define CALL(D)                                                                              \
  launch_prefill<D>(grid, s, static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), \
                    heads, kv_heads, cu_q, ctx_lens, tile_seq, tile_q0, tables, table_stride, \
                    static_cast<const bf16*>(k_pool), static_cast<const bf16*>(v_pool),      \
                    page_size, window, scale)
  SHK_DISPATCH_D(head_dim, CALL)
#undef CALL
  SHK_LAUNCH_CHECK("attention_prefill");
  return 0;
}
