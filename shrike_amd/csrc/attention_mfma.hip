// bfloat16 attention over the paged cache on the MFMA units (gfx950).
//
// One wavefront owns a tile of 16 "rows" that share a key/value head of one
// sequence: for a prompt portion the rows are 16 consecutive queries of one
// query head; for a decoded token they are the query heads of one group
// (padded to 16).  The wavefront walks its key range in chunks of 32 keys:
//
//   S = Q K^T      two 16x16 tiles, v_mfma_f32_16x16x32_bf16 over head_dim;
//                  K rows are read straight from the page (slabs of 32 elements:
//                  [head_dim / 32][slot][32], 64 bytes per key and slab)
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

// Maximum and sum over the four lanes j, j + 16, j + 32, j + 48 (one query's scores in
// the transposed products), in every one of them.  Two swaps of the vector unit (gfx950's
// v_permlane16_swap / v_permlane32_swap) instead of two trips through the LDS crossbar,
// which the chunk's chain of dependent steps would wait for: with rows of 16 lanes r0 r1
// r2 r3, the first swap of v with itself gives (r0 r0 r2 r2) and (r1 r1 r3 r3), the
// second, of what they combine to, (a a a a) and (b b b b).  Everything here is written
// so that the compiler sees it: an instruction in asm would hide from it what the
// swaps' operands have to wait for.
__device__ __forceinline__ float bits_as_float(unsigned v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ float lanes4_max(float v) {
  const unsigned b = __builtin_bit_cast(unsigned, v);
  const auto rows = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  const unsigned h = __builtin_bit_cast(unsigned, fmaxf(bits_as_float(rows[0]), bits_as_float(rows[1])));
  const auto halves = __builtin_amdgcn_permlane32_swap(h, h, false, false);
  return fmaxf(bits_as_float(halves[0]), bits_as_float(halves[1]));
}
__device__ __forceinline__ float lanes4_sum(float v) {
  const unsigned b = __builtin_bit_cast(unsigned, v);
  const auto rows = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  const unsigned h = __builtin_bit_cast(unsigned, bits_as_float(rows[0]) + bits_as_float(rows[1]));
  const auto halves = __builtin_amdgcn_permlane32_swap(h, h, false, false);
  return bits_as_float(halves[0]) + bits_as_float(halves[1]);
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
  const bf16* k_pool;    // [pages][kv_heads][D / 32][page_size][32]
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
             static_cast<size_t>(key0 % ps + j) * 32 + kg * 8;  // slab ds follows at ds * ps * 32
    }
#pragma unroll
    for (int ds = 0; ds < D / 32; ++ds) {
      c.k[tt][ds].u = make_uint4(0, 0, 0, 0);
      if (live) c.k[tt][ds].u = *reinterpret_cast<const uint4*>(krow + static_cast<size_t>(ds) * ps * 32);
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

// One chunk of 32 keys at `kb` for 16 rows: scores, running softmax state,
// O += P V.  p_lds: this wavefront's 16 x kPStride staging tile.
template <int D>
__device__ __forceinline__ void attend_chunk(const TileArgs& ta, const AFrag (&qf)[D / 32],
                                             const Chunk<D>& cur, int kb, const int (&row_pos)[4],
                                             const int (&row_lo)[4], int pos_max, int lo_min,
                                             f32x4 (&o)[D / 16], float (&m)[4], float (&l)[4],
                                             uint16_t* p_lds) {
  const int lane = threadIdx.x % kWave;
  const int j = lane % 16, kg = lane / 16;

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

  // ---- P through LDS into A-operand layout: rows 16, keys 32.  The tile belongs
  // to this wavefront alone; the fences order its own writes and reads.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      p_lds[(kg * 4 + r) * kPStride + tt * 16 + j] = bf16_bits(p[tt][r]);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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
}

// Walks keys [key_begin, key_end) (key_begin a multiple of 32) for 16 rows.
// qf: the rows' queries as A operands.  row_pos / row_lo: for this lane's four
// accumulator rows (4*(lane/16) + r), the last and first key each may read.
// pos_max / lo_min: the same bounds over all 16 rows.  NBUF - 1 chunks' loads
// are in flight while the current chunk is computed.
template <int D, int NBUF = 2>
__device__ __forceinline__ void attend_tile(const TileArgs& ta, const AFrag (&qf)[D / 32],
                                            const int (&row_pos)[4], const int (&row_lo)[4],
                                            int pos_max, int lo_min, int key_begin, int key_end,
                                            f32x4 (&o)[D / 16], float (&m)[4], float (&l)[4],
                                            uint16_t* p_lds) {
  const int ps = ta.page_size;
  const int last_entry = pos_max / ps;
  PageWindow pw = load_pages(ta.table, key_begin / ps, last_entry);
  Chunk<D> buf[NBUF];
  // the window must hold the entries of the 32 keys from `kb` before they are loaded
  auto fetch = [&](Chunk<D>& c, int kb) {
    if ((kb + 31) / ps >= pw.base + kWave) pw = load_pages(ta.table, kb / ps, last_entry);
    load_chunk<D>(c, ta, pw, kb, pos_max, lo_min);
  };
#pragma unroll
  for (int u = 0; u < NBUF - 1; ++u)
    if (key_begin + 32 * u < key_end) fetch(buf[u], key_begin + 32 * u);
  for (int kb0 = key_begin; kb0 < key_end; kb0 += 32 * NBUF) {
#pragma unroll
    for (int u = 0; u < NBUF; ++u) {
      const int kb = kb0 + 32 * u;
      if (kb < key_end) {
        const int ahead = kb + 32 * (NBUF - 1);
        if (ahead < key_end) fetch(buf[(u + NBUF - 1) % NBUF], ahead);
        attend_chunk<D>(ta, qf, buf[u], kb, row_pos, row_lo, pos_max, lo_min, o, m, l, p_lds);
      }
    }
  }
}

// max(a, b, c) in one instruction.  Written out because fmaxf() first quiets each
// operand that might be a signalling NaN (one more instruction per operand), which
// scores, being products or -inf, never are.  The operands must come from vector
// instructions, never straight from a matrix instruction: the compiler does not
// count the wait states that a matrix result needs for an instruction it cannot
// see into (scores scaled inside the exponent, and so fed unscaled from the
// matrix unit into this, came out wrong).
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// ------------------------------------------------------------------- decode
// grid (kv_heads, sequences, splits), kDecodeWaves wavefronts per workgroup.  A
// single wavefront needs about 1,700 cycles for a chunk of 32 keys whatever the
// memory does, so a workgroup's key range is dealt out to its wavefronts chunk
// by chunk, and their results are combined through LDS before anything is
// written.
//
// The two products are formed transposed, so that a lane owns one query head
// throughout and nothing passes through LDS:
//   S^T = K Q^T   A = 16 keys x head_dim, B = Q^T.  Row i of the A tile t is key
//                 8*(i/4) + 4*t + i%4 of the chunk, so lane (j, g) ends up with
//                 the scores of query j for the eight keys 8*g .. 8*g + 7;
//   O^T += V^T P^T  those eight probabilities, packed to bfloat16, are lane
//                 (j, g)'s B operand as they stand; A is V^T (8 keys of one
//                 element: one 16-byte load from the transposed page).
// Keys outside [lo, pos] are loaded from a slot of a page the sequence holds
// (the page of the nearest key inside the range) and masked.
//
// NT: keys and values are fetched with non-temporal loads.  Nothing is read twice
// within a launch, and from some 50 MB of keys and values per launch on the stream
// then runs a tenth faster (64 sequences of 2,200 keys: 49.7 us against 54.1; of
// 4,000: 86.0 against 95.4, 6.1 TB/s); below that size it is 1 to 4 % slower, so
// the caller says which it wants.

constexpr int kMaxSplits = 64;
constexpr int kDecodeWaves = 4;

template <bool V>
struct EdgeTag {
  static constexpr bool value = V;
};

template <int D>
struct DecodeChunk {
  AFrag k[2][D / 32];
  AFrag v[D / 16];
};

// x / page_size and x % page_size without a division: magic = ceil(2^32 / page_size)
// makes the high half of x * magic the quotient for 0 <= x < 2^32 / page_size.
struct PageDiv {
  int ps;
  uint32_t magic;
  __device__ __forceinline__ int div(int x) const {
    return static_cast<int>(__umulhi(static_cast<uint32_t>(x), magic));
  }
  __device__ __forceinline__ int mod(int x) const { return x - div(x) * ps; }
};

template <int D, bool NT>
__global__ void __launch_bounds__(kDecodeWaves* kWave)
    attention_decode_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                            int heads, int kv_heads, const int32_t* __restrict__ positions,
                            const int32_t* __restrict__ tables, int table_stride,
                            const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
                            int page_size, uint32_t page_magic, int window, float scale,
                            float* __restrict__ partial, int nsplit) {
  constexpr int NBUF = 2;  // chunk buffers: one computed, one in flight
  constexpr int kStep = 32 * kDecodeWaves;  // keys between two chunks of one wavefront
  __shared__ float m_lds[kDecodeWaves][16], l_lds[kDecodeWaves][16];
  __shared__ float4 o_lds[kDecodeWaves - 1][D / 16][kWave];
  const int kvh = blockIdx.x, seq = blockIdx.y, z = blockIdx.z;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave, j = lane % 16, g = lane / 16;
  const int group = heads / kv_heads;
  const PageDiv pd{page_size, page_magic};
  // decode sequences come first in the step: token index == sequence index
  const int pos = positions[seq];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  // this split's keys: chunks of 32 from the chunk that holds `lo`; this
  // wavefront's chunks are those at key_begin, key_begin + kStep, ...
  const int first = lo & ~31;
  const int chunks = (pos - first) / 32 + 1;
  const int per = (chunks + nsplit - 1) / nsplit;
  const int key_begin = first + z * per * 32 + wave * 32;
  int key_end = first + (z + 1) * per * 32;
  if (key_end > pos + 1) key_end = pos + 1;

  // softmax state of query head j in base-2 logarithms; `l` is this lane's share
  // of the sum (its eight keys of every chunk) until the end
  float m = -INFINITY, l = 0.f;
  f32x4 o[D / 16];  // element db*16 + 4*g + r of query j
#pragma unroll
  for (int db = 0; db < D / 16; ++db) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (key_begin < key_end) {
    AFrag qf[D / 32];
    const bf16* qrow = q + static_cast<size_t>(seq) * q_stride +
                       static_cast<size_t>(kvh * group + j) * D + g * 8;
#pragma unroll
    for (int ds = 0; ds < D / 32; ++ds) {
      qf[ds].u = make_uint4(0, 0, 0, 0);
      if (j < group) qf[ds].u = *reinterpret_cast<const uint4*>(qrow + ds * 32);
    }
    const float scale2 = scale * 1.4426950408889634f;
    const int32_t* table = tables + static_cast<size_t>(seq) * table_stride;
    // what of a load's address belongs to the lane: its row inside a half chunk
    // of 16 keys and whether it reads the first or the second half
    const bool k_second = j >= 8;
    int k_lane[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) k_lane[t] = (8 * ((j / 4) % 2) + 4 * t + j % 4) * 32 + g * 8;
    const bool v_second = g >= 2;
    const int v_lane = j * page_size + 8 * (g % 2);
    const size_t head_elems = static_cast<size_t>(page_size) * D;  // one kv head of one page

    auto fetch = [&](DecodeChunk<D>& c, int kb) {
      // pages of the two halves (wave-uniform), clamped into the range the sequence holds
      int ka = kb < lo ? lo : kb, kc = kb + 16 < lo ? lo : kb + 16;
      ka = ka > pos ? pos : ka;
      kc = kc > pos ? pos : kc;
      // scalar loads: they are counted apart from the vector loads in flight
      const int page_a = table[__builtin_amdgcn_readfirstlane(pd.div(ka))];
      const int page_c = table[__builtin_amdgcn_readfirstlane(pd.div(kc))];
      const size_t head_a = (static_cast<size_t>(page_a) * kv_heads + kvh) * head_elems;
      const size_t head_c = (static_cast<size_t>(page_c) * kv_heads + kvh) * head_elems;
      const int slot_a = pd.mod(kb), slot_c = pd.mod(kb + 16);
      // keys lie in slabs of 32 elements, [D / 32][page_size][32]
      const bf16* krow = k_pool + (k_second ? head_c + static_cast<size_t>(slot_c) * 32
                                            : head_a + static_cast<size_t>(slot_a) * 32);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ds = 0; ds < D / 32; ++ds)
          c.k[t][ds].v = NT ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(
                                  krow + k_lane[t] + static_cast<size_t>(ds) * page_size * 32))
                            : *reinterpret_cast<const bf16x8*>(krow + k_lane[t] +
                                                              static_cast<size_t>(ds) * page_size * 32);
      const bf16* vcol = v_pool + (v_second ? head_c + slot_c : head_a + slot_a) + v_lane;
#pragma unroll
      for (int db = 0; db < D / 16; ++db)
        c.v[db].v = NT ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(
                             vcol + static_cast<size_t>(db) * 16 * page_size))
                       : *reinterpret_cast<const bf16x8*>(vcol + static_cast<size_t>(db) * 16 * page_size);
    };

    auto attend_chunk = [&](const DecodeChunk<D>& c, int kb, auto edge_tag) {
      constexpr bool edge = decltype(edge_tag)::value;
      f32x4 s[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ds = 0; ds < D / 32; ++ds)
          s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c.k[t][ds].v, qf[ds].v, s[t], 0, 0, 0);
      }
      // this lane's keys are kb + 8*g + e, e = 4*t + r
      float sc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] = s[e / 4][e % 4] * scale2;
      const int g0 = kb + g * 8;
      if (edge) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (g0 + e > pos || g0 + e < lo) sc[e] = -INFINITY;
      }
      float mx = max3(max3(sc[0], sc[1], sc[2]), max3(sc[3], sc[4], sc[5]), fmaxf(sc[6], sc[7]));
      mx = lanes4_max(mx);
      const float m_new = fmaxf(m, mx);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
      float pr[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) pr[e] = __builtin_amdgcn_exp2f(sc[e] - m_safe);
      l = l * alpha + (((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7])));
      m = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
        for (int db = 0; db < D / 16; ++db) o[db] *= alpha;
      }
      AFrag pf;
#pragma unroll
      for (int e = 0; e < 8; ++e) pf.v[e] = static_cast<__bf16>(pr[e]);
      // Masked keys carry weight 0 but their slots may hold anything: zero them
      // so that 0 * x stays 0.
      uint4 keep_bits = make_uint4(~0u, ~0u, ~0u, ~0u);
      if (edge) {
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool a = g0 + 2 * e >= lo && g0 + 2 * e <= pos;
          const bool b = g0 + 2 * e + 1 >= lo && g0 + 2 * e + 1 <= pos;
          w[e] = (a ? 0x0000ffffu : 0u) | (b ? 0xffff0000u : 0u);
        }
        keep_bits = make_uint4(w[0], w[1], w[2], w[3]);
      }
#pragma unroll
      for (int db = 0; db < D / 16; ++db) {
        AFrag vf = c.v[db];
        if (edge) {
          vf.u.x &= keep_bits.x;
          vf.u.y &= keep_bits.y;
          vf.u.z &= keep_bits.z;
          vf.u.w &= keep_bits.w;
        }
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, o[db], 0, 0, 0);
      }
    };

    // interior chunks, the common case, carry no masking code
    auto attend = [&](const DecodeChunk<D>& c, int kb) {
      if (kb + 31 > pos || kb < lo)  // wave-uniform
        attend_chunk(c, kb, EdgeTag<true>{});
      else
        attend_chunk(c, kb, EdgeTag<false>{});
    };

    // NBUF - 1 chunks' loads are in flight while one chunk is computed.  Every step
    // issues a chunk's loads, past the end those of the last chunk again: a step
    // without loads would make the compiler wait for all loads in flight at each step.
    const int last_kb = key_begin + (key_end - 1 - key_begin) / kStep * kStep;
    DecodeChunk<D> buf[NBUF];
#pragma unroll
    for (int u = 0; u < NBUF - 1; ++u) {
      const int kb = key_begin + kStep * u;
      fetch(buf[u], kb < last_kb ? kb : last_kb);
    }
    for (int kb0 = key_begin; kb0 < key_end; kb0 += kStep * NBUF) {
#pragma unroll
      for (int u = 0; u < NBUF; ++u) {
        const int kb = kb0 + kStep * u;
        if (kb >= key_end) break;
        const int ahead = kb + kStep * (NBUF - 1);
        fetch(buf[(u + NBUF - 1) % NBUF], ahead < last_kb ? ahead : last_kb);
        attend(buf[u], kb);
      }
    }
    l = lanes4_sum(l);
  }

  // ---- the wavefronts' results become one: common maximum, sums in wavefront order
  if (g == 0) {
    m_lds[wave][j] = m;
    l_lds[wave][j] = l;
  }
  __syncthreads();
  float m_all = m_lds[0][j];
#pragma unroll
  for (int w = 1; w < kDecodeWaves; ++w) m_all = fmaxf(m_all, m_lds[w][j]);
  const float m_ref = (m_all == -INFINITY) ? 0.f : m_all;
  l = 0.f;
#pragma unroll
  for (int w = 0; w < kDecodeWaves; ++w)
    l += l_lds[w][j] * __builtin_amdgcn_exp2f(m_lds[w][j] - m_ref);  // 2^-inf = 0: nothing seen
  const float mine = __builtin_amdgcn_exp2f(m - m_ref);
  m = m_all;
#pragma unroll
  for (int db = 0; db < D / 16; ++db) o[db] *= mine;
  if (wave > 0) {
#pragma unroll
    for (int db = 0; db < D / 16; ++db)
      o_lds[wave - 1][db][lane] = make_float4(o[db][0], o[db][1], o[db][2], o[db][3]);
  }
  __syncthreads();
  if (wave > 0 || j >= group) return;
#pragma unroll
  for (int w = 0; w < kDecodeWaves - 1; ++w)
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      const float4 x = o_lds[w][db][lane];
      o[db][0] += x.x;
      o[db][1] += x.y;
      o[db][2] += x.z;
      o[db][3] += x.w;
    }

  const int head = kvh * group + j;
  if (nsplit == 1) {
    // the whole range in one wavefront: normalise and write the output row
    const float inv = 1.f / l;
    bf16* dst = out + (static_cast<size_t>(seq) * heads + head) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      uint2 packed;
      packed.x = bf16_bits(o[db][0] * inv) | (static_cast<uint32_t>(bf16_bits(o[db][1] * inv)) << 16);
      packed.y = bf16_bits(o[db][2] * inv) | (static_cast<uint32_t>(bf16_bits(o[db][3] * inv)) << 16);
      *reinterpret_cast<uint2*>(dst + db * 16) = packed;
    }
    return;
  }
  // partial: O [seq][head][split][D], then (max, sum) [seq][head][split][2]
  const size_t rows = static_cast<size_t>(gridDim.y) * heads * nsplit;
  const size_t row = (static_cast<size_t>(seq) * heads + head) * nsplit + z;
  float* dst = partial + row * D + 4 * g;
#pragma unroll
  for (int db = 0; db < D / 16; ++db)
    *reinterpret_cast<float4*>(dst + db * 16) = make_float4(o[db][0], o[db][1], o[db][2], o[db][3]);
  if (g == 0) *reinterpret_cast<float2*>(partial + rows * D + row * 2) = make_float2(m, l);
}

// out[seq][head][:] = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, splits in
// order.  One wavefront per (sequence, head); lane z holds split z's weight.
template <int D>
__global__ void __launch_bounds__(kWave)
    attention_merge_kernel(const float* __restrict__ partial, bf16* __restrict__ out, int nsplit) {
  constexpr int NE = (D + kWave - 1) / kWave;  // elements per lane
  constexpr int kBatch = 8;                    // splits in flight
  __shared__ float weight[kMaxSplits];
  const size_t rows = static_cast<size_t>(gridDim.x) * nsplit;
  const size_t row = blockIdx.x;  // seq * heads + head
  const int lane = threadIdx.x;
  const float* src = partial + row * nsplit * D;
  const float* ml = partial + rows * D + row * nsplit * 2;
  float2 mine = make_float2(-INFINITY, 0.f);
  if (lane < nsplit) mine = *reinterpret_cast<const float2*>(ml + lane * 2);

  float x[kBatch][NE];
  auto fetch = [&](int z0) {
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int d = lane + e * kWave;
        x[u][e] = (z0 + u < nsplit && d < D) ? src[static_cast<size_t>(z0 + u) * D + d] : 0.f;
      }
  };
  fetch(0);  // travels while the weights are formed

  const float mx = wave_max(mine.x);
  const float w = mine.x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mine.x - mx);
  weight[lane] = w;
  // splits in order: the denominator is summed by every lane from the weights in LDS
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const float wl = w * mine.y;
  float den = 0.f;
  for (int zz = 0; zz < nsplit; ++zz) den += __shfl(wl, zz, kWave);

  float acc[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) acc[e] = 0.f;
  for (int z0 = 0; z0 < nsplit; z0 += kBatch) {
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const float wz = z0 + u < nsplit ? weight[z0 + u] : 0.f;
#pragma unroll
      for (int e = 0; e < NE; ++e) acc[e] += wz * x[u][e];
    }
    if (z0 + kBatch < nsplit) fetch(z0 + kBatch);
  }
  const float inv = 1.f / den;
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    const int d = lane + e * kWave;
    if (d < D) out[row * D + d] = from_float<bf16>(acc[e] * inv);
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
// A workgroup of 16 wavefronts serves every query head of one key/value head for
// a run of 16-query tiles of one sequence.  The chunk of 32 keys is fetched once
// and staged in LDS in operand layout; a wavefront owns one "unit" (query head,
// query tile) (the code allows several, which then share every fragment read
// from LDS).  The softmax arithmetic, not the matrix unit, bounds a wavefront,
// and the workgroup with the last queries sets the kernel's time, hence many
// wavefronts with little each: for 2,048 queries of 28 heads over 4, sixteen
// wavefronts with one unit take 96 us, eight with two 104 us, four with four 150
// us.  Unit u < tiles * group is tile u / group, head u % group of the key/value
// head.  The products are formed transposed as in the decode kernel (S^T = K Q^T,
// O^T += V^T P^T): a lane owns one query, and P needs no trip through LDS.
// grid (entries of wg_seq / wg_q0 x kv_heads); wg_seq / wg_q0 as tile_seq / tile_q0
// above, in steps of 16 * tiles queries, in any order.

constexpr int kUnitsPerWave = 1;
// wavefronts per workgroup: 16, or 8 where that many would make too few workgroups
// for the chip (a portion of a few hundred queries)
constexpr int kSharedWaves = 16, kSharedWavesSmall = 8;

template <int D, int WAVES>
__global__ void __launch_bounds__(WAVES* kWave) __attribute__((amdgpu_waves_per_eu(4)))
    attention_prefill_shared_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                                    int heads, int kv_heads, int tiles,
                                    const int32_t* __restrict__ cu_q,
                                    const int32_t* __restrict__ ctx_lens,
                                    const int32_t* __restrict__ wg_seq,
                                    const int32_t* __restrict__ wg_q0,
                                    const int32_t* __restrict__ tables, int table_stride,
                                    const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
                                    int page_size, uint32_t page_magic, int window, float scale,
                                    float* __restrict__ partial, int nsplit, int first_token,
                                    int partial_rows) {
  constexpr int U = kUnitsPerWave;
  constexpr int kKFrags = 2 * (D / 32), kVFrags = D / 16, kFrags = kKFrags + kVFrags;
  // fragments each wavefront stages; where they do not divide, some are staged twice
  constexpr int kPer = (kFrags + WAVES - 1) / WAVES;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  __shared__ u32x4 kv[2][kFrags][kWave];

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int j = lane % 16, g = lane / 16;
  const PageDiv pd{page_size, page_magic};
  // Workgroups start in the order of the host's list (every key/value head of an entry
  // side by side): the host puts the entries that read the most keys first.
  const int z = blockIdx.x % nsplit;  // which share of the entry's keys
  const int wg = blockIdx.x / (nsplit * kv_heads), kvh = (blockIdx.x / nsplit) % kv_heads;
  const int seq = wg_seq[wg], q0 = wg_q0[wg];
  const int group = heads / kv_heads;
  const int tok0 = cu_q[seq], q_len = cu_q[seq + 1] - tok0;
  const int start = ctx_lens[seq] - q_len;  // position of the portion's first token
  const int q_end = (q0 + 16 * tiles < q_len) ? q0 + 16 * tiles : q_len;
  const size_t head_elems = static_cast<size_t>(page_size) * D;
  const int32_t* table = tables + static_cast<size_t>(seq) * table_stride;

  // bounds over the whole workgroup: what has to be staged
  const int pos_min = start + q0, pos_max = start + q_end - 1;
  const int lo_min = (window > 0 && pos_min - window + 1 > 0) ? pos_min - window + 1 : 0;
  const int key_begin = lo_min & ~31;
  const int nchunks = (pos_max - key_begin) / 32 + 1;
  // this workgroup's share of the chunks (all of them without splits; none at all
  // for the last shares of an entry with few keys)
  const int per_split = (nchunks + nsplit - 1) / nsplit;
  const int c_first = z * per_split;
  const int c_end = c_first + per_split < nchunks ? c_first + per_split : nchunks;

  // this wavefront's units; a lane owns query j of each
  AFrag qf[U][D / 32];
  int q_pos[U], q_lo[U];  // last and first key this lane's query reads (-1: no query)
  float m[U], l[U];       // base-2 logarithms; l is the lane's share of the sum until the end
  f32x4 o[U][D / 16];     // element db*16 + 4*g + r of the lane's query
  int unit_head[U], unit_q0[U], unit_rows[U];
  const float scale2 = scale * 1.4426950408889634f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int unit = wave * U + u;
    const bool valid = unit < tiles * group && q0 + (unit / group) * 16 < q_len;
    unit_head[u] = kvh * group + unit % group;
    unit_q0[u] = q0 + (unit / group) * 16;
    unit_rows[u] = !valid ? 0 : (q_len - unit_q0[u] < 16 ? q_len - unit_q0[u] : 16);
    const int qrow_i = j < unit_rows[u] ? j : 0;  // an address inside the portion for every lane
    const bf16* qrow = q + static_cast<size_t>(tok0 + (valid ? unit_q0[u] : 0) + qrow_i) * q_stride +
                       static_cast<size_t>(unit_head[u]) * D + g * 8;
#pragma unroll
    for (int ds = 0; ds < D / 32; ++ds) {
      qf[u][ds].u = make_uint4(0, 0, 0, 0);
      if (j < unit_rows[u]) qf[u][ds].u = *reinterpret_cast<const uint4*>(qrow + ds * 32);
    }
    q_pos[u] = j < unit_rows[u] ? start + unit_q0[u] + j : -1;
    q_lo[u] = (window > 0 && q_pos[u] - window + 1 > 0) ? q_pos[u] - window + 1 : 0;
    m[u] = -INFINITY;
    l[u] = 0.f;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) o[u][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- staging.  Wavefront w fetches fragments w, w + WAVES, ...  Fragment f < kKFrags
  // is K tile f / (D/32), head_dim slice f % (D/32); row i of K tile t is key
  // 8*(i/4) + 4*t + i%4 of the chunk, so that lane (j, g) of a score tile ends up
  // with the eight keys 8*g .. 8*g + 7.  The others are V^T blocks of 16 elements.
  // Every load is unconditional (addresses clamped into pages the sequence holds).
  const bool second_k = j >= 8, second_v = g >= 2;
  int lane_off[kPer];
  bool is_k[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int f = (wave + WAVES * i) % kFrags;
    is_k[i] = f < kKFrags;
    if (is_k[i]) {
      const int t = f / (D / 32), ds = f % (D / 32);
      lane_off[i] = (8 * ((j / 4) % 2) + 4 * t + j % 4) * 32 + ds * page_size * 32 + g * 8;
    } else {
      const int db = f - kKFrags;
      lane_off[i] = (db * 16 + j) * page_size + 8 * (g % 2);
    }
  }
  auto fetch = [&](u32x4 (&held)[kPer], int chunk) {
    const int kb = key_begin + 32 * (chunk < nchunks ? chunk : nchunks - 1);
    int ka = kb < lo_min ? lo_min : kb, kc = kb + 16 < lo_min ? lo_min : kb + 16;
    ka = ka > pos_max ? pos_max : ka;
    kc = kc > pos_max ? pos_max : kc;
    const int page_a = table[__builtin_amdgcn_readfirstlane(pd.div(ka))];
    const int page_c = table[__builtin_amdgcn_readfirstlane(pd.div(kc))];
    const size_t head_a = (static_cast<size_t>(page_a) * kv_heads + kvh) * head_elems;
    const size_t head_c = (static_cast<size_t>(page_c) * kv_heads + kvh) * head_elems;
    const int slot_a = pd.mod(kb), slot_c = pd.mod(kb + 16);
    const bf16* krow = k_pool + (second_k ? head_c + static_cast<size_t>(slot_c) * 32
                                          : head_a + static_cast<size_t>(slot_a) * 32);
    const bf16* vcol = v_pool + (second_v ? head_c + slot_c : head_a + slot_a);
#pragma unroll
    for (int i = 0; i < kPer; ++i)
      held[i] = *reinterpret_cast<const u32x4*>((is_k[i] ? krow : vcol) + lane_off[i]);
    __builtin_amdgcn_sched_barrier(0);  // the loads go out before the multiplications
  };
  auto put = [&](const u32x4 (&held)[kPer], int chunk, int buf) {
    const int kb = key_begin + 32 * chunk;
    const int g0 = kb + g * 8;  // a V fragment's lane holds keys g0 .. g0 + 7
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      u32x4 x = held[i];
      // keys outside [lo_min, pos_max] carry weight 0, but their slots may hold anything;
      // only the first and the last chunk have such keys
      if (!is_k[i] && (kb < lo_min || kb + 31 > pos_max)) {
        asm volatile("");  // stays a branch: as selects the comparisons would run for every chunk
        u32x4 keep;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool a = g0 + 2 * e >= lo_min && g0 + 2 * e <= pos_max;
          const bool b = g0 + 2 * e + 1 >= lo_min && g0 + 2 * e + 1 <= pos_max;
          keep[e] = (a ? 0x0000ffffu : 0u) | (b ? 0xffff0000u : 0u);
        }
        x &= keep;
      }
      kv[buf][(wave + WAVES * i) % kFrags][lane] = x;
    }
  };

  // ---- one chunk for this wavefront's units, from LDS buffer `buf`
  // chunks at or before `last_plain` lie wholly inside what every query of the
  // workgroup reads (none without a window's lower bound to check)
  const int last_plain = window > 0 ? -1 : (pos_min + 1 - key_begin) / 32 - 1;
  auto attend = [&](int buf, int chunk) {
    const int kb = key_begin + 32 * chunk;
    const int g0 = kb + g * 8;
    const bool edge = chunk > last_plain;
    u32x4 kf[2][D / 32];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ds = 0; ds < D / 32; ++ds) kf[t][ds] = kv[buf][t * (D / 32) + ds][lane];
    AFrag pf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      f32x4 s[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ds = 0; ds < D / 32; ++ds)
          s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[t][ds]),
                                                         qf[u][ds].v, s[t], 0, 0, 0);
      }
      // this lane's keys are g0 + e, e = 4*t + r
      float sc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) sc[e] = s[e / 4][e % 4] * scale2;
      if (edge) {  // wave-uniform: some query of the workgroup does not read the whole chunk
        // (the empty statement keeps this a branch: turned into selects, the
        // comparisons would run for every chunk)
        asm volatile("");
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (g0 + e > q_pos[u] || g0 + e < q_lo[u]) sc[e] = -INFINITY;
      }
      float mx = max3(max3(sc[0], sc[1], sc[2]), max3(sc[3], sc[4], sc[5]), fmaxf(sc[6], sc[7]));
      mx = lanes4_max(mx);
      const float m_new = fmaxf(m[u], mx);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m[u] - m_safe);
      float pr[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) pr[e] = __builtin_amdgcn_exp2f(sc[e] - m_safe);
      l[u] = l[u] * alpha +
             (((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7])));
      m[u] = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // some query's maximum rose
#pragma unroll
        for (int db = 0; db < D / 16; ++db) o[u][db] *= alpha;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) pf[u].v[e] = static_cast<__bf16>(pr[e]);
    }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      const u32x4 vf = kv[buf][kKFrags + db][lane];
#pragma unroll
      for (int u = 0; u < U; ++u)
        o[u][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf), pf[u].v,
                                                           o[u][db], 0, 0, 0);
    }
  };

  // Chunk c is multiplied from LDS buffer c % 2 while the loads of chunks c + 1 and
  // c + 2 are in flight.  The loop's body has no branch, so the loads stay where
  // they are written.
  if (c_first < c_end) {  // the same for every wavefront of the workgroup
    u32x4 even[kPer], odd[kPer];
    fetch(even, c_first);
    fetch(odd, c_first + 1);
    put(even, c_first, 0);
    __syncthreads();
    int c = c_first;
    for (; c + 2 < c_end; c += 2) {
      fetch(even, c + 2);
      attend(0, c);
      put(odd, c + 1, 1);
      __syncthreads();
      fetch(odd, c + 3);
      attend(1, c + 1);
      put(even, c + 2, 0);
      __syncthreads();
    }
    attend(0, c);
    if (c + 1 < c_end) {
      put(odd, c + 1, 1);
      __syncthreads();
      attend(1, c + 1);
    }
  }

#pragma unroll
  for (int u = 0; u < U; ++u) {
    float total = l[u];
    total = lanes4_sum(total);
    if (j >= unit_rows[u]) continue;
    if (nsplit > 1) {
      // a share's result, for attention_merge_kernel: O [row][share][D], then (maximum,
      // sum) [row][share][2], row = the token's index among the step's prompt tokens x head
      const size_t row = static_cast<size_t>(tok0 + unit_q0[u] + j - first_token) * heads + unit_head[u];
      float* dst = partial + (row * nsplit + z) * D + 4 * g;
#pragma unroll
      for (int db = 0; db < D / 16; ++db)
        *reinterpret_cast<float4*>(dst + db * 16) =
            make_float4(o[u][db][0], o[u][db][1], o[u][db][2], o[u][db][3]);
      if (g == 0)
        *reinterpret_cast<float2*>(partial + static_cast<size_t>(partial_rows) * nsplit * D +
                                   (row * nsplit + z) * 2) = make_float2(m[u], total);
      continue;
    }
    const float inv = 1.f / total;
    bf16* dst = out + static_cast<size_t>(tok0 + unit_q0[u] + j) * heads * D +
                static_cast<size_t>(unit_head[u]) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      uint2 packed;
      packed.x = bf16_bits(o[u][db][0] * inv) |
                 (static_cast<uint32_t>(bf16_bits(o[u][db][1] * inv)) << 16);
      packed.y = bf16_bits(o[u][db][2] * inv) |
                 (static_cast<uint32_t>(bf16_bits(o[u][db][3] * inv)) << 16);
      *reinterpret_cast<uint2*>(dst + db * 16) = packed;
    }
  }
}

template <int D>
static void launch_decode(dim3 grid, hipStream_t s, const bf16* q, int q_stride, bf16* out,
                          int heads, int kv_heads, const int32_t* positions, const int32_t* tables,
                          int table_stride, const bf16* k_pool, const bf16* v_pool, int page_size,
                          int window, float scale, float* partial, int nsplit, int streaming) {
  const uint32_t magic = static_cast<uint32_t>(((1ull << 32) + page_size - 1) / page_size);
  if (streaming)
    attention_decode_kernel<D, true><<<grid, kDecodeWaves * kWave, 0, s>>>(
        q, q_stride, out, heads, kv_heads, positions, tables, table_stride, k_pool, v_pool, page_size,
        magic, window, scale, partial, nsplit);
  else
    attention_decode_kernel<D, false><<<grid, kDecodeWaves * kWave, 0, s>>>(
        q, q_stride, out, heads, kv_heads, positions, tables, table_stride, k_pool, v_pool, page_size,
        magic, window, scale, partial, nsplit);
  if (nsplit > 1)
    attention_merge_kernel<D><<<grid.y * heads, kWave, 0, s>>>(partial, out, nsplit);
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
                                  float scale, bool small, float* partial, int nsplit,
                                  int first_token, int prompt_tokens) {
  const uint32_t magic = static_cast<uint32_t>(((1ull << 32) + page_size - 1) / page_size);
  const int rows = prompt_tokens * heads;
  if (small)
    attention_prefill_shared_kernel<D, kSharedWavesSmall><<<grid, kSharedWavesSmall * kWave, 0, s>>>(
        q, q_stride, out, heads, kv_heads, tiles, cu_q, ctx_lens, wg_seq, wg_q0, tables,
        table_stride, k_pool, v_pool, page_size, magic, window, scale, partial, nsplit, first_token,
        rows);
  else
    attention_prefill_shared_kernel<D, kSharedWaves><<<grid, kSharedWaves * kWave, 0, s>>>(
        q, q_stride, out, heads, kv_heads, tiles, cu_q, ctx_lens, wg_seq, wg_q0, tables,
        table_stride, k_pool, v_pool, page_size, magic, window, scale, partial, nsplit, first_token,
        rows);
  if (nsplit > 1)
    attention_merge_kernel<D><<<rows, kWave, 0, s>>>(
        partial, out + static_cast<size_t>(first_token) * heads * D, nsplit);
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
                                         int nsplit, int streaming, void* stream) {
  if (check_mfma_shapes("attention_decode", heads, kv_heads, head_dim, page_size, q_stride)) return 1;
  SHK_REQUIRE(heads / kv_heads <= 16, "attention_decode: at most 16 query heads per key/value head");
  SHK_REQUIRE(num_seqs >= 0 && num_seqs <= 65535 && nsplit >= 1 && nsplit <= kMaxSplits,
              "attention_decode: bad sizes num_seqs=%d nsplit=%d (at most %d splits)", num_seqs,
              nsplit, kMaxSplits);
  if (num_seqs == 0) return 0;
  SHK_REQUIRE(q && out && positions && tables && k_pool && v_pool && partial && table_stride > 0,
              "attention_decode: null pointer");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0, "attention_decode: q is not 16-byte aligned");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(out) % 8 == 0 && reinterpret_cast<uintptr_t>(partial) % 16 == 0,
              "attention_decode: out must be 8-byte and partial 16-byte aligned");
  SHK_REQUIRE(static_cast<long long>(table_stride) * page_size * page_size < (1ll << 32),
              "attention_decode: a block table of %d pages of %d is beyond the kernel's range",
              table_stride, page_size);
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(kv_heads, num_seqs, nsplit);
#define CALL(D)                                                                              \
  launch_decode<D>(grid, s, static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), heads, \
                   kv_heads, positions, tables, table_stride, static_cast<const bf16*>(k_pool),    \
                   static_cast<const bf16*>(v_pool), page_size, window, scale, partial, nsplit,    \
                   streaming)
  SHK_DISPATCH_D(head_dim, CALL)
#undef CALL
  SHK_LAUNCH_CHECK("attention_decode");
  return 0;
}

// Query tiles of 16 that one workgroup of the shared-key prefill kernel serves for
// a given number of query heads per key/value head; 0: the shape is not served.
extern "C" int shk_attention_prefill_shared_tiles(int heads, int kv_heads, int head_dim, int small) {
  const int group = heads / kv_heads;
  const int units = kUnitsPerWave * (small ? kSharedWavesSmall : kSharedWaves);
  if (group < 1 || group > units || head_dim > 128) return 0;
  return units / group;
}

extern "C" int shk_attention_prefill_shared_bf16(const void* q, int q_stride, void* out,
                                                 int num_wgs, int heads, int kv_heads,
                                                 int head_dim, const int32_t* cu_q,
                                                 const int32_t* ctx_lens, const int32_t* wg_seq,
                                                 const int32_t* wg_q0, const int32_t* tables,
                                                 int table_stride, const void* k_pool,
                                                 const void* v_pool, int page_size, int window,
                                                 float scale, int small, float* partial, int nsplit,
                                                 int first_token, int prompt_tokens, void* stream) {
  if (check_mfma_shapes("attention_prefill_shared", heads, kv_heads, head_dim, page_size, q_stride))
    return 1;
  const int tiles = shk_attention_prefill_shared_tiles(heads, kv_heads, head_dim, small);
  SHK_REQUIRE(tiles > 0, "attention_prefill_shared: %d query heads per key/value head or head_dim %d "
              "is not served", heads / kv_heads, head_dim);
  SHK_REQUIRE(nsplit >= 1 && nsplit <= kMaxSplits, "attention_prefill_shared: %d key splits (at most %d)",
              nsplit, kMaxSplits);
  SHK_REQUIRE(num_wgs >= 0 && static_cast<long long>(num_wgs) * kv_heads * nsplit < (1ll << 31),
              "attention_prefill_shared: bad sizes");
  if (num_wgs == 0) return 0;
  SHK_REQUIRE(nsplit == 1 || (partial && first_token >= 0 && prompt_tokens > 0 &&
                              reinterpret_cast<uintptr_t>(partial) % 16 == 0 &&
                              static_cast<long long>(prompt_tokens) * heads < (1ll << 31)),
              "attention_prefill_shared: key splits need a 16-byte aligned partial buffer, the index "
              "of the first prompt token and the number of prompt tokens");
  SHK_REQUIRE(q && out && cu_q && ctx_lens && wg_seq && wg_q0 && tables && k_pool && v_pool &&
                  table_stride > 0,
              "attention_prefill_shared: null pointer");
  SHK_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0,
              "attention_prefill_shared: q must be 16-byte and out 8-byte aligned");
  SHK_REQUIRE(static_cast<long long>(table_stride) * page_size * page_size < (1ll << 32),
              "attention_prefill_shared: a block table of %d pages of %d is beyond the kernel's range",
              table_stride, page_size);
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(num_wgs * kv_heads * nsplit);
#define CALL(D)                                                                                \
  launch_prefill_shared<D>(grid, s, static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), \
                           heads, kv_heads, tiles, cu_q, ctx_lens, wg_seq, wg_q0, tables,      \
                           table_stride, static_cast<const bf16*>(k_pool),                     \
                           static_cast<const bf16*>(v_pool), page_size, window, scale, small != 0, \
                           partial, nsplit, first_token, prompt_tokens)
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
