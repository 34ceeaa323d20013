// Differential attention in bfloat16 on the matrix cores of gfx950: portions of prompts in tiles of 64 query
// rows, and single rows (decoded tokens) with the query heads of a kv head side by side.
//
// A page holds keys as [row][2 dk] (a row's two maps side by side) and values transposed as [dv][row], so both
// products read their operands along the dimension they reduce over, straight from memory:
//   S^T (16 keys x 16 columns)  = K (16 x dk) . Q^T           v_mfma_f32_16x16x32_bf16, once per map
//   O^T (dv x 16 columns)      += V^T (dv x 32 keys) . P^T    v_mfma_f32_16x16x32_bf16, once per map, the same V
// The transposed score tile leaves each lane with four keys of one column, the layout the second product wants
// for P^T.  Each map has its own running maximum, sum and output; at the end o = a1 - lambda a2 is divided by its
// root mean square over dv and multiplied by out_scale.  Scores, softmax, the difference and the norm are 32-bit.
//
// What the 16 columns are: for a tile, 16 consecutive tokens of one query head (a workgroup's four wavefronts take
// four such runs of the same head); for single rows, the query heads that share one kv head, for one token (four
// wavefronts take the blocks of keys in turns and merge through LDS).
// A column at position p sees the keys lo..p, lo the start of p's block of `block` positions (0: position 0),
// raised to p - window + 1 by a window.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define DA_LOG2E 1.4426950408889634f

union Frag8 {
  uint4 u;
  bf16x8 v;
};

struct DiffPages {
  const bf16_t* pool;   // [pages][K: [n_kv][P][2 dk] | V: [n_kv][dv][P]]
  const int* table;     // block-table row of the request
  int P, n_kv, kvh;
};

// fragments of two blocks of 16 keys, [keyA, keyA + 16) and [keyB, keyB + 16)
template <int DK, int DV>
struct DiffPair {
  Frag8 k[2][2][DK / 32];   // [block][map]: row lane % 16, dims 32 s + 8 (lane / 16) .. + 7
  Frag8 v[DV / 16];         // V^T: row (dim) 16 d + lane % 16; elements 0..3: keys 4 (lane / 16) .. + 3 of block A, 4..7: of block B
  int keyA, keyB;
  bool validA, validB;
};

// keyA is a multiple of 16; keyB = keyA + 16.  A block beyond `last_key` or on a page given back does not count; its
// loads go to the request's page of block `safe` (one that exists), so that they never leave the pool.
template <int DK, int DV>
__device__ __forceinline__ void load_pair(const DiffPages& kv, int keyA, int last_key, int safe_key, DiffPair<DK, DV>& f) {
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int keyB = keyA + 16;
  int pageA = keyA <= last_key ? kv.table[keyA / kv.P] : -1;
  int pageB = keyB <= last_key ? kv.table[keyB / kv.P] : -1;
  f.keyA = keyA;
  f.keyB = keyB;
  f.validA = pageA >= 0;
  f.validB = pageB >= 0;
  int rowA = keyA % kv.P, rowB = keyB % kv.P;
  if (pageA < 0) {
    pageA = kv.table[safe_key / kv.P];
    rowA = safe_key % kv.P;
  }
  if (pageB < 0) {
    pageB = kv.table[safe_key / kv.P];
    rowB = safe_key % kv.P;
  }
  const size_t page_elems = (size_t)kv.n_kv * kv.P * (2 * DK + DV);
  const bf16_t* ka = kv.pool + (size_t)pageA * page_elems + ((size_t)kv.kvh * kv.P + rowA) * (2 * DK);
  const bf16_t* kb = kv.pool + (size_t)pageB * page_elems + ((size_t)kv.kvh * kv.P + rowB) * (2 * DK);
  const size_t v_base = (size_t)kv.n_kv * kv.P * (2 * DK) + (size_t)kv.kvh * DV * kv.P;
  const bf16_t* va = kv.pool + (size_t)pageA * page_elems + v_base + rowA;
  const bf16_t* vb = kv.pool + (size_t)pageB * page_elems + v_base + rowB;
  const unsigned k_lane = (unsigned)(r16 * 2 * DK + quad * 8);
  const unsigned v_lane = (unsigned)(r16 * kv.P + quad * 4);
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) {
      f.k[0][mp][s].u = *reinterpret_cast<const uint4*>(ka + k_lane + mp * DK + s * 32);
      f.k[1][mp][s].u = *reinterpret_cast<const uint4*>(kb + k_lane + mp * DK + s * 32);
    }
  const unsigned v_step = 16u * kv.P;
#pragma unroll
  for (int d = 0; d < DV / 16; ++d) {
    const uint2 a = *reinterpret_cast<const uint2*>(va + v_lane + d * v_step);
    const uint2 b = *reinterpret_cast<const uint2*>(vb + v_lane + d * v_step);
    f.v[d].u = make_uint4(a.x, a.y, b.x, b.y);
  }
}

// the running softmax of one map over the columns of a wavefront
template <int DV>
struct MapState {
  float m, l;            // maximum (units of log 2) of the column; this lane's share of the sum of weights
  floatx4 o[DV / 16];    // O^T: rows (dims) 16 d + 4 (lane / 16) + i, column lane % 16
  __device__ __forceinline__ void clear() {
    m = -INFINITY;
    l = 0.f;
#pragma unroll
    for (int d = 0; d < DV / 16; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
};

// One pair of blocks for this wavefront's 16 columns, both maps.
//   qf      Q^T fragments per map: column lane % 16, dims 32 s + 8 (lane / 16) .. + 7
//   lo, hi  the keys this lane's column sees: lo <= key <= hi (lo > hi: none)
//   plain   every key of both blocks is visible to every column (the same in every lane)
//   kv_last last position of the request that has been written (rows after it hold anything, NaN included)
template <int DK, int DV>
__device__ __forceinline__ void attend_pair(DiffPair<DK, DV>& f, const Frag8 (*qf)[DK / 32], int lo, int hi, bool plain,
                                            int kv_last, float scale2, MapState<DV>* st) {
  const int quad = (threadIdx.x & 63) >> 4;
  bool see[8] = {false, false, false, false, false, false, false, false};
  if (!plain) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ka = f.keyA + quad * 4 + i, kb = f.keyB + quad * 4 + i;
      see[i] = f.validA & (ka >= lo) & (ka <= hi);
      see[4 + i] = f.validB & (kb >= lo) & (kb <= hi);
      // 0 * NaN is NaN: values of rows that were never written (or of a stand-in page) become zero
      const bool zero_a = !f.validA | (ka > kv_last), zero_b = !f.validB | (kb > kv_last);
      const unsigned keep_a = zero_a ? ((i & 1) ? 0x0000FFFFu : 0xFFFF0000u) : 0xFFFFFFFFu;
      const unsigned keep_b = zero_b ? ((i & 1) ? 0x0000FFFFu : 0xFFFF0000u) : 0xFFFFFFFFu;
#pragma unroll
      for (int d = 0; d < DV / 16; ++d) {
        unsigned* wv = reinterpret_cast<unsigned*>(&f.v[d].u);
        wv[i >> 1] &= keep_a;
        wv[2 + (i >> 1)] &= keep_b;
      }
    }
  }
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) {
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[0][mp][s].v, qf[mp][s].v, sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[1][mp][s].v, qf[mp][s].v, sb, 0, 0, 0);
    }
    float sv[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sv[i] = (plain || see[i]) ? sa[i] * scale2 : -INFINITY;
      sv[4 + i] = (plain || see[4 + i]) ? sb[i] * scale2 : -INFINITY;
    }
    MapState<DV>& s = st[mp];
    float bm = sv[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) bm = fmaxf(bm, sv[i]);
    bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(s.m, bm);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    float pv[8], ps = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pv[i] = __builtin_amdgcn_exp2f(sv[i] - m_safe);
      ps += pv[i];
    }
    Frag8 pf;
    pf.u = make_uint4(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]), pack_bf16x2(pv[4], pv[5]), pack_bf16x2(pv[6], pv[7]));
    if (__builtin_amdgcn_ballot_w64(m_new != s.m) != 0) {
      const float alpha = __builtin_amdgcn_exp2f(s.m - m_safe);      // m = -inf: 0, and l and o are 0 anyway
      s.l *= alpha;
#pragma unroll
      for (int d = 0; d < DV / 16; ++d)
#pragma unroll
        for (int i = 0; i < 4; ++i) s.o[d][i] *= alpha;
      s.m = m_new;
    }
    s.l += ps;
#pragma unroll
    for (int d = 0; d < DV / 16; ++d) s.o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[d].v, pf.v, s.o[d], 0, 0, 0);
  }
}

// Pairs first, first + stride, ... below `end` (pair p covers the keys 32 p .. 32 p + 31), the next pair's loads in
// flight while a pair is computed.  lo_max / hi_min: the largest lo and the smallest hi of the wavefront's live columns.
template <int DK, int DV>
__device__ __forceinline__ void walk(const DiffPages& kv, const Frag8 (*qf)[DK / 32], int first, int end, int stride, int lo, int hi,
                                     int lo_max, int hi_min, int kv_last, int safe_key, float scale2, MapState<DV>* st) {
  if (first >= end) return;
  DiffPair<DK, DV> f0, f1;
  load_pair<DK, DV>(kv, first * 32, kv_last, safe_key, f0);
  for (int p = first; p < end; p += 2 * stride) {
    const bool more1 = p + stride < end;
    if (more1) load_pair<DK, DV>(kv, (p + stride) * 32, kv_last, safe_key, f1);
    {
      const bool plain = f0.validA && f0.validB && f0.keyA >= lo_max && f0.keyB + 15 <= hi_min;
      attend_pair<DK, DV>(f0, qf, lo, hi, plain, kv_last, scale2, st);
    }
    if (!more1) break;
    if (p + 2 * stride < end) load_pair<DK, DV>(kv, (p + 2 * stride) * 32, kv_last, safe_key, f0);
    {
      const bool plain = f1.validA && f1.validB && f1.keyA >= lo_max && f1.keyB + 15 <= hi_min;
      attend_pair<DK, DV>(f1, qf, lo, hi, plain, kv_last, scale2, st);
    }
  }
}

__device__ __forceinline__ int first_visible(int p, int block, int window) {
  int lo = block > 0 ? (p / block) * block : 0;
  if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
  return lo;
}

// o = a1 - lambda a2 of this lane's column, normed over dv, to out (the column's row of [.., dv]); `live`: the column counts
template <int DV>
__device__ __forceinline__ void finish_column(MapState<DV>* st, float lambda, float eps, float out_scale, bf16_t* dst, bool live) {
  const int quad = (threadIdx.x & 63) >> 4;
  float inv[2];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    float l = st[mp].l;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    inv[mp] = l > 0.f ? 1.f / l : 0.f;
  }
  float ss = 0.f;
  floatx4 o[DV / 16];
#pragma unroll
  for (int d = 0; d < DV / 16; ++d)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[d][i] = st[0].o[d][i] * inv[0] - lambda * (st[1].o[d][i] * inv[1]);
      ss = fmaf(o[d][i], o[d][i], ss);
    }
  ss += __shfl_xor(ss, 16, 64);
  ss += __shfl_xor(ss, 32, 64);
  const float g = out_scale / sqrtf(ss / (float)DV + eps);
  if (!live) return;
#pragma unroll
  for (int d = 0; d < DV / 16; ++d)
    *reinterpret_cast<uint2*>(dst + d * 16 + quad * 4) = make_uint2(pack_bf16x2(o[d][0] * g, o[d][1] * g), pack_bf16x2(o[d][2] * g, o[d][3] * g));
}

// ------------------------------------------------------------------------------------------ tiles of a portion
// tiles int32 [n][3] = (entry, first row, rows <= 64); entries int32 [.][4] = (row0, tokens, start, -).  q [M][n_head][2][DK],
// out [M][n_head][DV].  Grid (tiles, heads), four wavefronts of 16 rows each.
template <int DK, int DV>
__global__ void __launch_bounds__(256)
diff_tiles_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool, const int* __restrict__ table, int table_stride,
                  const int* __restrict__ tiles, const int* __restrict__ entries, bf16_t* __restrict__ out, int n_head, int n_kv,
                  int P, float scale2, int block, int window, float lambda, float eps, float out_scale) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int e = tiles[3 * blockIdx.x], row0 = tiles[3 * blockIdx.x + 1] + 16 * wave;
  const int n_rows = tiles[3 * blockIdx.x + 2] - 16 * wave;
  if (n_rows <= 0) return;
  const int h = blockIdx.y;
  const int e_row0 = entries[4 * e], e_n = entries[4 * e + 1], e_start = entries[4 * e + 2];
  const int kv_last = e_start + e_n - 1;
  const bool live = r16 < n_rows;
  const int row = row0 + (live ? r16 : 0);
  const int p = e_start + (row - e_row0);
  const int lo = live ? first_visible(p, block, window) : 1, hi = live ? p : 0;
  int lo_min = live ? lo : 0x7fffffff, lo_max = live ? lo : 0, hi_min = live ? hi : 0x7fffffff, hi_max = hi;
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) {
    lo_min = min(lo_min, __shfl_xor(lo_min, o, 64));
    lo_max = max(lo_max, __shfl_xor(lo_max, o, 64));
    hi_min = min(hi_min, __shfl_xor(hi_min, o, 64));
    hi_max = max(hi_max, __shfl_xor(hi_max, o, 64));
  }
  DiffPages kv{pool, table + (size_t)e * table_stride, P, n_kv, h / (n_head / n_kv)};
  Frag8 qf[2][DK / 32];
  const bf16_t* qrow = q + ((size_t)row * n_head + h) * 2 * DK + quad * 8;
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) qf[mp][s].u = *reinterpret_cast<const uint4*>(qrow + mp * DK + s * 32);
  MapState<DV> st[2];
  st[0].clear();
  st[1].clear();
  walk<DK, DV>(kv, qf, lo_min / 32, hi_max / 32 + 1, 1, lo, hi, lo_max, hi_min, kv_last, hi_max, scale2, st);
  finish_column<DV>(st, lambda, eps, out_scale, out + ((size_t)row * n_head + h) * DV, live);
}

// ------------------------------------------------------------------------------------------ tiles, keys and values through LDS
// The same tiles with the four wavefronts sharing what they read: a pair of blocks (32 keys: their two maps and the values)
// is fetched once by the workgroup into one of two LDS stages while the pair before it is multiplied from the other, one
// barrier a pair.  Key and value rows are padded by 16 bytes, so that the fragments' reads spread over the banks; a value row
// holds, quarter by quarter, four keys of the first block and the same four of the second: a lane's fragment in one read.
template <int DK, int DV>
struct DiffStage {
  static constexpr int KROW = 2 * DK + 8;       // bfloat16 elements of a key row
  static constexpr int VROW = 32 + 8;           // of a value row: per quarter q its keys 4 q .. 4 q + 3 of block A, then of block B
  static constexpr int K_ELEMS = 32 * KROW, ELEMS = K_ELEMS + DV * VROW;
  static constexpr int K_UNITS = 32 * (2 * DK / 8), V_UNITS = DV * 4;      // 16-byte pieces fetched per pair
  static constexpr int K_PER = (K_UNITS + 255) / 256, V_PER = (V_UNITS + 255) / 256;
};

// the workgroup's fetch of a pair into registers (thread t the 16-byte pieces t, t + 256, ...), and their way into a stage
template <int DK, int DV>
__device__ __forceinline__ void fetch_pair(const bf16_t* ka, const bf16_t* kb, const bf16_t* va, const bf16_t* vb, int P,
                                           uint4 (&kreg)[DiffStage<DK, DV>::K_PER], uint4 (&vreg)[DiffStage<DK, DV>::V_PER]) {
  using S = DiffStage<DK, DV>;
#pragma unroll
  for (int i = 0; i < S::K_PER; ++i) {
    const int u = threadIdx.x + 256 * i;
    if (S::K_UNITS % 256 == 0 || u < S::K_UNITS) {
      const int key = u / (2 * DK / 8), part = u % (2 * DK / 8);
      kreg[i] = *reinterpret_cast<const uint4*>((key < 16 ? ka : kb) + (size_t)(key & 15) * (2 * DK) + part * 8);
    }
  }
#pragma unroll
  for (int i = 0; i < S::V_PER; ++i) {
    const int u = threadIdx.x + 256 * i;
    if (S::V_UNITS % 256 == 0 || u < S::V_UNITS) {
      const int d = u >> 2, piece = u & 3;
      vreg[i] = *reinterpret_cast<const uint4*>(((piece & 2) ? vb : va) + (size_t)d * P + (piece & 1) * 8);
    }
  }
}
template <int DK, int DV>
__device__ __forceinline__ void park_pair(bf16_t* to, const uint4 (&kreg)[DiffStage<DK, DV>::K_PER],
                                          const uint4 (&vreg)[DiffStage<DK, DV>::V_PER]) {
  using S = DiffStage<DK, DV>;
#pragma unroll
  for (int i = 0; i < S::K_PER; ++i) {
    const int u = threadIdx.x + 256 * i;
    if (S::K_UNITS % 256 == 0 || u < S::K_UNITS) {
      const int key = u / (2 * DK / 8), part = u % (2 * DK / 8);
      *reinterpret_cast<uint4*>(to + key * S::KROW + part * 8) = kreg[i];
    }
  }
#pragma unroll
  for (int i = 0; i < S::V_PER; ++i) {
    const int u = threadIdx.x + 256 * i;
    if (S::V_UNITS % 256 == 0 || u < S::V_UNITS) {
      // the piece holds keys 8 h .. 8 h + 7 of block `blk`: the quarters 2 h and 2 h + 1, four keys each
      const int d = u >> 2, piece = u & 3, blk = piece >> 1, h = piece & 1;
      bf16_t* dst = to + S::K_ELEMS + d * S::VROW + (2 * h) * 8 + blk * 4;
      *reinterpret_cast<uint2*>(dst) = make_uint2(vreg[i].x, vreg[i].y);
      *reinterpret_cast<uint2*>(dst + 8) = make_uint2(vreg[i].z, vreg[i].w);
    }
  }
}

template <int DK, int DV>
__global__ void __launch_bounds__(256)
diff_tiles_lds_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool, const int* __restrict__ table, int table_stride,
                      const int* __restrict__ tiles, const int* __restrict__ entries, bf16_t* __restrict__ out, int n_head, int n_kv,
                      int P, float scale2, int block, int window, float lambda, float eps, float out_scale, int heads_per_round) {
  using S = DiffStage<DK, DV>;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16_t* const lds = reinterpret_cast<bf16_t*>(lds_raw);      // two stages of S::ELEMS
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  // The tiles come from the one that walks the most keys to the one that walks the fewest, and workgroups start in the
  // grid's order, a compute unit taking one of every `heads_per_round` heads' worth at a time: every other such group of
  // heads walks the list backwards, so that a unit's long tile stands beside a short one.
  const int h = blockIdx.y;
  const int t = ((h / heads_per_round) & 1) ? gridDim.x - 1 - blockIdx.x : blockIdx.x;
  const int e = tiles[3 * t], tile_row0 = tiles[3 * t + 1], tile_rows = tiles[3 * t + 2];
  const int row0 = tile_row0 + 16 * wave, n_rows = tile_rows - 16 * wave;      // n_rows <= 0: a wavefront without rows (it still fetches)
  const int kvh = h / (n_head / n_kv);
  const int e_row0 = entries[4 * e], e_n = entries[4 * e + 1], e_start = entries[4 * e + 2];
  const int kv_last = e_start + e_n - 1;
  const bool live = r16 < n_rows;
  const int row = live ? row0 + r16 : tile_row0;
  const int p = e_start + (row - e_row0);
  const int lo = live ? first_visible(p, block, window) : 1, hi = live ? p : 0;
  int lo_min = live ? lo : 0x7fffffff, lo_max = live ? lo : 0, hi_min = live ? hi : 0x7fffffff, hi_max = live ? hi : -1;
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) {
    lo_min = min(lo_min, __shfl_xor(lo_min, o, 64));
    lo_max = max(lo_max, __shfl_xor(lo_max, o, 64));
    hi_min = min(hi_min, __shfl_xor(hi_min, o, 64));
    hi_max = max(hi_max, __shfl_xor(hi_max, o, 64));
  }
  // the workgroup's range of pairs: from the first key its first row sees to its last row's own
  const int p_first = e_start + (tile_row0 - e_row0), p_last = p_first + tile_rows - 1;
  const int pair0 = first_visible(p_first, block, window) / 32, pair1 = p_last / 32 + 1;
  const int* tab = table + (size_t)e * table_stride;
  const size_t page_elems = (size_t)n_kv * P * (2 * DK + DV);
  const size_t v_base = (size_t)n_kv * P * (2 * DK) + (size_t)kvh * DV * P;

  Frag8 qf[2][DK / 32];
  const bf16_t* qrow = q + ((size_t)row * n_head + h) * 2 * DK + quad * 8;
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) qf[mp][s].u = *reinterpret_cast<const uint4*>(qrow + mp * DK + s * 32);
  MapState<DV> st[2];
  st[0].clear();
  st[1].clear();

  uint4 kreg[S::K_PER], vreg[S::V_PER];
  bool validA = false, validB = false;      // of the pair in flight; the same in every lane
  auto fetch = [&](int pair) __attribute__((always_inline)) {
    const int keyA = pair * 32, keyB = keyA + 16;
    int pageA = keyA <= kv_last ? tab[keyA / P] : -1;
    int pageB = keyB <= kv_last ? tab[keyB / P] : -1;
    validA = pageA >= 0;
    validB = pageB >= 0;
    int rowA = keyA % P, rowB = keyB % P;
    if (pageA < 0) {
      pageA = tab[p_last / P];
      rowA = p_last / 16 * 16 % P;
    }
    if (pageB < 0) {
      pageB = tab[p_last / P];
      rowB = p_last / 16 * 16 % P;
    }
    const bf16_t* ka = pool + (size_t)pageA * page_elems + ((size_t)kvh * P + rowA) * (2 * DK);
    const bf16_t* kb = pool + (size_t)pageB * page_elems + ((size_t)kvh * P + rowB) * (2 * DK);
    fetch_pair<DK, DV>(ka, kb, pool + (size_t)pageA * page_elems + v_base + rowA, pool + (size_t)pageB * page_elems + v_base + rowB, P,
                       kreg, vreg);
  };
  auto park = [&](bf16_t* to) __attribute__((always_inline)) { park_pair<DK, DV>(to, kreg, vreg); };

  fetch(pair0);
  park(lds);
  bool curA = validA, curB = validB;
  __syncthreads();
  for (int pair = pair0, cur = 0; pair < pair1; ++pair, cur ^= 1) {
    const bool more = pair + 1 < pair1;
    if (more) fetch(pair + 1);
    const int keyA = pair * 32;
    if (n_rows > 0 && keyA <= hi_max && keyA + 31 >= lo_min) {
      DiffPair<DK, DV> f;
      f.keyA = keyA;
      f.keyB = keyA + 16;
      f.validA = curA;
      f.validB = curB;
      const bf16_t* ks = lds + cur * S::ELEMS;
      const bf16_t* vs = ks + S::K_ELEMS;
#pragma unroll
      for (int mp = 0; mp < 2; ++mp)
#pragma unroll
        for (int s = 0; s < DK / 32; ++s) {
          f.k[0][mp][s].u = *reinterpret_cast<const uint4*>(ks + r16 * S::KROW + mp * DK + s * 32 + quad * 8);
          f.k[1][mp][s].u = *reinterpret_cast<const uint4*>(ks + (16 + r16) * S::KROW + mp * DK + s * 32 + quad * 8);
        }
#pragma unroll
      for (int d = 0; d < DV / 16; ++d) {
        f.v[d].u = *reinterpret_cast<const uint4*>(vs + (16 * d + r16) * S::VROW + quad * 8);
      }
      const bool plain = curA && curB && keyA >= lo_max && keyA + 31 <= hi_min;
      attend_pair<DK, DV>(f, qf, lo, hi, plain, kv_last, scale2, st);
    }
    if (more) park(lds + (cur ^ 1) * S::ELEMS);
    curA = validA;
    curB = validB;
    __syncthreads();
  }
  if (n_rows > 0) finish_column<DV>(st, lambda, eps, out_scale, out + ((size_t)row * n_head + h) * DV, live);
}

// ------------------------------------------------------------------------------------------ single rows
// rows int32 [n] (null: row r is r); the 16 columns are the query heads of kv head blockIdx.y.  The four wavefronts take
// the pairs of blocks in turns; wavefronts 1..3 leave their state in LDS and the first one merges and finishes.
template <int DK, int DV>
__global__ void __launch_bounds__(256)
diff_rows_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ pool, const int* __restrict__ table, int table_stride,
                 const int* __restrict__ pos, const int* __restrict__ slot, const int* __restrict__ rows, bf16_t* __restrict__ out,
                 int n_head, int n_kv, int P, float scale2, int block, int window, float lambda, float eps, float out_scale,
                 float* __restrict__ part, int n_splits) {
  extern __shared__ float lds[];     // [3 wavefronts][2 maps][DV / 4 + 2][64]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int m = rows ? rows[blockIdx.x] : blockIdx.x;
  const int kvh = blockIdx.y;
  const int per = n_head / n_kv;
  const int p = pos[m];
  const bool live = r16 < per;
  const int h = kvh * per + (live ? r16 : 0);
  const int lo_all = first_visible(p, block, window);
  const int lo = live ? lo_all : 1, hi = live ? p : 0;
  DiffPages kv{pool, table + (size_t)slot[m] * table_stride, P, n_kv, kvh};
  Frag8 qf[2][DK / 32];
  const bf16_t* qrow = q + ((size_t)m * n_head + h) * 2 * DK + quad * 8;
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) qf[mp][s].u = *reinterpret_cast<const uint4*>(qrow + mp * DK + s * 32);
  MapState<DV> st[2];
  st[0].clear();
  st[1].clear();
  // gridDim.z workgroups share a row's keys: workgroup z, wavefront v the pairs 4 z + v, 4 z + v + 4 gridDim.z, ...
  walk<DK, DV>(kv, qf, lo_all / 32 + 4 * blockIdx.z + wave, p / 32 + 1, 4 * n_splits, lo, hi, lo_all, p, p, p, scale2, st);
  constexpr int PER_MAP = (DV / 4 + 2) * 64;
  if (wave > 0) {
    float* mine = lds + (size_t)(wave - 1) * 2 * PER_MAP;
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      float* dstp = mine + mp * PER_MAP;
#pragma unroll
      for (int d = 0; d < DV / 16; ++d)
#pragma unroll
        for (int i = 0; i < 4; ++i) dstp[(d * 4 + i) * 64 + lane] = st[mp].o[d][i];
      dstp[DV / 4 * 64 + lane] = st[mp].m;
      dstp[(DV / 4 + 1) * 64 + lane] = st[mp].l;
    }
  }
  __syncthreads();
  if (wave > 0) return;
  for (int w = 0; w < 3; ++w) {
    const float* theirs = lds + (size_t)w * 2 * PER_MAP;
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      const float* src = theirs + mp * PER_MAP;
      const float m2 = src[DV / 4 * 64 + lane], l2 = src[(DV / 4 + 1) * 64 + lane];
      const float mm = fmaxf(st[mp].m, m2);
      const float m_safe = (mm == -INFINITY) ? 0.f : mm;
      const float a = __builtin_amdgcn_exp2f(st[mp].m - m_safe), b = __builtin_amdgcn_exp2f(m2 - m_safe);
      st[mp].l = st[mp].l * a + l2 * b;
#pragma unroll
      for (int d = 0; d < DV / 16; ++d)
#pragma unroll
        for (int i = 0; i < 4; ++i) st[mp].o[d][i] = st[mp].o[d][i] * a + src[(d * 4 + i) * 64 + lane] * b;
      st[mp].m = mm;
    }
  }
  if (n_splits == 1) {
    finish_column<DV>(st, lambda, eps, out_scale, out + ((size_t)m * n_head + h) * DV, live);
    return;
  }
  // the workgroup's share goes to memory as it lies in the lanes; diff_rows_merge_kernel adds the shares up
  float* mine = part + (((size_t)blockIdx.x * n_kv + kvh) * n_splits + blockIdx.z) * 2 * PER_MAP;
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    float* dstp = mine + mp * PER_MAP;
#pragma unroll
    for (int d = 0; d < DV / 16; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) dstp[(d * 4 + i) * 64 + lane] = st[mp].o[d][i];
    dstp[DV / 4 * 64 + lane] = st[mp].m;
    dstp[(DV / 4 + 1) * 64 + lane] = st[mp].l;
  }
}

// one wavefront per (row, kv head): the shares of the workgroups that split the row's keys, in ascending order
template <int DV>
__global__ void __launch_bounds__(64)
diff_rows_merge_kernel(const float* __restrict__ part, const int* __restrict__ rows, bf16_t* __restrict__ out, int n_head, int n_kv,
                       int n_splits, float lambda, float eps, float out_scale) {
  constexpr int PER_MAP = (DV / 4 + 2) * 64;
  const int lane = threadIdx.x, r16 = lane & 15;
  const int m = rows ? rows[blockIdx.x] : blockIdx.x;
  const int kvh = blockIdx.y, per = n_head / n_kv;
  const bool live = r16 < per;
  const int h = kvh * per + (live ? r16 : 0);
  MapState<DV> st[2];
  st[0].clear();
  st[1].clear();
  for (int s = 0; s < n_splits; ++s) {
    const float* theirs = part + (((size_t)blockIdx.x * n_kv + kvh) * n_splits + s) * 2 * PER_MAP;
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      const float* src = theirs + mp * PER_MAP;
      const float m2 = src[DV / 4 * 64 + lane], l2 = src[(DV / 4 + 1) * 64 + lane];
      const float mm = fmaxf(st[mp].m, m2);
      const float m_safe = (mm == -INFINITY) ? 0.f : mm;
      const float a = __builtin_amdgcn_exp2f(st[mp].m - m_safe), b = __builtin_amdgcn_exp2f(m2 - m_safe);
      st[mp].l = st[mp].l * a + l2 * b;
#pragma unroll
      for (int d = 0; d < DV / 16; ++d)
#pragma unroll
        for (int i = 0; i < 4; ++i) st[mp].o[d][i] = st[mp].o[d][i] * a + src[(d * 4 + i) * 64 + lane] * b;
      st[mp].m = mm;
    }
  }
  finish_column<DV>(st, lambda, eps, out_scale, out + ((size_t)m * n_head + h) * DV, live);
}

// ------------------------------------------------------------------------------------------ host
static bool served(int dk, int dv, int page_size, int n_head, int n_kv) {
  auto size_ok = [](int d) { return d == 32 || d == 64 || d == 128; };
  return size_ok(dk) && size_ok(dv) && page_size % 16 == 0 && n_kv > 0 && n_head % n_kv == 0;
}

#define DA_DISPATCH(CALL)                                        \
  do {                                                           \
    if (dk == 32 && dv == 32) { CALL(32, 32); }                  \
    else if (dk == 32 && dv == 64) { CALL(32, 64); }             \
    else if (dk == 32 && dv == 128) { CALL(32, 128); }           \
    else if (dk == 64 && dv == 32) { CALL(64, 32); }             \
    else if (dk == 64 && dv == 64) { CALL(64, 64); }             \
    else if (dk == 64 && dv == 128) { CALL(64, 128); }           \
    else if (dk == 128 && dv == 32) { CALL(128, 32); }           \
    else if (dk == 128 && dv == 64) { CALL(128, 64); }           \
    else { CALL(128, 128); }                                     \
  } while (0)

extern "C" int ti_diff_attention_tiles_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* tiles,
                                            const int* entries, void* out, int n_tiles, int n_head, int n_kv, int dk, int dv,
                                            int page_size, float scale, int block, int window, float lambda, float eps,
                                            float out_scale, int use_lds, hipStream_t stream) {
  if (!served(dk, dv, page_size, n_head, n_kv)) {
    ti_set_error("diff_attention (tiles): sizes %d / %d, pages of %d are not served", dk, dv, page_size);
    return 3;
  }
  TI_REQUIRE(n_head <= 65535 && table_stride > 0 && block >= 0 && window >= 0, "diff_attention (tiles): bad arguments");
  if (n_tiles == 0) return 0;
  dim3 grid(n_tiles, n_head);
  int units = 0, device = 0;
  if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
    units = 256;
  const int heads_per_round = units / n_tiles > 0 ? units / n_tiles : 1;
  // keys and values shared through LDS (use_lds 0: every wavefront fetches its own, for tests and measurements)
#define DA_TILES(K, V)                                                                                                              \
  do {                                                                                                                              \
    if (use_lds)                                                                                                                    \
      diff_tiles_lds_kernel<K, V><<<grid, 256, 2 * DiffStage<K, V>::ELEMS * 2, stream>>>(                                           \
          (const bf16_t*)q, (const bf16_t*)pool, table, table_stride, tiles, entries, (bf16_t*)out, n_head, n_kv, page_size,        \
          scale * DA_LOG2E, block, window, lambda, eps, out_scale, heads_per_round);                                                \
    else                                                                                                                            \
      diff_tiles_kernel<K, V><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table, table_stride, tiles, entries, \
                                                        (bf16_t*)out, n_head, n_kv, page_size, scale * DA_LOG2E, block, window,     \
                                                        lambda, eps, out_scale);                                                    \
  } while (0)
  DA_DISPATCH(DA_TILES);
#undef DA_TILES
  TI_LAUNCH_CHECK();
  return 0;
}

extern "C" int ti_diff_attention_rows_bf16(const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                                           const int* slot, const int* rows, void* out, int n_rows, int n_head, int n_kv, int dk,
                                           int dv, int page_size, float scale, int block, int window, float lambda, float eps,
                                           float out_scale, float* part, int n_splits, hipStream_t stream) {
  if (!served(dk, dv, page_size, n_head, n_kv) || n_head / n_kv > 16) {
    ti_set_error("diff_attention (rows): sizes %d / %d, pages of %d, %d heads a kv head are not served", dk, dv, page_size,
                 n_kv > 0 ? n_head / n_kv : 0);
    return 3;
  }
  TI_REQUIRE(n_kv <= 65535 && table_stride > 0 && block >= 0 && window >= 0, "diff_attention (rows): bad arguments");
  TI_REQUIRE(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || part), "diff_attention (rows): %d splits need scratch", n_splits);
  if (n_rows == 0) return 0;
  dim3 grid(n_rows, n_kv, n_splits);
  const size_t lds = (size_t)3 * 2 * (dv / 4 + 2) * 64 * 4;
#define DA_ROWS(K, V)                                                                                                             \
  diff_rows_kernel<K, V><<<grid, 256, lds, stream>>>((const bf16_t*)q, (const bf16_t*)pool, table, table_stride, pos, slot, rows, \
                                                     (bf16_t*)out, n_head, n_kv, page_size, scale * DA_LOG2E, block, window,      \
                                                     lambda, eps, out_scale, part, n_splits)
  DA_DISPATCH(DA_ROWS);
#undef DA_ROWS
  TI_LAUNCH_CHECK();
  if (n_splits > 1) {
    const dim3 mgrid(n_rows, n_kv);
    if (dv == 32) diff_rows_merge_kernel<32><<<mgrid, 64, 0, stream>>>(part, rows, (bf16_t*)out, n_head, n_kv, n_splits, lambda, eps, out_scale);
    else if (dv == 64) diff_rows_merge_kernel<64><<<mgrid, 64, 0, stream>>>(part, rows, (bf16_t*)out, n_head, n_kv, n_splits, lambda, eps, out_scale);
    else diff_rows_merge_kernel<128><<<mgrid, 64, 0, stream>>>(part, rows, (bf16_t*)out, n_head, n_kv, n_splits, lambda, eps, out_scale);
    TI_LAUNCH_CHECK();
  }
  return 0;
}

// floats of scratch for ti_diff_attention_rows_bf16 with n_splits > 1
extern "C" long ti_diff_attention_rows_scratch(int n_rows, int n_kv, int dv, int n_splits) {
  return (long)n_rows * n_kv * n_splits * 2 * (dv / 4 + 2) * 64;
}
