// Differential attention for any sizes, float32 or bfloat16 storage, 32-bit arithmetic:
//   a short causal convolution over time on the channels of a fused q/k/v projection, with the last
//   taps - 1 projected rows of every request kept as its state;
//   the preparation of queries and keys (RMS norm per head and map, rotation of the first `rot_dims`
//   entries in the half-split layout) and the cache write;
//   the attention itself: every query head holds two maps (two queries against two keys, one value),
//   each an ordinary softmax over the visible keys; o = a1 - lambda a2, divided by its root mean
//   square over the value size and multiplied by `out_scale`.
// A key is visible to a query at position p if it is not later, lies in p's block of `block` positions
// counted from position 0 (block 0: no blocks) and, with a window, at most window - 1 behind.
// A page is K [n_kv][P][2 dk] (a row's two maps side by side) | V [n_kv][dv][P].
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

// ------------------------------------------------------------ short convolution over time
// out[m, c] = sum_j taps[c][j] * u(p - (K - 1) + j)[c], p the position of row m.  Rows of positions from the
// entry's start on are rows of this step; earlier ones are the request's state [K - 1][C] (row i is position
// start - (K - 1) + i; zeros at admission stand for what lies before the sequence).  Ascending j, fused
// multiply-adds: the same bits however the tokens were cut into steps.
__global__ void __launch_bounds__(256)
short_conv_kernel(const float* __restrict__ u, const float* __restrict__ taps, const float* __restrict__ state,
                  const int* __restrict__ entries, const int* __restrict__ entry_of, const int* __restrict__ pos,
                  float* __restrict__ out, int C, int K) {
  const int m = blockIdx.x;
  const int e = entry_of[m];
  const int row0 = entries[4 * e], start = entries[4 * e + 2], slot = entries[4 * e + 3];
  const int p = pos[m];
  const float* st_rows = state + (size_t)slot * (K - 1) * C;
  for (int c = threadIdx.x; c < C; c += 256) {
    float acc = 0.f;
    for (int j = 0; j < K; ++j) {
      const int s = p - (K - 1) + j;
      const float v = s >= start ? u[(size_t)(row0 + s - start) * C + c] : st_rows[(size_t)(s - start + K - 1) * C + c];
      acc = fmaf(taps[(size_t)c * K + j], v, acc);
    }
    out[(size_t)m * C + c] = acc;
  }
}

// the state after the step: the last K - 1 rows of the sequence so far.  A thread owns a channel and walks the
// state's rows upwards: what it still reads of the old state lies above what it has written.
__global__ void __launch_bounds__(256)
short_conv_state_kernel(const float* __restrict__ u, float* __restrict__ state, const int* __restrict__ entries, int C, int K) {
  const int e = blockIdx.x;
  const int row0 = entries[4 * e], n = entries[4 * e + 1], slot = entries[4 * e + 3];
  float* st_rows = state + (size_t)slot * (K - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256)
    for (int i = 0; i < K - 1; ++i) {
      const int r = n - (K - 1) + i;      // the step's row that lands here; below zero: a row the state already holds
      st_rows[(size_t)i * C + c] = r >= 0 ? u[(size_t)(row0 + r) * C + c] : st_rows[(size_t)(i + n) * C + c];
    }
}

extern "C" int ti_short_conv(const float* u, const float* taps, float* state, const int* entries, int n_entries,
                             const int* entry_of, const int* pos, float* out, int M, int C, int K, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && C > 0 && K >= 1 && n_entries >= 0, "short_conv: bad sizes M=%d C=%d taps=%d", M, C, K);
  TI_REQUIRE(K == 1 || state, "short_conv: %d taps need a state", K);
  if (M == 0) return 0;
  short_conv_kernel<<<M, 256, 0, stream>>>(u, taps, state, entries, entry_of, pos, out, C, K);
  TI_LAUNCH_CHECK();
  if (K > 1 && n_entries > 0) {
    dim3 grid(n_entries, (C + 255) / 256 < 64 ? (C + 255) / 256 : 64);
    short_conv_state_kernel<<<grid, 256, 0, stream>>>(u, state, entries, C, K);
    TI_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------------------ queries and keys prepared, cache written
// qkv f32 [M, n_head 2 dk + n_kv 2 dk + n_kv dv].  Every run of dk entries of q and k (a head's map) is divided
// by its root mean square and multiplied by the weight (q_w, k_w: [dk], shared by all heads and maps), then its
// first rot_dims entries are turned: entry i with entry i + rot_dims / 2 by the angle pos * inv_freq[i], cosine and
// sine times `mag` (the table [table_len][rot_dims / 2][2] holds them ready for positions below table_len).
// q goes to q_out (T) [M, n_head 2 dk], k and v into the page of the token's position.
// CONV: the rows of qkv are what the projection left, and every channel first passes the short convolution above (taps,
// state, entries, entry_of as in short_conv_kernel; the state itself is moved on by short_conv_state_kernel afterwards):
// the same sums in the same order as the convolution on its own, so the same bits.
template <typename T, bool CONV>
__global__ void __launch_bounds__(256)
diff_qk_prep_kernel(const float* __restrict__ qkv, const float* __restrict__ taps, const float* __restrict__ state,
                    const int* __restrict__ entries, const int* __restrict__ entry_of, int K,
                    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
                    const float* __restrict__ inv_freq, const float* __restrict__ rope_table, int table_len, float mag,
                    int rot_dims, const int* __restrict__ pos, const int* __restrict__ slot, const int* __restrict__ table,
                    int table_stride, T* __restrict__ pool, T* __restrict__ q_out, int n_head, int n_kv, int dk, int dv, int P) {
  __shared__ float s_unit[4][256];      // a wavefront's unit after the convolution (dk <= 256)
  const int m = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int p = pos[m];
  const int nq = n_head * 2 * dk, nk = n_kv * 2 * dk, nv = n_kv * dv;
  const int C = nq + nk + nv;
  const float* row = qkv + (size_t)m * C;
  int row0 = 0, start = 0;
  const float* st_rows = nullptr;
  if (CONV) {
    const int e = entry_of[m];
    row0 = entries[4 * e];
    start = entries[4 * e + 2];
    st_rows = state + (size_t)entries[4 * e + 3] * (K - 1) * C;
  }
  // channel c of this token behind the convolution (or as it is)
  auto channel = [&](int c) {
    if (!CONV) return row[c];
    float acc = 0.f;
    for (int j = 0; j < K; ++j) {
      const int s = p - (K - 1) + j;
      const float v = s >= start ? qkv[(size_t)(row0 + s - start) * C + c] : st_rows[(size_t)(s - start + K - 1) * C + c];
      acc = fmaf(taps[(size_t)c * K + j], v, acc);
    }
    return acc;
  };
  const int page = table[(size_t)slot[m] * table_stride + p / P];
  const int r = p % P;
  T* base = pool + (size_t)max(page, 0) * ((size_t)n_kv * P * (2 * dk + dv));
  const int half = rot_dims / 2;
  const int units = 2 * n_head + 2 * n_kv;
  float* unit = s_unit[wave];
  // a wavefront's piece of work: a map of a head (norm, rotation), or 64 channels of v; four pieces a workgroup
  const int u = blockIdx.y * 4 + wave;
  if (u < units) {
    const bool is_q = u < 2 * n_head;
    const float* w = is_q ? q_w : k_w;
    float ss = 0.f;
    for (int d = lane; d < dk; d += 64) {
      const float v = channel(u * dk + d);          // q's units, then k's: the row holds them in this order
      unit[d] = v;
      ss = fmaf(v, v, ss);
    }
    const float scale = 1.0f / sqrtf(group_sum<64>(ss) / (float)dk + eps);
    T* dst;
    if (is_q) {
      dst = q_out + (size_t)m * nq + (size_t)u * dk;
    } else {
      if (page < 0) return;        // the host reserves pages first; never write astray
      const int ku = u - 2 * n_head;
      dst = base + ((size_t)(ku >> 1) * P + r) * (2 * dk) + (size_t)(ku & 1) * dk;
    }
    for (int d = lane; d < dk; d += 64) {
      float v = unit[d] * scale * (w ? w[d] : 1.f);
      if (d < rot_dims) {
        const int i = d < half ? d : d - half;
        const int other = d < half ? d + half : d - half;
        const float o = unit[other] * scale * (w ? w[other] : 1.f);
        float c, s;
        if (rope_table && p < table_len) {
          c = rope_table[((size_t)p * half + i) * 2];
          s = rope_table[((size_t)p * half + i) * 2 + 1];
        } else {
          const float a = (float)p * inv_freq[i];
          c = cosf(a) * mag;
          s = sinf(a) * mag;
        }
        v = d < half ? v * c - o * s : v * c + o * s;
      }
      st<T>(dst + d, v);
    }
    return;
  }
  const int e = (u - units) * 64 + lane;
  if (page < 0 || e >= nv) return;
  T* vbase = base + (size_t)n_kv * P * 2 * dk;
  const int h = e / dv, d = e % dv;
  st<T>(vbase + ((size_t)h * dv + d) * P + r, channel(nq + nk + e));
}

// taps f32 [C][K] (null: no convolution), state f32 [slots][K - 1][C], entries int32 [n_entries][4], entry_of int32 [M]
extern "C" int ti_diff_qk_prep(int dtype, const float* qkv, const float* taps, float* state, const int* entries, int n_entries,
                               const int* entry_of, int K, const float* q_w, const float* k_w, float eps, const float* inv_freq,
                               const float* rope_table, int table_len, float mag, int rot_dims, const int* pos, const int* slot,
                               const int* table, int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int dk,
                               int dv, int page_size, hipStream_t stream) {
  TI_REQUIRE(n_head > 0 && n_kv > 0 && dk > 0 && dk <= 256 && dv > 0 && page_size > 0 && table_stride > 0,
             "diff_qk_prep: bad sizes heads=%d kv_heads=%d dk=%d dv=%d page=%d", n_head, n_kv, dk, dv, page_size);
  TI_REQUIRE(rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq),
             "diff_qk_prep: %d rotated entries do not fit a key of %d", rot_dims, dk);
  TI_REQUIRE(!taps || (K >= 1 && entries && entry_of && (K == 1 || state)), "diff_qk_prep: the convolution needs taps, entries and a state");
  if (M == 0) return 0;
  const int pieces = 2 * n_head + 2 * n_kv + (n_kv * dv + 63) / 64;
  const dim3 grid(M, (pieces + 3) / 4);
#define DQ_LAUNCH(T, CONV)                                                                                                          \
  diff_qk_prep_kernel<T, CONV><<<grid, 256, 0, stream>>>(qkv, taps, state, entries, entry_of, K, q_w, k_w, eps, inv_freq, rope_table,  \
                                                         table_len, mag, rot_dims, pos, slot, table, table_stride, (T*)pool,       \
                                                         (T*)q_out, n_head, n_kv, dk, dv, page_size)
  if (dtype == TI_F32) {
    if (taps) DQ_LAUNCH(float, true);
    else DQ_LAUNCH(float, false);
  } else if (dtype == TI_BF16) {
    if (taps) DQ_LAUNCH(bf16_t, true);
    else DQ_LAUNCH(bf16_t, false);
  } else {
    TI_REQUIRE(false, "diff_qk_prep: unknown dtype %d", dtype);
  }
#undef DQ_LAUNCH
  TI_LAUNCH_CHECK();
  if (taps && K > 1 && n_entries > 0) {
    const int C = n_head * 2 * dk + n_kv * (2 * dk + dv);
    dim3 grid(n_entries, (C + 255) / 256 < 64 ? (C + 255) / 256 : 64);
    short_conv_state_kernel<<<grid, 256, 0, stream>>>(qkv, state, entries, C, K);
    TI_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------------------ the attention, a workgroup per row and head
// Sixteen groups of sixteen lanes walk the visible keys in turns (key lo + g, lo + g + 16, ...: a key's group
// depends on its position alone), each with a running softmax per map; the groups are merged in a fixed order.
#define DA_GROUPS 16
#define DA_LANES 16
template <typename T, int DPL>
__global__ void __launch_bounds__(256)
diff_attention_kernel(const T* __restrict__ q, const T* __restrict__ pool, const int* __restrict__ table, int table_stride,
                      const int* __restrict__ pos, const int* __restrict__ slot, T* __restrict__ out, int n_head, int n_kv,
                      int dk, int dv, int P, float scale, int block, int window, float lambda, float eps, float out_scale) {
  constexpr int HD = DPL * DA_LANES;
  __shared__ float s_o[2][DA_GROUPS][HD];
  __shared__ float s_m[2][DA_GROUPS], s_l[2][DA_GROUPS];
  __shared__ float red[4];
  const int m = blockIdx.x, h = blockIdx.y;
  const int g = threadIdx.x / DA_LANES, lane = threadIdx.x % DA_LANES;
  const int kvh = h / (n_head / n_kv);
  const int p_q = pos[m];
  int lo = block > 0 ? (p_q / block) * block : 0;
  if (window > 0 && p_q - window + 1 > lo) lo = p_q - window + 1;
  const int* tab = table + (size_t)slot[m] * table_stride;
  const size_t page_elems = (size_t)n_kv * P * (2 * dk + dv);
  const size_t k_off = (size_t)kvh * P * 2 * dk;
  const size_t v_off = (size_t)n_kv * P * 2 * dk + (size_t)kvh * dv * P;

  float q1[DPL], q2[DPL], o1[DPL], o2[DPL];
  const T* qh = q + ((size_t)m * n_head + h) * 2 * dk;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = lane + i * DA_LANES;
    q1[i] = d < dk ? ld<T>(qh + d) : 0.f;
    q2[i] = d < dk ? ld<T>(qh + dk + d) : 0.f;
    o1[i] = o2[i] = 0.f;
  }
  float m1 = -INFINITY, m2 = -INFINITY, l1 = 0.f, l2 = 0.f;
  for (int p = lo + g; p <= p_q; p += DA_GROUPS) {
    const int page = tab[p / P];
    if (page < 0) continue;
    const T* kp = pool + (size_t)page * page_elems + k_off + (size_t)(p % P) * 2 * dk;
    const T* vp = pool + (size_t)page * page_elems + v_off + (p % P);
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + i * DA_LANES;
      if (d < dk) {
        s1 = fmaf(q1[i], ld<T>(kp + d), s1);
        s2 = fmaf(q2[i], ld<T>(kp + dk + d), s2);
      }
    }
    s1 = group_sum<DA_LANES>(s1) * scale;
    s2 = group_sum<DA_LANES>(s2) * scale;
    const float n1 = fmaxf(m1, s1), n2 = fmaxf(m2, s2);
    const float a1 = expf(m1 - n1), a2 = expf(m2 - n2);
    const float w1 = expf(s1 - n1), w2 = expf(s2 - n2);
    l1 = l1 * a1 + w1;
    l2 = l2 * a2 + w2;
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + i * DA_LANES;
      if (d < dv) {
        const float v = ld<T>(vp + (size_t)d * P);
        o1[i] = o1[i] * a1 + w1 * v;
        o2[i] = o2[i] * a2 + w2 * v;
      }
    }
    m1 = n1;
    m2 = n2;
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    s_o[0][g][lane + i * DA_LANES] = o1[i];
    s_o[1][g][lane + i * DA_LANES] = o2[i];
  }
  if (lane == 0) {
    s_m[0][g] = m1;
    s_l[0][g] = l1;
    s_m[1][g] = m2;
    s_l[1][g] = l2;
  }
  __syncthreads();
  // thread d merges entry d of both maps (dv <= 256), then the head's root mean square over all entries
  const int d = threadIdx.x;
  float o = 0.f;
  if (d < dv) {
    float a[2];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      float mm = -INFINITY;
#pragma unroll
      for (int j = 0; j < DA_GROUPS; ++j) mm = fmaxf(mm, s_m[mp][j]);
      float lt = 0.f, acc = 0.f;
#pragma unroll
      for (int j = 0; j < DA_GROUPS; ++j) {
        const float w = (s_m[mp][j] == -INFINITY) ? 0.f : expf(s_m[mp][j] - mm);
        lt += s_l[mp][j] * w;
        acc += s_o[mp][j][d] * w;
      }
      a[mp] = acc / lt;
    }
    o = a[0] - lambda * a[1];
  }
  const float ss = block_sum<256>(o * o, red);
  if (d < dv) st<T>(out + ((size_t)m * n_head + h) * dv + d, o * (1.0f / sqrtf(ss / (float)dv + eps)) * out_scale);
}

template <typename T>
static int launch_diff(int dpl, dim3 grid, const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                       const int* slot, void* out, int n_head, int n_kv, int dk, int dv, int P, float scale, int block,
                       int window, float lambda, float eps, float out_scale, hipStream_t stream) {
#define DA_CASE(D)                                                                                                      \
  case D:                                                                                                               \
    diff_attention_kernel<T, D><<<grid, 256, 0, stream>>>((const T*)q, (const T*)pool, table, table_stride, pos, slot,   \
                                                          (T*)out, n_head, n_kv, dk, dv, P, scale, block, window, lambda, \
                                                          eps, out_scale);                                              \
    break;
  switch (dpl) {
    DA_CASE(1) DA_CASE(2) DA_CASE(3) DA_CASE(4) DA_CASE(5) DA_CASE(6) DA_CASE(7) DA_CASE(8)
    DA_CASE(9) DA_CASE(10) DA_CASE(11) DA_CASE(12) DA_CASE(13) DA_CASE(14) DA_CASE(15) DA_CASE(16)
    default:
      return 1;
  }
#undef DA_CASE
  return 0;
}

// q: [M, n_head, 2, dk], out: [M, n_head, dv] in T
extern "C" int ti_diff_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride,
                                      const int* pos, const int* slot, void* out, int M, int n_head, int n_kv, int dk, int dv,
                                      int page_size, float scale, int block, int window, float lambda, float eps,
                                      float out_scale, hipStream_t stream) {
  TI_REQUIRE(dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256, "diff_attention: key size %d / value size %d are not served (up to 256)",
             dk, dv);
  TI_REQUIRE(n_head > 0 && n_kv > 0 && n_head % n_kv == 0, "diff_attention: heads %d / kv_heads %d", n_head, n_kv);
  TI_REQUIRE(n_head <= 65535, "diff_attention: too many heads (%d)", n_head);
  TI_REQUIRE(page_size > 0 && table_stride > 0 && block >= 0 && window >= 0, "diff_attention: bad page_size %d / table_stride %d",
             page_size, table_stride);
  if (M == 0) return 0;
  dim3 grid(M, n_head);
  const int big = dk > dv ? dk : dv;
  const int dpl = (big + DA_LANES - 1) / DA_LANES;
  int rc;
  if (dtype == TI_F32)
    rc = launch_diff<float>(dpl, grid, q, pool, table, table_stride, pos, slot, out, n_head, n_kv, dk, dv, page_size, scale, block,
                            window, lambda, eps, out_scale, stream);
  else if (dtype == TI_BF16)
    rc = launch_diff<bf16_t>(dpl, grid, q, pool, table, table_stride, pos, slot, out, n_head, n_kv, dk, dv, page_size, scale, block,
                             window, lambda, eps, out_scale, stream);
  else
    TI_REQUIRE(false, "diff_attention: unknown dtype %d", dtype);
  TI_REQUIRE(rc == 0, "diff_attention: no kernel for sizes %d / %d", dk, dv);
  TI_LAUNCH_CHECK();
  return 0;
}
