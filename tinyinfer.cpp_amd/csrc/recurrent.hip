// Recurrent mixers: the mLSTM cell (a matrix memory per head with a stabilised exponential input
// gate), as a scan over the tokens each request brings to a step, from and into the request's state.
//
// Per head, with keys k (dk), values v (dv), a log input gate i and a log forget gate f:
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T        (dk x dv)
//   n_t = the same with k_t alone                                            (dk)
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// The gates come from pre-activations a (with a bias b): i = cap tanh((a_i + b_i) / cap),
// f = logsigmoid(cap tanh((a_f + b_f) / cap)).  State, gates and everything else here is 32-bit.
//
// One workgroup per (request of the step, head).  A wavefront owns 64 / RG columns of S; the RG lanes
// that share a column hold a share of its rows each (RPL of them), in registers, for all tokens of the
// step.  The tokens' q, k, v and gates pass through LDS sixteen at a time.  Key sizes up to 64 take
// RG = 4; larger ones RG = 8: half the rows a lane, twice the wavefronts, which hide a token's chain
// of dependent operations better (a workgroup's wavefronts are all a compute unit runs).  Every element of S, n and o is
// computed by the same sequence of operations whether its token came alone or in a portion, so a
// sequence cut differently gives the same bits.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define ML_TB 16     // tokens staged at a time

__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// MODE 0: each workgroup one (entry, head): from the request's state slot over all its tokens and back into the slot.
// Long portions are cut into chunks (`chunks` int32 [n][4] = (entry, first row, tokens, 1 if the entry's first chunk +
// 2 if its last)), three launches:
// MODE 1: every chunk but an entry's last from an empty memory (S = 0, n = 0, m = -inf), no output: what the chunk
//         alone adds (S, n, its maximum m and F, the sum of its log forget gates) goes to `chunk_buf`;
//         then mlstm_combine_kernel walks an entry's chunks and leaves in `chunk_buf` the state each chunk starts from;
// MODE 2: every chunk from that state (an entry of a single chunk: from its slot) with output; an entry's last chunk
//         writes the slot.
// chunk_buf per (chunk, head): S [dk][dv], n [dk], m of the chunk alone, F, m the chunk starts from.
template <int RPL, int RG, int MAXT, int MODE>
__global__ void __launch_bounds__(MAXT)
mlstm_scan_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v, int off_i, int off_f,
                  const float* __restrict__ bias_i, const float* __restrict__ bias_f, float* __restrict__ state,
                  long slot_stride, const int* __restrict__ entries, const int* __restrict__ chunks,
                  float* __restrict__ chunk_buf, float* __restrict__ o, int heads, int dk, int dv, float cap, float q_scale) {
  constexpr int ML_COLS = TI_WAVE / RG;   // columns of the memory per wavefront
  constexpr int DP = RPL * RG;            // rows, padded
  extern __shared__ __align__(16) float lds[];
  float* lq = lds;                        // [ML_TB][DP]
  float* lk = lq + ML_TB * DP;            // [ML_TB][DP]
  float* lv = lk + ML_TB * DP;            // [ML_TB][dv]
  float* lgi = lv + ML_TB * dv;           // [ML_TB] log input gates
  float* lgf = lgi + ML_TB;               // [ML_TB] log forget gates
  float* lm = lgf + ML_TB;                // [ML_TB] the running maximum after each token
  float* ldc = lm + ML_TB;                // [ML_TB] exp(f + m before - m after): what the memory keeps
  float* ltk = ldc + ML_TB;               // [ML_TB] exp(i - m after): what the token adds
  float* lem = ltk + ML_TB;               // [ML_TB] exp(-m after)
  const int unit = blockIdx.x, h = blockIdx.y;
  int e = unit, row0, n_tok, flags = 3;
  if (MODE == 0) {
    row0 = entries[4 * e];
    n_tok = entries[4 * e + 1];
  } else {
    e = chunks[4 * unit];
    row0 = chunks[4 * unit + 1];
    n_tok = chunks[4 * unit + 2];
    flags = chunks[4 * unit + 3];
  }
  const bool whole = (flags & 3) == 3, last = (flags & 2) != 0;
  if (MODE == 1 && last) return;          // nobody reads what an entry's last chunk adds alone
  const int slot = entries[4 * e + 3];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, rg = lane / ML_COLS, c = lane % ML_COLS;
  const int n_waves = blockDim.x >> 6;
  const size_t per_head = (size_t)dk * dv + dk + 1;
  float* slot_base = state + (size_t)slot * slot_stride + (size_t)h * per_head;
  float* cb = (MODE == 0) ? nullptr : chunk_buf + ((size_t)unit * heads + h) * (per_head + 2);
  // where the memory comes from and where it goes
  const bool from_slot = MODE == 0 || (MODE == 2 && whole);
  const float* S_src = from_slot ? slot_base : cb;
  const float* m_src = from_slot ? slot_base + per_head - 1 : cb + per_head + 1;
  float* S_dst = (MODE == 0 || (MODE == 2 && last)) ? slot_base : (MODE == 1 ? cb : nullptr);
  const int ov = heads * dv;
  const int span = n_waves * ML_COLS;
  // n is a vector, not a matrix: the lanes that share a share of the rows split that share's n between them
  // (NPL rows a lane) and add their shares of n . q up over the whole wavefront
  constexpr int NPL = RPL >= ML_COLS ? RPL / ML_COLS : 1;
  const bool n_lane = c * NPL < RPL;                 // (a quarter of fewer than 16 rows leaves lanes without one)
  const int n_row0 = rg * RPL + c * NPL;
  float S[RPL], nn[NPL];
  float m = 0.f, F = 0.f;
  for (int j0 = 0; j0 < dv; j0 += span) {
    const int j = j0 + wave * ML_COLS + c;
    const bool active = j < dv;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int r = rg * RPL + i;
      S[i] = (MODE != 1 && active && r < dk) ? S_src[(size_t)r * dv + j] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < NPL; ++i) nn[i] = (MODE != 1 && n_lane && n_row0 + i < dk) ? S_src[(size_t)dk * dv + n_row0 + i] : 0.f;
    m = (MODE == 1) ? -INFINITY : *m_src;
    F = 0.f;
    for (int t0 = 0; t0 < n_tok; t0 += ML_TB) {
      const int tb = n_tok - t0 < ML_TB ? n_tok - t0 : ML_TB;
      __syncthreads();   // the reads of the tokens before are over
      for (int idx = threadIdx.x; idx < tb * DP; idx += blockDim.x) {
        const int t = idx / DP, r = idx % DP;
        const float* row = proj + (size_t)(row0 + t0 + t) * ld;
        lq[idx] = r < dk ? row[off_q + h * dk + r] * q_scale : 0.f;
        lk[idx] = r < dk ? row[off_k + h * dk + r] : 0.f;
      }
      for (int idx = threadIdx.x; idx < tb * dv; idx += blockDim.x) {
        const int t = idx / dv, jj = idx % dv;
        lv[idx] = proj[(size_t)(row0 + t0 + t) * ld + off_v + h * dv + jj];
      }
      if ((int)threadIdx.x < tb) {
        const float* row = proj + (size_t)(row0 + t0 + threadIdx.x) * ld;
        const float ai = row[off_i + h] + bias_i[h], af = row[off_f + h] + bias_f[h];
        lgi[threadIdx.x] = cap * tanhf(ai / cap);
        lgf[threadIdx.x] = log_sigmoid_f(cap * tanhf(af / cap));
      }
      __syncthreads();
      // the maxima are a chain over the tokens (one thread walks it); the three exponentials of a token hang on
      // nothing else, so a thread per token takes them off the loop that every lane walks
      if (threadIdx.x == 0) {
        float mm = m;
        for (int t = 0; t < tb; ++t) {
          mm = fmaxf(lgf[t] + mm, lgi[t]);
          lm[t] = mm;
        }
      }
      __syncthreads();
      if ((int)threadIdx.x < tb) {
        const int t = threadIdx.x;
        const float before = t ? lm[t - 1] : m, after = lm[t];
        ldc[t] = expf(lgf[t] + before - after);
        ltk[t] = expf(lgi[t] - after);
        lem[t] = expf(-after);
      }
      __syncthreads();
      for (int t = 0; t < tb; ++t) {
        const float decay = ldc[t], take = ltk[t];
        F += lgf[t];
        const float tv = active ? take * lv[t * dv + j] : 0.f;
        const float4* q4 = reinterpret_cast<const float4*>(lq + t * DP + rg * RPL);
        const float4* k4 = reinterpret_cast<const float4*>(lk + t * DP + rg * RPL);
        float a4[4] = {0.f, 0.f, 0.f, 0.f};     // four sums side by side: shorter chains
#pragma unroll
        for (int i = 0; i < RPL; i += 4) {
          const float4 qq = q4[i / 4], kk = k4[i / 4];
          const float qa[4] = {qq.x, qq.y, qq.z, qq.w}, ka[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            S[i + u] = fmaf(ka[u], tv, decay * S[i + u]);
            if (MODE != 1) a4[u] = fmaf(S[i + u], qa[u], a4[u]);
          }
        }
        float nq = 0.f;
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
          const float kr = n_lane ? lk[t * DP + n_row0 + i] : 0.f;      // (rows beyond dk hold zeros)
          nn[i] = fmaf(take, kr, decay * nn[i]);
          if (MODE != 1) nq = fmaf(nn[i], n_lane ? lq[t * DP + n_row0 + i] : 0.f, nq);
        }
        if (MODE != 1) {
          float acc = (a4[0] + a4[1]) + (a4[2] + a4[3]);
#pragma unroll
          for (int off = ML_COLS; off < TI_WAVE; off <<= 1) acc += __shfl_xor(acc, off, TI_WAVE);
          nq = group_sum<TI_WAVE>(nq);
          const float denom = fmaxf(fabsf(nq), lem[t]) + 1e-6f;
          if (rg == 0 && active) o[(size_t)(row0 + t0 + t) * ov + h * dv + j] = acc / denom;
        }
      }
      m = lm[tb - 1];
    }
    if (active && S_dst) {
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int r = rg * RPL + i;
        if (r < dk) S_dst[(size_t)r * dv + j] = S[i];
      }
    }
  }
  // n and m: every wavefront holds the same; the first one writes, after all have read
  __syncthreads();
  if (S_dst && wave == 0) {
#pragma unroll
    for (int i = 0; i < NPL; ++i)
      if (n_lane && n_row0 + i < dk) S_dst[(size_t)dk * dv + n_row0 + i] = nn[i];
    if (lane == 0) {
      S_dst[per_head - 1] = m;
      if (MODE == 1) S_dst[per_head] = F;
    }
  }
}

// An entry's chunks in order, for every entry of more than one chunk (`spans` int32 [R][2] = (first chunk, chunks)):
// with the running state (S, n, m) starting at the request's slot, chunk c gets the state it starts from in place
// of what it added alone (A_c, a_c, m_c, F_c), and the running state goes on as
//   m' = max(F_c + m, m_c);  S' = exp(F_c + m - m') S + exp(m_c - m') A_c;  n' likewise
// (the recurrence of the cell, taken a chunk at a time).  grid (entries, heads, slices of the elements).
__global__ void __launch_bounds__(256)
mlstm_combine_kernel(const float* __restrict__ state, long slot_stride, const int* __restrict__ entries,
                     const int* __restrict__ spans, float* __restrict__ chunk_buf, int heads, int dk, int dv) {
  const int e = blockIdx.x, h = blockIdx.y;
  const int first = spans[2 * e], n = spans[2 * e + 1];
  if (n < 2) return;
  const size_t per_head = (size_t)dk * dv + dk + 1, elems = per_head - 1, stride = per_head + 2;
  const float* slot_base = state + (size_t)entries[4 * e + 3] * slot_stride + (size_t)h * per_head;
  float m = slot_base[per_head - 1];
  const size_t idx = (size_t)blockIdx.z * blockDim.x + threadIdx.x;      // this thread's element of (S, n)
  const bool mine = idx < elems;
  float run = mine ? slot_base[idx] : 0.f;
  float* cb0 = chunk_buf + ((size_t)first * heads + h) * stride;
  const size_t step = (size_t)heads * stride;                            // from a chunk to the next
  // what the chunks added alone does not hang on the running state: four chunks' loads go out together
  for (int c0 = 0; c0 < n; c0 += 4) {
    float loc[4], m_c[4], F_c[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int cidx = c0 + k < n ? c0 + k : n - 1;
      const float* cb = cb0 + (size_t)cidx * step;
      const bool adds = c0 + k + 1 < n;                                  // an entry's last chunk has left nothing
      loc[k] = (mine && adds) ? cb[idx] : 0.f;
      m_c[k] = adds ? cb[per_head - 1] : 0.f;
      F_c[k] = adds ? cb[per_head] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (c0 + k >= n) break;
      float* cb = cb0 + (size_t)(c0 + k) * step;
      if (mine) cb[idx] = run;
      if (idx == 0) cb[per_head + 1] = m;
      if (c0 + k + 1 < n) {
        const float m_new = fmaxf(F_c[k] + m, m_c[k]);
        run = fmaf(expf(m_c[k] - m_new), loc[k], expf(F_c[k] + m - m_new) * run);
        m = m_new;
      }
    }
  }
}

static int mlstm_shape(int heads, int dk, int dv, float cap, int* rpl, int* waves, size_t* lds) {
  TI_REQUIRE(heads > 0 && heads <= 65535 && dk >= 1 && dk <= 256 && dv >= 1, "mlstm: heads %d, key size %d (up to 256), value size %d",
             heads, dk, dv);
  TI_REQUIRE(cap > 0.f, "mlstm: the gates' cap must be positive");
  // rows a lane and lanes a column: 8 x 4, 16 x 4, 16 x 8, 32 x 8 for key sizes up to 32, 64, 128, 256
  *rpl = dk <= 32 ? 8 : dk <= 128 ? 16 : 32;
  const int rg = dk <= 64 ? 4 : 8, cols = 64 / rg;
  const int max_waves = *rpl <= 16 ? 16 : 8;
  *waves = (dv + cols - 1) / cols;
  if (*waves > max_waves) *waves = max_waves;
  *lds = ((size_t)ML_TB * (2 * *rpl * rg + dv) + 6 * ML_TB) * sizeof(float);
  TI_REQUIRE(*lds <= 64 * 1024, "mlstm: value size %d needs %zu bytes of LDS", dv, *lds);
  return 0;
}

#define ML_ARGS proj, ld, off_q, off_k, off_v, off_i, off_f, bias_i, bias_f, state, slot_stride, entries, chunks, chunk_buf, o, heads, dk, \
                dv, cap, q_scale
#define ML_LAUNCH(MODE, GRID)                                                                                  \
  do {                                                                                                         \
    if (dk <= 32) mlstm_scan_kernel<8, 4, 1024, MODE><<<GRID, waves * 64, lds, stream>>>(ML_ARGS);             \
    else if (dk <= 64) mlstm_scan_kernel<16, 4, 1024, MODE><<<GRID, waves * 64, lds, stream>>>(ML_ARGS);       \
    else if (dk <= 128) mlstm_scan_kernel<16, 8, 1024, MODE><<<GRID, waves * 64, lds, stream>>>(ML_ARGS);      \
    else mlstm_scan_kernel<32, 8, 512, MODE><<<GRID, waves * 64, lds, stream>>>(ML_ARGS);                      \
  } while (0)

// proj f32 [M, ld]: the projections of the step's rows; off_*: the columns where the heads' q [heads][dk],
// k [heads][dk], v [heads][dv] and the gate pre-activations i, f [heads] start.  state f32: per slot
// (slot_stride floats apart) [heads][dk dv + dk + 1] = S row-major [dk][dv], n, m.  entries int32 [R][4] =
// (first row, tokens, -, state slot).  o f32 [M, heads dv].
extern "C" int ti_mlstm_scan(const float* proj, int ld, int off_q, int off_k, int off_v, int off_i, int off_f,
                             const float* bias_i, const float* bias_f, float* state, long slot_stride, const int* entries,
                             int n_entries, float* o, int heads, int dk, int dv, float cap, float q_scale,
                             hipStream_t stream) {
  int rpl, waves;
  size_t lds;
  if (int rc = mlstm_shape(heads, dk, dv, cap, &rpl, &waves, &lds)) return rc;
  if (n_entries == 0) return 0;
  const int* chunks = nullptr;
  float* chunk_buf = nullptr;
  ML_LAUNCH(0, dim3(n_entries, heads));
  TI_LAUNCH_CHECK();
  return 0;
}

// The same with the entries' tokens cut into chunks that run side by side: chunks int32 [n_chunks][4] = (entry,
// first row, tokens, 1 if the entry's first chunk + 2 if its last), in the entries' order; spans int32 [n_entries][2]
// = (an entry's first chunk, its number of chunks); chunk_buf f32 [n_chunks][heads][dk dv + dk + 3] scratch.  Every
// chunk alone, then the entries' chunks in order (element-wise), then every chunk from the state it starts from.
// Where the chunks are cut changes the order of the sums: the same values up to rounding, not the same bits.
extern "C" int ti_mlstm_scan_chunked(const float* proj, int ld, int off_q, int off_k, int off_v, int off_i, int off_f,
                                     const float* bias_i, const float* bias_f, float* state, long slot_stride,
                                     const int* entries, int n_entries, const int* chunks, int n_chunks, const int* spans,
                                     float* chunk_buf, float* o, int heads, int dk, int dv, float cap, float q_scale,
                                     hipStream_t stream) {
  int rpl, waves;
  size_t lds;
  if (int rc = mlstm_shape(heads, dk, dv, cap, &rpl, &waves, &lds)) return rc;
  TI_REQUIRE(chunks && spans && chunk_buf && n_chunks >= n_entries, "mlstm: %d chunks for %d entries, or no lists", n_chunks, n_entries);
  if (n_entries == 0) return 0;
  if (n_chunks > n_entries) {
    ML_LAUNCH(1, dim3(n_chunks, heads));
    const size_t elems = (size_t)dk * dv + dk;
    const unsigned slices = (unsigned)((elems + 255) / 256);
    mlstm_combine_kernel<<<dim3(n_entries, heads, slices), 256, 0, stream>>>(state, slot_stride, entries, spans, chunk_buf, heads,
                                                                            dk, dv);
  }
  ML_LAUNCH(2, dim3(n_chunks, heads));
  TI_LAUNCH_CHECK();
  return 0;
}

// out[m, h, j] = o[m, h, j] / sqrt(mean_j o[m, h, :]^2 + eps) * w[h dv + j] * sigmoid(gate[m, h dv + j])
// (gate: rows of `ld` floats, the head's pre-activations from column off_g on), in T.  A wavefront per (row, head).
template <typename T>
__global__ void __launch_bounds__(64)
gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, int ld, int off_g,
                       const float* __restrict__ w, T* __restrict__ out, int heads, int dv, float eps) {
  const int m = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* src = o + ((size_t)m * heads + h) * dv;
  float ss = 0.f;
  for (int j = lane; j < dv; j += TI_WAVE) ss = fmaf(src[j], src[j], ss);
  const float scale = 1.0f / sqrtf(group_sum<TI_WAVE>(ss) / (float)dv + eps);
  const float* g = gate + (size_t)m * ld + off_g + h * dv;
  T* dst = out + ((size_t)m * heads + h) * dv;
  for (int j = lane; j < dv; j += TI_WAVE) {
    const float sg = 1.0f / (1.0f + expf(-g[j]));
    st<T>(dst + j, src[j] * scale * w[h * dv + j] * sg);
  }
}

extern "C" int ti_gated_head_norm(int out_dtype, const float* o, const float* gate, int ld, int off_g, const float* w,
                                  void* out, int M, int heads, int dv, float eps, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && heads > 0 && heads <= 65535 && dv > 0, "gated_head_norm: bad sizes M=%d heads=%d dv=%d", M, heads, dv);
  if (M == 0) return 0;
  dim3 grid(M, heads);
  if (out_dtype == TI_F32)
    gated_head_norm_kernel<float><<<grid, 64, 0, stream>>>(o, gate, ld, off_g, w, (float*)out, heads, dv, eps);
  else if (out_dtype == TI_BF16)
    gated_head_norm_kernel<bf16_t><<<grid, 64, 0, stream>>>(o, gate, ld, off_g, w, (bf16_t*)out, heads, dv, eps);
  else
    TI_REQUIRE(false, "gated_head_norm: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}
