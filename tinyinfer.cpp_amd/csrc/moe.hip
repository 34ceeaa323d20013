// A mixture of experts for any sizes, float32 or bfloat16 storage: the router (logits and scores in
// 32-bit, the `top` largest scores chosen, ties to the lower index) and the experts row by row:
//   y[m] = sum over the chosen experts e, in the order they were chosen, of  W_down[e] act(W_up[e] (s_e h[m]))
// with the score scaling the expert's input (scale_input) or its output, and act = relu(z)^2.
// Products accumulate in 32-bit with fused multiply-adds in a fixed order; what a product reads is rounded
// to the storage type first (the scaled input, the activated rows), as a matrix-core kernel's operands are.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 64

// score kinds
#define MOE_SIGMOID 0
#define MOE_SOFTMAX 1

template <typename T> struct Piece;
template <> struct Piece<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  }
};
template <> struct Piece<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
    const uint4 a = *reinterpret_cast<const uint4*>(p);
    const unsigned w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// the wavefront's share of a . b over n elements: a in LDS or memory as floats through `fa`, b a row of the weight
template <typename T, bool VEC, class FA>
__device__ __forceinline__ float wave_dot(FA fa, const T* __restrict__ b, int n, int lane) {
  float z = 0.f;
  if (VEC) {
    constexpr int N = Piece<T>::N;
    for (int c = lane * N; c < n; c += 64 * N) {
      float v[N];
      Piece<T>::load(b + c, v);
#pragma unroll
      for (int i = 0; i < N; ++i) z = fmaf(fa(c + i), v[i], z);
    }
  } else {
    for (int c = lane; c < n; c += 64) z = fmaf(fa(c), ld<T>(b + c), z);
  }
  return group_sum<64>(z);
}

// ------------------------------------------------------------ router
// A workgroup per token.  Logits: wavefront w takes experts w, w + 4, ...; lanes share the token's row in pieces of
// 16 bytes (lane l the pieces l, l + 64, ... in ascending order, then a butterfly).  Choice: the first wavefront
// holds the scores (lane l the experts l, l + 64, ...) and takes the largest `top` times.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ h, const float* __restrict__ router, int* __restrict__ ids, float* __restrict__ wts,
                 int W, int E, int top, int score_kind, int renormalize) {
  __shared__ float s_score[MOE_MAX_EXPERTS];
  __shared__ float red[4];
  const int m = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* row = h + (size_t)m * W;
  for (int e = wave; e < E; e += 4) {
    const float z = wave_dot<T, VEC>([&](int c) { return router[(size_t)e * W + c]; }, row, W, lane);
    if (lane == 0) s_score[e] = z;
  }
  __syncthreads();
  if (score_kind == MOE_SOFTMAX) {
    float mx = -INFINITY;
    for (int e = threadIdx.x; e < E; e += 256) mx = fmaxf(mx, s_score[e]);
    mx = block_max<256>(mx, red);
    float sum = 0.f;
    for (int e = threadIdx.x; e < E; e += 256) sum += expf(s_score[e] - mx);
    sum = block_sum<256>(sum, red);
    for (int e = threadIdx.x; e < E; e += 256) s_score[e] = expf(s_score[e] - mx) / sum;
  } else {
    for (int e = threadIdx.x; e < E; e += 256) s_score[e] = 1.0f / (1.0f + expf(-s_score[e]));
  }
  __syncthreads();
  if (wave != 0) return;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float s = s_score[e];
      if (s > best) {      // ascending e: the first of equals stays
        best = s;
        at = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oa = __shfl_xor(at, o, 64);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (lane == 0) {
      ids[(size_t)m * top + k] = at;
      wts[(size_t)m * top + k] = best;
      s_score[at] = -INFINITY;
    }
    total += best;
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  if (renormalize && lane < top) wts[(size_t)m * top + lane] /= total;
}

extern "C" int ti_moe_route(int dtype, const void* h, const float* router, int* ids, float* wts, int M, int W, int E, int top,
                            int score_kind, int renormalize, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && W > 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= E && top <= MOE_MAX_TOP,
             "moe_route: bad sizes M=%d W=%d experts=%d top=%d (up to %d experts, top up to %d)", M, W, E, top, MOE_MAX_EXPERTS,
             MOE_MAX_TOP);
  TI_REQUIRE(score_kind == MOE_SIGMOID || score_kind == MOE_SOFTMAX, "moe_route: unknown score kind %d", score_kind);
  if (M == 0) return 0;
  const int piece = dtype == TI_F32 ? 4 : 8;
  const bool vec = W % piece == 0 && ((uintptr_t)h & 15) == 0;
#define MOE_ROUTE(T, V) moe_route_kernel<T, V><<<M, 256, 0, stream>>>((const T*)h, router, ids, wts, W, E, top, score_kind, renormalize)
  if (dtype == TI_F32) {
    if (vec) MOE_ROUTE(float, true);
    else MOE_ROUTE(float, false);
  } else if (dtype == TI_BF16) {
    if (vec) MOE_ROUTE(bf16_t, true);
    else MOE_ROUTE(bf16_t, false);
  } else {
    TI_REQUIRE(false, "moe_route: unknown dtype %d", dtype);
  }
#undef MOE_ROUTE
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ the experts, an output a wavefront
// up [E][F][W], down [E][W][F] in T.  Two kernels: act[(m, k)][f] = relu(up[e_k][f] . (s_k h[m]))^2 rounded to T, for every
// token m and chosen expert k; then y[m][c] = sum_k down[e_k][c] . act[(m, k)], k ascending.  A wavefront owns ROWS outputs;
// its lanes share a row of the weight in pieces of 16 bytes (lane l the pieces l, l + 64, ... in ascending order, then a
// butterfly): the order of every sum is fixed, whatever else the step holds.
#define MOE_ROWS 4      // outputs a wavefront
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_up_rows_kernel(const T* __restrict__ h, const int* __restrict__ ids, const float* __restrict__ wts, const T* __restrict__ up,
                   T* __restrict__ act, int W, int F, int top, int scale_input) {
  extern __shared__ float hs[];      // [W] the expert's input
  const int pair = blockIdx.x, m = pair / top;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = ids[pair];
  const float s = wts[pair];
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ld<T>(h + (size_t)m * W + c);
    float r = scale_input ? v * s : v;
    if (sizeof(T) == 2) r = bf2f(f2bf(r));
    hs[c] = r;
  }
  __syncthreads();
  const int f0 = (blockIdx.y * 4 + wave) * MOE_ROWS;
  const T* wu = up + (size_t)e * F * W;
#pragma unroll
  for (int r = 0; r < MOE_ROWS; ++r) {
    const int f = f0 + r;
    if (f >= F) break;
    const float z = wave_dot<T, VEC>([&](int c) { return hs[c]; }, wu + (size_t)f * W, W, lane);
    if (lane == 0) {
      float a = fmaxf(z, 0.f);
      st<T>(act + (size_t)pair * F + f, a * a);
    }
  }
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_down_rows_kernel(const T* __restrict__ act, const int* __restrict__ ids, const float* __restrict__ wts, const T* __restrict__ down,
                     float* __restrict__ y, int W, int F, int top, int scale_input) {
  const int m = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int c0 = (blockIdx.y * 4 + wave) * MOE_ROWS;
#pragma unroll
  for (int r = 0; r < MOE_ROWS; ++r) {
    const int c = c0 + r;
    if (c >= W) break;
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int pair = m * top + k;
      const T* a = act + (size_t)pair * F;
      const T* wd = down + ((size_t)ids[pair] * W + c) * F;
      float z = wave_dot<T, VEC>([&](int f) { return ld<T>(a + f); }, wd, F, lane);
      if (!scale_input) z *= wts[pair];
      acc = k == 0 ? z : acc + z;
    }
    if (lane == 0) y[(size_t)m * W + c] = acc;
  }
}

// act: scratch in the dtype of h, [M top][F]
extern "C" int ti_moe_experts_rows(int dtype, const void* h, const int* ids, const float* wts, const void* up, const void* down,
                                   void* act, float* y, int M, int W, int F, int top, int scale_input, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && W > 0 && F > 0 && top > 0, "moe_experts: bad sizes M=%d W=%d F=%d top=%d", M, W, F, top);
  TI_REQUIRE((size_t)W * 4 <= 64 * 1024, "moe_experts: a width of %d does not fit the workgroup's 64 KB", W);
  if (M == 0) return 0;
  const size_t lds = (size_t)W * 4;
  const dim3 up_grid(M * top, (F + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS)), down_grid(M, (W + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS));
  TI_REQUIRE(up_grid.y <= 65535 && down_grid.y <= 65535, "moe_experts: sizes W=%d F=%d are too large", W, F);
  const size_t es = dtype == TI_F32 ? 4 : 2;
  const int piece = (int)(16 / es);
  const bool vec = W % piece == 0 && F % piece == 0 && (((uintptr_t)up | (uintptr_t)down | (uintptr_t)act) & 15) == 0;
#define MOE_LAUNCH(T, V)                                                                                                              do {                                                                                                                                  moe_up_rows_kernel<T, V><<<up_grid, 256, lds, stream>>>((const T*)h, ids, wts, (const T*)up, (T*)act, W, F, top, scale_input);      moe_down_rows_kernel<T, V><<<down_grid, 256, 0, stream>>>((const T*)act, ids, wts, (const T*)down, y, W, F, top, scale_input);    } while (0)
  if (dtype == TI_F32) {
    if (vec) MOE_LAUNCH(float, true);
    else MOE_LAUNCH(float, false);
  } else if (dtype == TI_BF16) {
    if (vec) MOE_LAUNCH(bf16_t, true);
    else MOE_LAUNCH(bf16_t, false);
  } else {
    TI_REQUIRE(false, "moe_experts: unknown dtype %d", dtype);
  }
#undef MOE_LAUNCH
  TI_LAUNCH_CHECK();
  return 0;
}
