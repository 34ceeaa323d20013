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

// ------------------------------------------------------------ router
// A workgroup per token.  Logits: wavefront w takes experts w, w + 4, ...; lanes share a row of the router
// (lane l the entries l, l + 64, ... in ascending order, then a butterfly).  Choice: the first wavefront
// holds the scores (lane l the experts l, l + 64, ...) and takes the largest `top` times.
template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ h, const float* __restrict__ router, int* __restrict__ ids, float* __restrict__ wts,
                 int W, int E, int top, int score_kind, int renormalize) {
  __shared__ float s_score[MOE_MAX_EXPERTS];
  __shared__ float red[4];
  const int m = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* row = h + (size_t)m * W;
  for (int e = wave; e < E; e += 4) {
    const float* r = router + (size_t)e * W;
    float z = 0.f;
    for (int c = lane; c < W; c += 64) z = fmaf(ld<T>(row + c), r[c], z);
    z = group_sum<64>(z);
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
  if (dtype == TI_F32) moe_route_kernel<float><<<M, 256, 0, stream>>>((const float*)h, router, ids, wts, W, E, top, score_kind, renormalize);
  else if (dtype == TI_BF16) moe_route_kernel<bf16_t><<<M, 256, 0, stream>>>((const bf16_t*)h, router, ids, wts, W, E, top, score_kind, renormalize);
  else TI_REQUIRE(false, "moe_route: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ the experts, a workgroup per token
// up [E][F][W], down [E][W][F] in T; y f32 [M][W].  A wavefront owns an output and its lanes share the row of the
// weight; the same wavefront owns the same output for every chosen expert, so the sum over them is in order.
template <typename T>
__global__ void __launch_bounds__(256)
moe_experts_rows_kernel(const T* __restrict__ h, const int* __restrict__ ids, const float* __restrict__ wts,
                        const T* __restrict__ up, const T* __restrict__ down, float* __restrict__ y, int W, int F, int top,
                        int scale_input) {
  extern __shared__ float lds[];
  float* hs = lds;          // [W] the expert's input
  float* act = lds + W;     // [F] its activated rows
  const int m = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int k = 0; k < top; ++k) {
    const int e = ids[(size_t)m * top + k];
    const float s = wts[(size_t)m * top + k];
    __syncthreads();
    for (int c = threadIdx.x; c < W; c += 256) {
      const float v = ld<T>(h + (size_t)m * W + c);
      float r = scale_input ? v * s : v;
      if (sizeof(T) == 2) r = bf2f(f2bf(r));
      hs[c] = r;
    }
    __syncthreads();
    const T* wu = up + (size_t)e * F * W;
    for (int f = wave; f < F; f += 4) {
      const T* r = wu + (size_t)f * W;
      float z = 0.f;
      for (int c = lane; c < W; c += 64) z = fmaf(hs[c], ld<T>(r + c), z);
      z = group_sum<64>(z);
      if (lane == 0) {
        float a = fmaxf(z, 0.f);
        a *= a;
        if (sizeof(T) == 2) a = bf2f(f2bf(a));
        act[f] = a;
      }
    }
    __syncthreads();
    const T* wd = down + (size_t)e * W * F;
    for (int c = wave; c < W; c += 4) {
      const T* r = wd + (size_t)c * F;
      float z = 0.f;
      for (int f = lane; f < F; f += 64) z = fmaf(act[f], ld<T>(r + f), z);
      z = group_sum<64>(z);
      if (!scale_input) z *= s;
      if (lane == 0) y[(size_t)m * W + c] = k == 0 ? z : y[(size_t)m * W + c] + z;
    }
  }
}

extern "C" int ti_moe_experts_rows(int dtype, const void* h, const int* ids, const float* wts, const void* up, const void* down,
                                   float* y, int M, int W, int F, int top, int scale_input, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && W > 0 && F > 0 && top > 0, "moe_experts: bad sizes M=%d W=%d F=%d top=%d", M, W, F, top);
  const size_t lds = (size_t)(W + F) * 4;
  TI_REQUIRE(lds <= 64 * 1024, "moe_experts: a width of %d beside an expert size of %d does not fit the workgroup's 64 KB", W, F);
  if (M == 0) return 0;
  if (dtype == TI_F32)
    moe_experts_rows_kernel<float><<<M, 256, lds, stream>>>((const float*)h, ids, wts, (const float*)up, (const float*)down, y, W, F,
                                                            top, scale_input);
  else if (dtype == TI_BF16)
    moe_experts_rows_kernel<bf16_t><<<M, 256, lds, stream>>>((const bf16_t*)h, ids, wts, (const bf16_t*)up, (const bf16_t*)down, y,
                                                             W, F, top, scale_input);
  else
    TI_REQUIRE(false, "moe_experts: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}
