// Kernels of layers that norm what a sublayer returns instead of what it reads: the RMS norm of a
// 32-bit row written (or added) into the 32-bit residual, and the rounding of the residual to the
// compute dtype for the products that read it directly.  All arithmetic is 32-bit.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

// x[m] (+)= y'[m] / sqrt(mean(y'[m]^2) + eps) * g, with y'[m] = y[m], or, with `gather`, the sum of the
// n_gather rows y[gather[m n_gather + k]] in ascending k (the rows a token's experts left; without a list: the rows
// y[m n_gather + k]).
// A workgroup per row; each thread owns the elements t, t + 256, ... in both passes, so y and x may be
// the same memory.  The sum of squares: per thread in ascending order, then block_sum (fixed order).
// RT: also `rounded` (RT) [M][H] = the new x rounded, for the product that reads the residual next.
// V4: four elements a thread at a time (H a multiple of 4, 16-byte aligned operands): fewer, wider loads in flight.
template <typename RT, bool V4>
__global__ void __launch_bounds__(256)
norm_residual_kernel(float* x, const float* y, const float* __restrict__ g,      // (y may be x)
                     const int* __restrict__ gather, int n_gather, int H, float eps, int accumulate, RT* __restrict__ rounded) {
  __shared__ float red[4];
  const int m = blockIdx.x;
  constexpr int N = V4 ? 4 : 1;
  // elements i .. i + N - 1 of the row to be normed
  auto value = [&](int i, float* v) {
    const int terms = (gather || n_gather > 1) ? n_gather : 1;
    for (int k = 0; k < terms; ++k) {
      const size_t r = gather ? (size_t)gather[(size_t)m * n_gather + k] : (size_t)m * terms + k;
      float t[N];
      if (V4) {
        const float4 a = *reinterpret_cast<const float4*>(y + r * H + i);
        t[0] = a.x;
        if (N > 1) { t[1] = a.y; t[2] = a.z; t[3] = a.w; }
      } else {
        t[0] = y[r * H + i];
      }
#pragma unroll
      for (int j = 0; j < N; ++j) v[j] = k == 0 ? t[j] : v[j] + t[j];
    }
  };
  float ss = 0.f;
  for (int i = threadIdx.x * N; i < H; i += 256 * N) {
    float v[N];
    value(i, v);
#pragma unroll
    for (int j = 0; j < N; ++j) ss = fmaf(v[j], v[j], ss);
  }
  ss = block_sum<256>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)H + eps);
  float* row = x + (size_t)m * H;
  for (int i = threadIdx.x * N; i < H; i += 256 * N) {
    float v[N];
    value(i, v);
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float add = v[j] * scale * g[i + j];
      const float now = accumulate ? row[i + j] + add : add;
      row[i + j] = now;
      if (rounded) st<RT>(rounded + (size_t)m * H + i + j, now);
    }
  }
}

extern "C" int ti_norm_residual(float* x, const float* y, const float* g, const int* gather, int n_gather, int M, int H,
                                float eps, int accumulate, void* rounded, int rounded_dtype, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0 && (!gather || n_gather > 0), "norm_residual: bad sizes M=%d H=%d gather=%d", M, H, n_gather);
  TI_REQUIRE(!rounded || rounded_dtype == TI_F32 || rounded_dtype == TI_BF16, "norm_residual: unknown dtype %d", rounded_dtype);
  if (M == 0) return 0;
  const bool v4 = H % 4 == 0 && (((uintptr_t)x | (uintptr_t)y | (uintptr_t)g) & 15) == 0;
  if (rounded && rounded_dtype == TI_BF16) {
    if (v4) norm_residual_kernel<bf16_t, true><<<M, 256, 0, stream>>>(x, y, g, gather, n_gather, H, eps, accumulate, (bf16_t*)rounded);
    else norm_residual_kernel<bf16_t, false><<<M, 256, 0, stream>>>(x, y, g, gather, n_gather, H, eps, accumulate, (bf16_t*)rounded);
  } else {
    if (v4) norm_residual_kernel<float, true><<<M, 256, 0, stream>>>(x, y, g, gather, n_gather, H, eps, accumulate, (float*)rounded);
    else norm_residual_kernel<float, false><<<M, 256, 0, stream>>>(x, y, g, gather, n_gather, H, eps, accumulate, (float*)rounded);
  }
  TI_LAUNCH_CHECK();
  return 0;
}

// out = x rounded to the compute dtype
template <typename T>
__global__ void round_rows_kernel(const float* __restrict__ x, T* __restrict__ out, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) st<T>(out + i, x[i]);
}
// eight elements a thread (n a multiple of 8, 16-byte aligned operands): the same bits
__global__ void __launch_bounds__(256) round_rows_wide_kernel(const float* __restrict__ x, bf16_t* __restrict__ out, long n8) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (long)gridDim.x * blockDim.x) {
    const float4 a = reinterpret_cast<const float4*>(x)[2 * i], b = reinterpret_cast<const float4*>(x)[2 * i + 1];
    reinterpret_cast<uint4*>(out)[i] = make_uint4(pack_bf16x2(a.x, a.y), pack_bf16x2(a.z, a.w), pack_bf16x2(b.x, b.y),
                                                  pack_bf16x2(b.z, b.w));
  }
}

extern "C" int ti_round_rows(int out_dtype, const float* x, void* out, long n, hipStream_t stream) {
  TI_REQUIRE(n >= 0, "round_rows: bad count %ld", n);
  if (n == 0) return 0;
  if (out_dtype == TI_BF16 && n % 8 == 0 && (((uintptr_t)x | (uintptr_t)out) & 15) == 0) {
    const long n8 = n / 8;
    const unsigned blocks = (unsigned)((n8 + 255) / 256 < 8192 ? (n8 + 255) / 256 : 8192);
    round_rows_wide_kernel<<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, n8);
    TI_LAUNCH_CHECK();
    return 0;
  }
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  if (out_dtype == TI_F32) round_rows_kernel<float><<<blocks, 256, 0, stream>>>(x, (float*)out, n);
  else if (out_dtype == TI_BF16) round_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, n);
  else TI_REQUIRE(false, "round_rows: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// x *= s
__global__ void scale_kernel(float* __restrict__ x, float s, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) x[i] *= s;
}

extern "C" int ti_scale(float* x, float s, long n, hipStream_t stream) {
  TI_REQUIRE(n >= 0, "scale: bad count %ld", n);
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  scale_kernel<<<blocks, 256, 0, stream>>>(x, s, n);
  TI_LAUNCH_CHECK();
  return 0;
}
