// A branch output that carries factors: the residual takes
//     x += vec * (fa * a + fb * b)          a, b: rows in bfloat16 or float32 (b optional), vec: float32 [D] (optional)
// (a may be the not yet formed sum of a token's expert outputs, a[n] = sum_j routed[inv[n * k + j]], added up in the
// order of j from zero)
// and the same launch forms the next norm's rows, h = x / sqrt(mean(x^2) + eps) * w, in the run dtype (and in float32
// for a router).  It is what a layer leaves pending whose branches have a multiplier and a learned scale per
// channel, and whose mixer may be two mixers side by side with a weight each.  One block per row, the row in
// registers (wider rows are read again); every sum in an order that depends on the width alone.
#include "common.h"

using namespace jle;

namespace {

struct ScaledArgs {
  float* x;        // [N, D] residual, updated in place
  const void* a;   // [N, D] or null
  const void* b;   // [N, D] or null
  const float* vec;
  const float* w;  // norm weight or null
  void* h;         // [N, D] run dtype or null (the sum only)
  float* h32;      // [N, D] or null
  float fa, fb, eps;
  int a_bf16, b_bf16, h_bf16, D;
  const int* a_inv;  // a is [M, D], the rows of expert outputs: token n's are inv[n * k + j], j < k; null: a is [N, D]
  int a_k;
};

__device__ __forceinline__ float term(const void* p, int is_bf16, size_t i) {
  return is_bf16 ? bf16_to_float(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

__device__ __forceinline__ float updated(const ScaledArgs& p, size_t base, int d) {
  float v = p.x[base + d];
  if (p.a != nullptr) {
    float ta;
    if (p.a_inv != nullptr) {
      ta = 0.f;
      const int* rows = p.a_inv + (size_t)blockIdx.x * p.a_k;
      for (int j = 0; j < p.a_k; ++j) ta += term(p.a, p.a_bf16, (size_t)rows[j] * p.D + d);
    } else {
      ta = term(p.a, p.a_bf16, base + d);
    }
    float t = p.fa * ta;
    if (p.b != nullptr) t = __builtin_fmaf(p.fb, term(p.b, p.b_bf16, base + d), t);
    v = p.vec != nullptr ? __builtin_fmaf(p.vec[d], t, v) : v + t;
  }
  return v;
}

__device__ __forceinline__ void put(const ScaledArgs& p, size_t i, float h) {
  if (p.h_bf16) ((bf16_t*)p.h)[i] = float_to_bf16(h);
  else ((float*)p.h)[i] = h;
  if (p.h32 != nullptr) p.h32[i] = h;
}

template <int THREADS, int EPT>
__global__ __launch_bounds__(THREADS) void scaled_add_norm_kernel(ScaledArgs p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  float v[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    v[i] = d < D ? updated(p, base, d) : 0.f;
  }
  if (p.a != nullptr) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int d = threadIdx.x + THREADS * i;
      if (d < D) p.x[base + d] = v[i];
    }
  }
  if (p.h == nullptr) return;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < EPT; ++i) ss = __builtin_fmaf(v[i], v[i], ss);
  const float inv = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)D + p.eps);
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    if (d < D) {
      const float h = v[i] * inv;
      put(p, base + d, p.w != nullptr ? h * p.w[d] : h);
    }
  }
}

template <int THREADS>
__global__ __launch_bounds__(THREADS) void scaled_add_norm_wide_kernel(ScaledArgs p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += THREADS) {
    const float v = updated(p, base, d);
    p.x[base + d] = v;
    ss = __builtin_fmaf(v, v, ss);
  }
  if (p.h == nullptr) return;
  const float inv = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)D + p.eps);
  for (int d = threadIdx.x; d < D; d += THREADS) {
    const float h = p.x[base + d] * inv;  // (this thread's own store)
    put(p, base + d, p.w != nullptr ? h * p.w[d] : h);
  }
}

}  // namespace

// a_kind / b_kind: 0 none, 1 bfloat16, 2 float32.  h null: the sum only.  b needs a.  a_inv: a is a sum of expert
// outputs in pieces (see above), a_k of them a token.
JLE_API int jle_scaled_add_norm(float* x, const void* a, int a_kind, float fa, const void* b, int b_kind, float fb,
                                const float* vec, const float* w, float eps, void* h, int h_bf16, float* h32, int N,
                                int D, const int* a_inv, int a_k, hipStream_t s) {
  if (N <= 0) return 0;
  if (D <= 0 || x == nullptr || (a == nullptr) != (a_kind == 0) || (b == nullptr) != (b_kind == 0) ||
      (b != nullptr && a == nullptr) || (h == nullptr && h32 != nullptr) || (a_inv != nullptr && (a == nullptr || a_k < 1)))
    return JLE_BAD_ARG;
  ScaledArgs p{x, a, b, vec, w, h, h32, fa, fb, eps, a_kind == 1, b_kind == 1, h_bf16, D, a_inv, a_k};
  // (which kernel: by the width alone, never by the step's size)
  if (D <= 256)
    hipLaunchKernelGGL((scaled_add_norm_kernel<64, 4>), dim3(N), dim3(64), 0, s, p);
  else if (D <= 1024)
    hipLaunchKernelGGL((scaled_add_norm_kernel<256, 4>), dim3(N), dim3(256), 0, s, p);
  else if (D <= 4096)
    hipLaunchKernelGGL((scaled_add_norm_kernel<256, 16>), dim3(N), dim3(256), 0, s, p);
  else if (D <= 8192)
    hipLaunchKernelGGL((scaled_add_norm_kernel<512, 16>), dim3(N), dim3(512), 0, s, p);
  else
    hipLaunchKernelGGL((scaled_add_norm_wide_kernel<512>), dim3(N), dim3(512), 0, s, p);
  JLE_LAUNCH_CHECK();
  return 0;
}
