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

constexpr int kPiecesInRegisters = 8;

// where the pieces of row n's expert sum lie, looked up once per row (up to kPiecesInRegisters of them)
struct Pieces {
  size_t at[kPiecesInRegisters];
  int count;  // -1: a is a plain row (or has more pieces than are kept here: looked up per element)
};

__device__ __forceinline__ Pieces pieces_of(const ScaledArgs& p, size_t n) {
  Pieces r;
  r.count = (p.a_inv != nullptr && p.a_k <= kPiecesInRegisters) ? p.a_k : -1;
#pragma unroll
  for (int j = 0; j < kPiecesInRegisters; ++j)
    r.at[j] = j < r.count ? (size_t)p.a_inv[n * p.a_k + j] * p.D : 0;
  return r;
}

__device__ __forceinline__ float updated(const ScaledArgs& p, const Pieces& pc, size_t base, int d) {
  float v = p.x[base + d];
  if (p.a != nullptr) {
    float ta;
    if (pc.count >= 0) {
      ta = 0.f;
#pragma unroll
      for (int j = 0; j < kPiecesInRegisters; ++j)
        if (j < pc.count) ta += term(p.a, p.a_bf16, pc.at[j] + d);
    } else if (p.a_inv != nullptr) {
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

// AT, BT: the terms' types (no choice by a flag inside the loops: every array's loads of a row stand together, under
// one test that is the same for the whole launch, so that they are all on their way before the first is used)
template <int THREADS, int EPT, typename AT, typename BT>
__global__ __launch_bounds__(THREADS) void scaled_add_norm_kernel(ScaledArgs p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  const AT* __restrict__ pa = (const AT*)p.a;
  const BT* __restrict__ pb = (const BT*)p.b;
  float v[EPT], t[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    v[i] = d < D ? p.x[base + d] : 0.f;
    t[i] = 0.f;
  }
  if (pa != nullptr) {
    if (p.a_inv != nullptr) {  // (the pieces of an expert sum, added up in their order from zero)
      const int* rows = p.a_inv + (size_t)blockIdx.x * p.a_k;
      for (int j = 0; j < p.a_k; ++j) {
        const size_t at = (size_t)rows[j] * D;
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
          const int d = threadIdx.x + THREADS * i;
          if (d < D) t[i] += Num<AT>::load(pa + at + d);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        const int d = threadIdx.x + THREADS * i;
        if (d < D) t[i] = Num<AT>::load(pa + base + d);
      }
    }
#pragma unroll
    for (int i = 0; i < EPT; ++i) t[i] *= p.fa;
    if (pb != nullptr) {
      float u[EPT];
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        const int d = threadIdx.x + THREADS * i;
        u[i] = d < D ? Num<BT>::load(pb + base + d) : 0.f;
      }
#pragma unroll
      for (int i = 0; i < EPT; ++i) t[i] = __builtin_fmaf(p.fb, u[i], t[i]);
    }
    if (p.vec != nullptr) {
      float u[EPT];
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        const int d = threadIdx.x + THREADS * i;
        u[i] = d < D ? p.vec[d] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < EPT; ++i) v[i] = __builtin_fmaf(u[i], t[i], v[i]);
    } else {
#pragma unroll
      for (int i = 0; i < EPT; ++i) v[i] += t[i];
    }
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int d = threadIdx.x + THREADS * i;
      if (d < D) p.x[base + d] = v[i];
    }
  }
  if (p.h == nullptr) return;
  float w[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {  // (asked for before the statistics are there)
    const int d = threadIdx.x + THREADS * i;
    w[i] = (p.w != nullptr && d < D) ? p.w[d] : 1.f;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < EPT; ++i) ss = __builtin_fmaf(v[i], v[i], ss);
  const float inv = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)D + p.eps);
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    if (d < D) {
      const float h = v[i] * inv;
      put(p, base + d, p.w != nullptr ? h * w[i] : h);
    }
  }
}

template <int THREADS>
__global__ __launch_bounds__(THREADS) void scaled_add_norm_wide_kernel(ScaledArgs p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  float ss = 0.f;
  const Pieces pc = pieces_of(p, blockIdx.x);
  for (int d = threadIdx.x; d < D; d += THREADS) {
    const float v = updated(p, pc, base, d);
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
  // (which kernel: by the width and the terms' types alone, never by the step's size)
#define JLE_SCALED(AT, BT)                                                                                \
  do {                                                                                                    \
    if (D <= 256) hipLaunchKernelGGL((scaled_add_norm_kernel<64, 4, AT, BT>), dim3(N), dim3(64), 0, s, p);  \
    else if (D <= 1024) hipLaunchKernelGGL((scaled_add_norm_kernel<256, 4, AT, BT>), dim3(N), dim3(256), 0, s, p); \
    else if (D <= 2048) hipLaunchKernelGGL((scaled_add_norm_kernel<256, 8, AT, BT>), dim3(N), dim3(256), 0, s, p); \
    else if (D <= 4096) hipLaunchKernelGGL((scaled_add_norm_kernel<256, 16, AT, BT>), dim3(N), dim3(256), 0, s, p); \
    else if (D <= 8192) hipLaunchKernelGGL((scaled_add_norm_kernel<512, 16, AT, BT>), dim3(N), dim3(512), 0, s, p); \
    else hipLaunchKernelGGL((scaled_add_norm_wide_kernel<512>), dim3(N), dim3(512), 0, s, p);             \
  } while (0)
  const bool a16 = a_kind == 1, b16 = b_kind == 1;
  if (a16 && (b16 || b == nullptr)) JLE_SCALED(bf16_t, bf16_t);
  else if (a16) JLE_SCALED(bf16_t, float);
  else if (b16) JLE_SCALED(float, bf16_t);
  else JLE_SCALED(float, float);
#undef JLE_SCALED
  JLE_LAUNCH_CHECK();
  return 0;
}
