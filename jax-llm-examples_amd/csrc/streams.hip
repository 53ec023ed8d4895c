// Several residual streams per token, and the embedding with a sinusoidal position vector.
//
// streams_mix_norm: xs is float32 [N][S][D].  A pending branch output y (a plain tensor or the not yet formed sum
// of a token's expert outputs, see rows.h) is worked in first, all streams at once from the old ones:
//   X_t <- sum_s mix[s][t] X_s + outw[t] y          (the sum over s in order, float32)
// then u = sum_s inw[s] X_s (inw null: the plain sum), and h = u / sqrt(mean(u^2) + eps) * w.
// One block per token; a thread takes four neighbouring elements at 4 (thread + 256 i) where the width is a multiple
// of 4 (16-byte loads and stores, a row up to 4,096 wide is read once), else the elements d = thread, thread + 256,
// ...  The kernels are compiled for up to 2, 4, 8 and 16 streams, so that the arrays over streams are registers
// and a model with few streams pays for few.  A token's result depends on its own row only, and which kernel runs
// and the order in which the sum of squares is formed depend on the width and the number of streams only.
#include "common.h"
#include "rows.h"

using namespace jle;

constexpr int kMaxStreams = 16;
constexpr int kStreamThreads = 256;
constexpr int kStreamRegs = 8;  // elements of u a thread keeps (rows up to 2048 wide are read once)

__device__ __forceinline__ f32x4_t fma4(float a, f32x4_t x, f32x4_t c) {
  return f32x4_t{fmaf(a, x[0], c[0]), fmaf(a, x[1], c[1]), fmaf(a, x[2], c[2]), fmaf(a, x[3], c[3])};
}

constexpr int kStreamChunks = 4;  // chunks of four elements of u a thread keeps

template <typename DT, typename OT, int SMAX>
__global__ __launch_bounds__(kStreamThreads) void streams_mix_norm_vec_kernel(
    float* __restrict__ xs, Delta<DT> delta, const float* __restrict__ mix, const float* __restrict__ outw,
    const float* __restrict__ inw, const float* __restrict__ w, float eps, OT* __restrict__ out,
    float* __restrict__ out32, int S, int D, int do_norm) {
  __shared__ float red[kStreamThreads / 64];
  __shared__ float s_mix[SMAX * SMAX], s_out[SMAX], s_in[SMAX];
  const size_t n = blockIdx.x;
  const bool update = delta.any();
  for (int i = threadIdx.x; i < S * S; i += kStreamThreads) s_mix[i] = update ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < S; i += kStreamThreads) {
    s_out[i] = update ? outw[i] : 0.f;
    s_in[i] = inw != nullptr ? inw[i] : 1.0f;
  }
  __syncthreads();
  float* row = xs + n * (size_t)S * D;
  DeltaRow<DT> dr = {nullptr, nullptr, false, true};
  if (update) dr = delta_row(delta, n, D);
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  // four neighbouring elements of the row: the update of their streams, and u
  auto chunk = [&](int d) -> f32x4_t {
    f32x4_t x[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) x[s] = s < S ? load4<float>(row + (size_t)s * D + d) : zero;
    if (update) {
      const f32x4_t y = delta_row_at4<false, DT>(delta, dr, n, d, D);
      f32x4_t nx[SMAX];
#pragma unroll
      for (int t = 0; t < SMAX; ++t) {
        f32x4_t a = zero;
        if (t < S) {
#pragma unroll
          for (int s = 0; s < SMAX; ++s)
            if (s < S) a = fma4(s_mix[s * S + t], x[s], a);
          a = fma4(s_out[t], y, a);
          store4<float>(row + (size_t)t * D + d, a);
        }
        nx[t] = a;
      }
#pragma unroll
      for (int t = 0; t < SMAX; ++t) x[t] = nx[t];
    }
    f32x4_t u = zero;
#pragma unroll
    for (int s = 0; s < SMAX; ++s)
      if (s < S) u = fma4(s_in[s], x[s], u);
    return u;
  };
  f32x4_t keep[kStreamChunks];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kStreamChunks; ++i) {
    const int d = 4 * (threadIdx.x + kStreamThreads * i);
    keep[i] = zero;
    if (d < D) {
      keep[i] = chunk(d);
      ss = add_squares4(ss, keep[i]);
    }
  }
  for (int d = 4 * (threadIdx.x + kStreamThreads * kStreamChunks); d < D; d += 4 * kStreamThreads)
    ss = add_squares4(ss, chunk(d));
  if (!do_norm) return;
  const float tot = block_sum<kStreamThreads>(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)D + eps);
  auto put = [&](int d, f32x4_t u) {
    f32x4_t h = {u[0] * inv, u[1] * inv, u[2] * inv, u[3] * inv};
    if (w != nullptr) {
      const f32x4_t ww = load4<float>(w + d);
      h = f32x4_t{h[0] * ww[0], h[1] * ww[1], h[2] * ww[2], h[3] * ww[3]};
    }
    if (out != nullptr) store4<OT>(out + n * D + d, h);
    if (out32 != nullptr) store4<float>(out32 + n * D + d, h);
  };
#pragma unroll
  for (int i = 0; i < kStreamChunks; ++i) {
    const int d = 4 * (threadIdx.x + kStreamThreads * i);
    if (d < D) put(d, keep[i]);
  }
  for (int d = 4 * (threadIdx.x + kStreamThreads * kStreamChunks); d < D; d += 4 * kStreamThreads) {
    f32x4_t u = zero;  // (a wide row: formed again from what this thread wrote)
    for (int s = 0; s < S; ++s) u = fma4(s_in[s], load4<float>(row + (size_t)s * D + d), u);
    put(d, u);
  }
}

template <typename DT, typename OT, int SMAX>
__global__ __launch_bounds__(kStreamThreads) void streams_mix_norm_kernel(
    float* __restrict__ xs, Delta<DT> delta, const float* __restrict__ mix, const float* __restrict__ outw,
    const float* __restrict__ inw, const float* __restrict__ w, float eps, OT* __restrict__ out,
    float* __restrict__ out32, int S, int D, int do_norm) {
  __shared__ float red[kStreamThreads / 64];
  __shared__ float s_mix[SMAX * SMAX], s_out[SMAX], s_in[SMAX];
  const size_t n = blockIdx.x;
  const bool update = delta.any();
  for (int i = threadIdx.x; i < S * S; i += kStreamThreads) s_mix[i] = update ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < S; i += kStreamThreads) {
    s_out[i] = update ? outw[i] : 0.f;
    s_in[i] = inw != nullptr ? inw[i] : 1.0f;
  }
  __syncthreads();
  float* row = xs + n * (size_t)S * D;
  // one element of the row: the update of its streams, and u
  auto element = [&](int d) -> float {
    float x[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) x[s] = s < S ? row[(size_t)s * D + d] : 0.f;
    if (update) {
      const float y = delta.at(n, d, D);
      float nx[SMAX];
#pragma unroll
      for (int t = 0; t < SMAX; ++t) {
        float a = 0.f;
        if (t < S) {
#pragma unroll
          for (int s = 0; s < SMAX; ++s)
            if (s < S) a = fmaf(s_mix[s * S + t], x[s], a);
          a = fmaf(s_out[t], y, a);
          row[(size_t)t * D + d] = a;
        }
        nx[t] = a;
      }
#pragma unroll
      for (int t = 0; t < SMAX; ++t) x[t] = nx[t];
    }
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < SMAX; ++s)
      if (s < S) u = fmaf(s_in[s], x[s], u);
    return u;
  };
  float keep[kStreamRegs];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kStreamRegs; ++i) {
    const int d = threadIdx.x + kStreamThreads * i;
    keep[i] = 0.f;
    if (d < D) {
      keep[i] = element(d);
      ss = fmaf(keep[i], keep[i], ss);
    }
  }
  for (int d = threadIdx.x + kStreamThreads * kStreamRegs; d < D; d += kStreamThreads) {
    const float u = element(d);
    ss = fmaf(u, u, ss);
  }
  if (!do_norm) return;
  const float tot = block_sum<kStreamThreads>(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)D + eps);
  auto put = [&](int d, float u) {
    float h = u * inv;
    if (w != nullptr) h *= w[d];
    if (out != nullptr) Num<OT>::store(out + n * D + d, h);
    if (out32 != nullptr) out32[n * D + d] = h;
  };
#pragma unroll
  for (int i = 0; i < kStreamRegs; ++i) {
    const int d = threadIdx.x + kStreamThreads * i;
    if (d < D) put(d, keep[i]);
  }
  for (int d = threadIdx.x + kStreamThreads * kStreamRegs; d < D; d += kStreamThreads) {
    float u = 0.f;  // (a wide row: formed again from what this thread wrote)
    for (int s = 0; s < S; ++s) u = fmaf(s_in[s], row[(size_t)s * D + d], u);
    put(d, u);
  }
}

// delta: kind 0 none, 1 a plain tensor, 2 the sum of expert outputs (routed, inv, k, shared or null); delta_bf16 its
// element type.  out: the normed rows in the run dtype (out_bf16) or null; out32: the same in float32 or null.
JLE_API int jle_streams_mix_norm(float* xs, int kind, const void* plain, const void* routed, const int* inv, int k,
                                 const void* shared, int delta_bf16, const float* mix, const float* outw,
                                 const float* inw, const float* w, float eps, void* out, int out_bf16, float* out32,
                                 int N, int S, int D, int do_norm, hipStream_t s) {
  if (N <= 0) return 0;
  if (S < 1 || S > kMaxStreams || D < 1 || kind < 0 || kind > 2) return JLE_BAD_ARG;
  if (kind != 0 && (mix == nullptr || outw == nullptr)) return JLE_BAD_ARG;
  if (kind == 1 && plain == nullptr) return JLE_BAD_ARG;
  if (kind == 2 && (routed == nullptr || inv == nullptr || k < 1)) return JLE_BAD_ARG;
  const bool vec = D % 4 == 0;  // (rows of 4 k elements from 16-byte aligned arrays)
#define LAUNCH_S(DT, OT, SMAX)                                                                                     \
  do {                                                                                                             \
    if (vec)                                                                                                       \
      hipLaunchKernelGGL((streams_mix_norm_vec_kernel<DT, OT, SMAX>), dim3(N), dim3(kStreamThreads), 0, s, xs, dl, \
                         mix, outw, inw, w, eps, (OT*)out, out32, S, D, do_norm);                                  \
    else                                                                                                           \
      hipLaunchKernelGGL((streams_mix_norm_kernel<DT, OT, SMAX>), dim3(N), dim3(kStreamThreads), 0, s, xs, dl,     \
                         mix, outw, inw, w, eps, (OT*)out, out32, S, D, do_norm);                                  \
  } while (0)
#define LAUNCH(DT, OT)                                                                                             \
  do {                                                                                                             \
    Delta<DT> dl = {kind == 1 ? (const DT*)plain : nullptr, kind == 2 ? (const DT*)routed : nullptr, inv,          \
                    kind == 2 ? (const DT*)shared : nullptr, k};                                                   \
    if (S <= 2) LAUNCH_S(DT, OT, 2);                                                                               \
    else if (S <= 4) LAUNCH_S(DT, OT, 4);                                                                          \
    else if (S <= 8) LAUNCH_S(DT, OT, 8);                                                                          \
    else LAUNCH_S(DT, OT, 16);                                                                                     \
  } while (0)
  if (delta_bf16) {
    if (out_bf16) LAUNCH(bf16_t, bf16_t);
    else LAUNCH(bf16_t, float);
  } else {
    if (out_bf16) LAUNCH(float, bf16_t);
    else LAUNCH(float, float);
  }
#undef LAUNCH
#undef LAUNCH_S
  JLE_LAUNCH_CHECK();
  return 0;
}

// out[n][s][:] = table[tok[n]] * mult + wave(pos[n]) for every stream s: entry 2i of the wave is sin(pos * rates[i]),
// entry 2i + 1 the cosine; the angle is a float32 product, sine and cosine of it the accurate ones.
template <typename T>
__global__ void embed_sinusoid_kernel(const int* __restrict__ tok, const int* __restrict__ pos,
                                      const T* __restrict__ table, float mult, const float* __restrict__ rates,
                                      float* __restrict__ out, int S, int D) {
  const size_t n = blockIdx.x;
  const T* src = table + (size_t)tok[n] * D;
  const float p = (float)pos[n];
  float* dst = out + n * (size_t)S * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float ang = p * rates[d >> 1];
    const float v = Num<T>::load(src + d) * mult + ((d & 1) ? cosf(ang) : sinf(ang));
    for (int s = 0; s < S; ++s) dst[(size_t)s * D + d] = v;
  }
}

JLE_API int jle_embed_sinusoid(const int* tok, const int* pos, const void* table, int is_bf16, float mult,
                               const float* rates, float* out, int N, int S, int D, hipStream_t s) {
  if (N <= 0) return 0;
  if (S < 1 || D < 1) return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(embed_sinusoid_kernel<bf16_t>, dim3(N), dim3(256), 0, s, tok, pos, (const bf16_t*)table, mult,
                       rates, out, S, D);
  else
    hipLaunchKernelGGL(embed_sinusoid_kernel<float>, dim3(N), dim3(256), 0, s, tok, pos, (const float*)table, mult,
                       rates, out, S, D);
  JLE_LAUNCH_CHECK();
  return 0;
}
