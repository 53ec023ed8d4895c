// Between an attention mixer's projected (and convolved) rows and the attention kernels, for mixers whose heads do
// not fit the fused preparation kernels: queries and keys of dk elements a head, values of dv, pages with heads of
// D >= max(dk, dv) elements (zeros behind the real ones), more key heads than value heads (a value head is written
// once for each of the `share` key heads that use it: two score maps over the same values), an RMS norm of q and k
// with or without weights before or behind the rotation, the rotation over adjacent or half-split pairs of the
// leading elements with a magnitude on sines and cosines.
//     rows [N, Hq dk + Hk dk + Hv dv]  ->  q_out [N, Hq, D],  pages [.., 2, Hk, ps, D] (values [D][ps])
// and the combination of two score maps' outputs into one head's:
//     d = a1 - lam a2;  d / sqrt(mean(d^2) + eps) * scale * sigmoid(gate)
// One wavefront per (token, head); a lane holds elements lane, lane + 64, ...  Everything in float32; the order of
// every sum depends on the sizes only.
#include "common.h"

using namespace jle;

namespace {

constexpr int kMaxPerLane = 8;  // heads of up to 512 elements

template <typename T>
struct HeadsArgs {
  const T* rows;
  const int* positions;
  const int* slot_mapping;
  const float* inv_freq;  // [rotary_dim / 2] or null
  const float* wq;        // [dk] or null
  const float* wk;
  T* q_out;
  T* kv_cache;  // or null
  float magnitude, norm_eps;  // norm_eps < 0: no norm
  int rotary_dim, half_pairs, norm_first, Hq, Hk, Hv, dk, dv, D, ps;
};

template <typename T>
__global__ __launch_bounds__(64) void heads_prepare_kernel(HeadsArgs<T> a) {
  __shared__ float sh[kMaxPerLane * 64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool is_q = h < a.Hq, is_v = h >= a.Hq + a.Hk;
  if (!is_q && a.kv_cache == nullptr) return;
  const int C = (a.Hq + a.Hk) * a.dk + a.Hv * a.dv;
  const int dim = is_v ? a.dv : a.dk;
  const int c0 = is_v ? (a.Hq + a.Hk) * a.dk + (h - a.Hq - a.Hk) * a.dv : h * a.dk;
  const T* src = a.rows + (size_t)n * C + c0;
  float x[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int e = lane + 64 * i;
    x[i] = e < dim ? Num<T>::load(src + e) : 0.f;
  }
  if (!is_v) {
    const float* w = is_q ? a.wq : a.wk;
    if (a.norm_eps >= 0.f && a.norm_first) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) ss = __builtin_fmaf(x[i], x[i], ss);
      const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + a.norm_eps);
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int e = lane + 64 * i;
        if (e < dim) x[i] = w != nullptr ? x[i] * inv * w[e] : x[i] * inv;
      }
    }
    if (a.inv_freq != nullptr && a.rotary_dim > 0) {
      const int rd = a.rotary_dim, hr = rd / 2;
      const float pos = (float)a.positions[n];
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) sh[lane + 64 * i] = x[i];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int e = lane + 64 * i;
        if (e < rd) {
          const bool first = a.half_pairs ? e < hr : (e & 1) == 0;
          const int j = a.half_pairs ? (first ? e : e - hr) : e >> 1;
          const int partner = a.half_pairs ? (first ? e + hr : e - hr) : e ^ 1;
          float sn, cs;
          sincosf(pos * a.inv_freq[j], &sn, &cs);
          sn *= a.magnitude;
          cs *= a.magnitude;
          const float other = sh[partner];
          x[i] = first ? x[i] * cs - other * sn : x[i] * cs + other * sn;
        }
      }
    }
    if (a.norm_eps >= 0.f && !a.norm_first) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) ss = __builtin_fmaf(x[i], x[i], ss);
      const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + a.norm_eps);
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int e = lane + 64 * i;
        if (e < dim) x[i] = w != nullptr ? x[i] * inv * w[e] : x[i] * inv;
      }
    }
  }
  if (is_q) {
    T* dst = a.q_out + ((size_t)n * a.Hq + h) * a.D;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int e = lane + 64 * i;
      if (e < a.D) Num<T>::store(dst + e, x[i]);  // (zeros behind the real elements)
    }
    return;
  }
  const int slot = a.slot_mapping[n];
  const size_t page = (size_t)(slot / a.ps);
  const int off = slot % a.ps;
  const size_t plane = (size_t)a.Hk * a.ps * a.D;
  if (!is_v) {
    T* dst = a.kv_cache + page * 2 * plane + ((size_t)(h - a.Hq) * a.ps + off) * a.D;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int e = lane + 64 * i;
      if (e < a.D) Num<T>::store(dst + e, x[i]);
    }
    return;
  }
  const int share = a.Hk / a.Hv, vh = h - a.Hq - a.Hk;
  for (int s = 0; s < share; ++s) {
    T* dst = a.kv_cache + page * 2 * plane + plane + (size_t)(vh * share + s) * a.ps * a.D + off;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int e = lane + 64 * i;
      if (e < a.D) Num<T>::store(dst + (size_t)e * a.ps, x[i]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(const T* __restrict__ o, const T* __restrict__ gate,
                                                          T* __restrict__ out, float lam, float out_scale, float eps,
                                                          int H, int G, int D, int dv) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = H / G, g = h / r, j = h - g * r;
  const T* a1 = o + ((size_t)n * 2 * H + (size_t)(g * 2 + 0) * r + j) * D;
  const T* a2 = o + ((size_t)n * 2 * H + (size_t)(g * 2 + 1) * r + j) * D;
  float d[kMaxPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int e = lane + 64 * i;
    d[i] = e < dv ? Num<T>::load(a1 + e) - lam * Num<T>::load(a2 + e) : 0.f;
    ss = __builtin_fmaf(d[i], d[i], ss);
  }
  const float inv = out_scale / sqrtf(wave_sum(ss) / (float)dv + eps);
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int e = lane + 64 * i;
    if (e < dv) {
      float v = d[i] * inv;
      const size_t at = ((size_t)n * H + h) * dv + e;
      if (gate != nullptr) v *= 1.0f / (1.0f + expf(-Num<T>::load(gate + at)));
      Num<T>::store(out + at, v);
    }
  }
}

}  // namespace

JLE_API int jle_heads_prepare(const void* rows, const int* positions, const int* slot_mapping, const float* inv_freq,
                              int rotary_dim, int half_pairs, float magnitude, float norm_eps, int norm_first,
                              const float* wq, const float* wk, void* q_out, void* kv_cache, int is_bf16, int N, int Hq,
                              int Hk, int Hv, int dk, int dv, int D, int ps, hipStream_t s) {
  if (N <= 0) return 0;
  if (rows == nullptr || q_out == nullptr || Hq <= 0 || Hk <= 0 || Hv <= 0 || Hk % Hv || dk <= 0 || dv <= 0 ||
      D < dk || D < dv || D > 64 * kMaxPerLane || Hq + Hk + Hv > 65535 || ps <= 0)
    return JLE_BAD_ARG;
  if (rotary_dim < 0 || rotary_dim % 2 || rotary_dim > dk || (rotary_dim > 0 && (inv_freq == nullptr || positions == nullptr)))
    return JLE_BAD_ARG;
  if (kv_cache != nullptr && slot_mapping == nullptr) return JLE_BAD_ARG;
  const dim3 grid(N, Hq + Hk + Hv);
  if (is_bf16) {
    HeadsArgs<bf16_t> a{(const bf16_t*)rows, positions, slot_mapping, inv_freq, wq, wk, (bf16_t*)q_out, (bf16_t*)kv_cache,
                        magnitude, norm_eps, rotary_dim, half_pairs, norm_first, Hq, Hk, Hv, dk, dv, D, ps};
    hipLaunchKernelGGL(heads_prepare_kernel<bf16_t>, grid, dim3(64), 0, s, a);
  } else {
    HeadsArgs<float> a{(const float*)rows, positions, slot_mapping, inv_freq, wq, wk, (float*)q_out, (float*)kv_cache,
                       magnitude, norm_eps, rotary_dim, half_pairs, norm_first, Hq, Hk, Hv, dk, dv, D, ps};
    hipLaunchKernelGGL(heads_prepare_kernel<float>, grid, dim3(64), 0, s, a);
  }
  JLE_LAUNCH_CHECK();
  return 0;
}

// o [N, 2 H, D] in the order [kv head][map][query head of the group]; gate [N, H dv] or null; out [N, H dv].
JLE_API int jle_diff_combine(const void* o, const void* gate, void* out, float lam, float out_scale, float eps,
                             int is_bf16, int N, int H, int G, int D, int dv, hipStream_t s) {
  if (N <= 0) return 0;
  if (o == nullptr || out == nullptr || H <= 0 || G <= 0 || H % G || dv <= 0 || D < dv || dv > 64 * kMaxPerLane ||
      H > 65535)
    return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(diff_combine_kernel<bf16_t>, dim3(N, H), dim3(64), 0, s, (const bf16_t*)o, (const bf16_t*)gate,
                       (bf16_t*)out, lam, out_scale, eps, H, G, D, dv);
  else
    hipLaunchKernelGGL(diff_combine_kernel<float>, dim3(N, H), dim3(64), 0, s, (const float*)o, (const float*)gate,
                       (float*)out, lam, out_scale, eps, H, G, D, dv);
  JLE_LAUNCH_CHECK();
  return 0;
}
