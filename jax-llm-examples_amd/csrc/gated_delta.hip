// The gated delta rule: a matrix memory S (dk x dv, float32) per head and request, written and read token by token,
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with q, k unit vectors per kv head (x / sqrt(sum(x^2) + floor), q times dk^(-1/2)), beta = sigmoid(b),
// g = exp(-exp(A) softplus(a + dt)).  Three kernels:
//   gdr_prepare_kernel   the unit vectors (float32), beta and the decay of every token of the step
//   gdr_scan_kernel      the recurrence: a column of S depends on nothing but itself, k, q, v of its own place, beta
//                        and g, so a wavefront takes 64 / KS columns of one head, KS lanes share a column (each
//                        holds R consecutive rows of it in registers), and the two dot products are finished with
//                        KS - 1 lane swaps; the next token's rows are asked for before this token's are used
//   gdr_out_kernel       o / sqrt(mean(o^2) + eps) * w * silu(gate), rounded to the run dtype
// The memory lies [slot][half][H][dk][dv]; a step reads the half `phase` and writes the other.  Every sum is formed
// in an order that depends on the sizes alone, token after token: cutting a sequence into steps changes no bit.
#include "common.h"

using namespace jle;

namespace {

template <typename T>
__global__ __launch_bounds__(64) void gdr_prepare_kernel(const T* __restrict__ rows, const float* __restrict__ gates,
                                                         const float* __restrict__ a_log,
                                                         const float* __restrict__ dt_bias, float* __restrict__ qn,
                                                         float* __restrict__ kn, float* __restrict__ beta,
                                                         float* __restrict__ decay, float floor, int H, int G, int dk,
                                                         int dv) {
  const int n = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int C = 2 * G * dk + H * dv;
  if (g == G) {  // the write strengths and decays of the token's heads
    for (int h = lane; h < H; h += 64) {
      const float b = gates[(size_t)n * 2 * H + h], a = gates[(size_t)n * 2 * H + H + h] + dt_bias[h];
      beta[(size_t)n * H + h] = 1.0f / (1.0f + expf(-b));
      const float sp = a > 20.f ? a : log1pf(expf(a));
      decay[(size_t)n * H + h] = expf(-expf(a_log[h]) * sp);
    }
    return;
  }
  for (int which = 0; which < 2; ++which) {
    const T* src = rows + (size_t)n * C + (size_t)(which * G + g) * dk;
    float* dst = (which == 0 ? qn : kn) + ((size_t)n * G + g) * dk;
    float ss = 0.f;
    for (int e = lane; e < dk; e += 64) {
      const float x = Num<T>::load(src + e);
      ss = __builtin_fmaf(x, x, ss);
    }
    float inv = 1.0f / sqrtf(wave_sum(ss) + floor);
    if (which == 0) inv *= 1.0f / sqrtf((float)dk);
    for (int e = lane; e < dk; e += 64) dst[e] = Num<T>::load(src + e) * inv;
  }
}

template <typename T, int R>
__global__ __launch_bounds__(64) void gdr_scan_kernel(const T* __restrict__ rows, const float* __restrict__ qn,
                                                      const float* __restrict__ kn, const float* __restrict__ beta,
                                                      const float* __restrict__ decay, float* __restrict__ state,
                                                      const int* __restrict__ cu_seqlens,
                                                      const int* __restrict__ state_slots,
                                                      const int* __restrict__ state_phase, float* __restrict__ o_raw,
                                                      int H, int G, int dk, int dv, int KS) {
  const int seg = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int cols = 64 / KS;
  const int ks = lane / cols, c = blockIdx.z * cols + (lane - ks * cols);
  const bool live = c < dv;
  const int g = h / (H / G);
  const int C = 2 * G * dk + H * dv;
  const int t0 = cu_seqlens[seg], t1 = cu_seqlens[seg + 1];
  const size_t slot = (size_t)state_slots[seg];
  const int phase = state_phase[seg];
  const float* s_old = state + ((slot * 2 + phase) * H + h) * (size_t)dk * dv;
  float* s_new = state + ((slot * 2 + (1 - phase)) * H + h) * (size_t)dk * dv;
  const int k0 = ks * R;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (live && k0 + i < dk) ? s_old[(size_t)(k0 + i) * dv + c] : 0.f;
  // this token's rows and the next one's, each in registers of its own (asked for a token ahead)
  float kc[R], qc[R], vc = 0.f, bc = 0.f, gc = 1.f;
  auto fetch = [&](int t, float (&k_)[R], float (&q_)[R], float& v_, float& b_, float& g_) {
    const float* kp = kn + ((size_t)t * G + g) * dk + k0;
    const float* qp = qn + ((size_t)t * G + g) * dk + k0;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      k_[i] = k0 + i < dk ? kp[i] : 0.f;
      q_[i] = k0 + i < dk ? qp[i] : 0.f;
    }
    v_ = live ? Num<T>::load(rows + (size_t)t * C + 2 * G * dk + (size_t)h * dv + c) : 0.f;
    b_ = beta[(size_t)t * H + h];
    g_ = decay[(size_t)t * H + h];
  };
  if (t0 < t1) fetch(t0, kc, qc, vc, bc, gc);
  for (int t = t0; t < t1; ++t) {
    float kx[R], qx[R], vx = 0.f, bx = 0.f, gx = 1.f;
    if (t + 1 < t1) {
      fetch(t + 1, kx, qx, vx, bx, gx);
    } else {
#pragma unroll
      for (int i = 0; i < R; ++i) kx[i] = qx[i] = 0.f;
    }
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      S[i] *= gc;
      dot = __builtin_fmaf(S[i], kc[i], dot);
    }
    for (int o = cols; o < 64; o <<= 1) dot += __shfl_xor(dot, o, 64);
    const float u = bc * (vc - dot);
    float out = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      S[i] = __builtin_fmaf(kc[i], u, S[i]);
      out = __builtin_fmaf(S[i], qc[i], out);
    }
    for (int o = cols; o < 64; o <<= 1) out += __shfl_xor(out, o, 64);
    if (live && ks == 0) o_raw[((size_t)t * H + h) * dv + c] = out;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      kc[i] = kx[i];
      qc[i] = qx[i];
    }
    vc = vx;
    bc = bx;
    gc = gx;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (k0 + i < dk) s_new[(size_t)(k0 + i) * dv + c] = S[i];
  }
}

template <typename T>
__global__ __launch_bounds__(64) void gdr_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate,
                                                     const float* __restrict__ w, T* __restrict__ out, float eps, int H,
                                                     int dv) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)n * H + h) * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += 64) {
    const float x = o_raw[base + e];
    ss = __builtin_fmaf(x, x, ss);
  }
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
  for (int e = lane; e < dv; e += 64) {
    const float z = Num<T>::load(gate + base + e);
    Num<T>::store(out + base + e, o_raw[base + e] * inv * w[e] * (z / (1.0f + expf(-z))));
  }
}

template <typename T>
int launch_gdr(const T* rows, const float* gates, const float* a_log, const float* dt_bias, const float* norm_w,
               const T* gate, float* state, const int* cu_seqlens, const int* state_slots, const int* state_phase,
               float* qn, float* kn, float* beta, float* decay, float* o_raw, T* out, int N, int R_, int H, int G, int dk,
               int dv, float eps, float floor, hipStream_t s) {
  hipLaunchKernelGGL(gdr_prepare_kernel<T>, dim3(N, G + 1), dim3(64), 0, s, rows, gates, a_log, dt_bias, qn, kn, beta,
                     decay, floor, H, G, dk, dv);
  JLE_LAUNCH_CHECK();
  // lanes a column: the fewest that leave a lane at most 16 rows of it (by the sizes alone)
  int KS = 1;
  while (KS < 64 && (dk + KS - 1) / KS > 16) KS <<= 1;
  const int per = (dk + KS - 1) / KS, cols = 64 / KS;
  const dim3 grid(R_, H, (dv + cols - 1) / cols);
#define JLE_SCAN(RR)                                                                                               \
  hipLaunchKernelGGL((gdr_scan_kernel<T, RR>), grid, dim3(64), 0, s, rows, qn, kn, beta, decay, state, cu_seqlens, \
                     state_slots, state_phase, o_raw, H, G, dk, dv, KS)
  if (per <= 4) JLE_SCAN(4);
  else if (per <= 8) JLE_SCAN(8);
  else if (per <= 16) JLE_SCAN(16);
  else JLE_SCAN(32);
#undef JLE_SCAN
  JLE_LAUNCH_CHECK();
  hipLaunchKernelGGL(gdr_out_kernel<T>, dim3(N, H), dim3(64), 0, s, o_raw, gate, norm_w, out, eps, H, dv);
  JLE_LAUNCH_CHECK();
  return 0;
}

}  // namespace

// rows [N, 2 G dk + H dv] (q | k | v behind convolution and activation) and gate [N, H dv] in the run dtype; gates
// float32 [N, 2 H] (write strengths, then decays, before their biases and squashing); state float32 [slots, 2, H, dk,
// dv]; qn, kn [N, G, dk], beta, decay [N, H], o_raw [N, H, dv]: float32 scratch; out [N, H dv] in the run dtype.
JLE_API int jle_gated_delta(const void* rows, int is_bf16, const float* gates, const float* a_log, const float* dt_bias,
                            const float* norm_w, const void* gate, float* state, const int* cu_seqlens,
                            const int* state_slots, const int* state_phase, float* qn, float* kn, float* beta,
                            float* decay, float* o_raw, void* out, int N, int R, int H, int G, int dk, int dv, float eps,
                            float floor, hipStream_t s) {
  if (N <= 0) return 0;
  if (R <= 0 || H <= 0 || G <= 0 || H % G || dk <= 0 || dk > 2048 || dv <= 0 || H > 65535 || G + 1 > 65535 ||
      rows == nullptr || gates == nullptr || state == nullptr || out == nullptr || gate == nullptr)
    return JLE_BAD_ARG;
  if (is_bf16)
    return launch_gdr<bf16_t>((const bf16_t*)rows, gates, a_log, dt_bias, norm_w, (const bf16_t*)gate, state, cu_seqlens,
                              state_slots, state_phase, qn, kn, beta, decay, o_raw, (bf16_t*)out, N, R, H, G, dk, dv, eps,
                              floor, s);
  return launch_gdr<float>((const float*)rows, gates, a_log, dt_bias, norm_w, (const float*)gate, state, cu_seqlens,
                           state_slots, state_phase, qn, kn, beta, decay, o_raw, (float*)out, N, R, H, G, dk, dv, eps,
                           floor, s);
}
