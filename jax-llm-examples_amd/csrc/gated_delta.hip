// The gated delta rule: a matrix memory S (dk x dv, float32) per head and request, written and read token by token,
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with q, k unit vectors per kv head (x / sqrt(sum(x^2) + floor), q times dk^(-1/2)), beta = sigmoid(b),
// g = exp(-exp(A) softplus(a + dt)).  Three kernels:
//   gdr_prepare_kernel   the unit vectors (float32), beta and the decay of every token of the step
//   gdr_scan_kernel      the recurrence: a column of S depends on nothing but itself, k, q, v of its own place, beta
//                        and g, so a wavefront takes 64 / KS columns of one head, KS neighbouring lanes share a
//                        column (each holds R consecutive rows of it in registers), and the two dot products are
//                        finished with log2(KS) lane swaps; the next tokens' rows are asked for before these are used
//   gdr_out_kernel       o / sqrt(mean(o^2) + eps) * w * silu(gate), rounded to the run dtype
// The memory lies [slot][half][H][dv][dk] (a column's rows together); a step reads the half `phase` and writes the other.  Every sum is formed
// in an order that depends on the sizes alone, token after token: cutting a sequence into steps changes no bit.
#include "common.h"

using namespace jle;

namespace {

template <typename T>
__global__ __launch_bounds__(64) void gdr_prepare_kernel(const T* __restrict__ rows, const float* __restrict__ gates,
                                                         const float* __restrict__ a_log,
                                                         const float* __restrict__ dt_bias, float* __restrict__ qn,
                                                         float* __restrict__ kn, float* __restrict__ beta,
                                                         float* __restrict__ decay, float* __restrict__ kq,
                                                         float floor, int H, int G, int dk, int dv, int dkp) {
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
    float* dst = (which == 0 ? qn : kn) + ((size_t)n * G + g) * dkp;  // (rows of dkp >= dk floats, zeros behind)
    float ss = 0.f;
    for (int e = lane; e < dk; e += 64) {
      const float x = Num<T>::load(src + e);
      ss = __builtin_fmaf(x, x, ss);
    }
    float inv = 1.0f / sqrtf(wave_sum(ss) + floor);
    if (which == 0) inv *= 1.0f / sqrtf((float)dk);
    for (int e = lane; e < dkp; e += 64) dst[e] = e < dk ? Num<T>::load(src + e) * inv : 0.f;
  }
  // the product of the token's own two unit vectors (what its write adds to its own read-out)
  const float* qd = qn + ((size_t)n * G + g) * dkp;
  const float* kd = kn + ((size_t)n * G + g) * dkp;
  float d = 0.f;
  for (int e = lane; e < dk; e += 64) d = __builtin_fmaf(qd[e], kd[e], d);  // (this lane's own stores)
  d = wave_sum(d);
  if (lane == 0) kq[(size_t)n * G + g] = d;
}

// KS lanes share a column, each with R consecutive rows of it (KS * R = dkp >= dk, the unit vectors' rows padded with
// zeros to that).  The wavefront brings the unit vectors, write strengths and decays of TB tokens into shared memory
// at a time (asked for while the TB tokens before are worked on), and a lane its own values into registers.
// the sum over the KS neighbouring lanes that share a column (every one of them gets it, the same bits in all):
// within a row of 16 lanes by the lane-permuting operand modes, beyond by the cross-lane read
template <int CTRL>
__device__ __forceinline__ float lanes_permuted(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int KS>
__device__ __forceinline__ float column_lanes_sum(float v) {
  if (KS >= 2) v += lanes_permuted<0xB1>(v);    // lanes 1 0 3 2 of every four
  if (KS >= 4) v += lanes_permuted<0x4E>(v);    // lanes 2 3 0 1 of every four
  if (KS >= 8) v += lanes_permuted<0x141>(v);   // every eight mirrored
  if (KS >= 16) v += lanes_permuted<0x140>(v);  // every sixteen mirrored
  if (KS >= 32) v += __shfl_xor(v, 16, 64);
  if (KS >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

typedef float f32x4 __attribute__((ext_vector_type(4)));  // (a plain vector type: arrays of it stay in registers)

template <int KS, int R>
struct ScanShape {
  static constexpr int kDkp = KS * R;
  static constexpr int kTB = kDkp <= 256 ? 16 : kDkp <= 512 ? 8 : kDkp <= 1024 ? 4 : 2;
  static constexpr int kVecs = (kTB * kDkp / 4 + 63) / 64;  // 16-byte pieces a lane brings in per array
};

template <typename T, int KS, int R>
__global__ __launch_bounds__(64) void gdr_scan_kernel(const T* __restrict__ rows, const float* __restrict__ qn,
                                                      const float* __restrict__ kn, const float* __restrict__ beta,
                                                      const float* __restrict__ decay, const float* __restrict__ kq,
                                                      float* __restrict__ state,
                                                      const int* __restrict__ cu_seqlens,
                                                      const int* __restrict__ state_slots,
                                                      const int* __restrict__ state_phase, float* __restrict__ o_raw,
                                                      int H, int G, int dk, int dv) {
  using Shape = ScanShape<KS, R>;
  constexpr int TB = Shape::kTB, DKP = Shape::kDkp, NV = Shape::kVecs, cols = 64 / KS;
  __shared__ f32x4 sk[TB * DKP / 4], sq[TB * DKP / 4];
  __shared__ f32x4 ssc[TB];  // a token's decay, write strength and k . q together: one trip to shared memory
  const int seg = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int ks = lane % KS, c = blockIdx.z * cols + lane / KS;  // (a column's lanes are neighbours)
  const bool live = c < dv;
  const int g = h / (H / G);
  const int C = 2 * G * dk + H * dv;
  const int t0 = cu_seqlens[seg], t1 = cu_seqlens[seg + 1];
  if (t0 >= t1) return;
  const size_t slot = (size_t)state_slots[seg];
  const int phase = state_phase[seg];
  const float* s_old = state + ((slot * 2 + phase) * H + h) * (size_t)dk * dv;
  float* s_new = state + ((slot * 2 + (1 - phase)) * H + h) * (size_t)dk * dv;
  const int k0 = ks * R;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = 0.f;
  // (a column's dk rows lie together: its KS lanes read neighbouring pieces of R floats)
  if (live) {
    if (dk % 4 == 0) {
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        if (k0 + i < dk) {
          const float4 v = *reinterpret_cast<const float4*>(s_old + (size_t)c * dk + k0 + i);
          S[i] = v.x; S[i + 1] = v.y; S[i + 2] = v.z; S[i + 3] = v.w;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < R; ++i)
        if (k0 + i < dk) S[i] = s_old[(size_t)c * dk + k0 + i];
    }
  }

  f32x4 stk[NV], stq[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) stk[j] = stq[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  float vnext[TB], vcur[TB], bnext = 0.f, gnext = 1.f, kqnext = 0.f;
  auto ask = [&](int tb) __attribute__((always_inline)) {  // the TB tokens from tb on (those beyond the segment's end: its last token again, unused)
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int f = lane + 64 * j;
      if (f < TB * DKP / 4) {
        const int tt = f / (DKP / 4), off = f - tt * (DKP / 4);
        const size_t row = ((size_t)min(tb + tt, t1 - 1) * G + g) * DKP;
        stk[j] = reinterpret_cast<const f32x4*>(kn + row)[off];
        stq[j] = reinterpret_cast<const f32x4*>(qn + row)[off];
      }
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt)
      vnext[tt] = live ? Num<T>::load(rows + (size_t)min(tb + tt, t1 - 1) * C + 2 * G * dk + (size_t)h * dv + c) : 0.f;
    if (lane < TB) {  // (places behind the segment's end: a step that changes nothing, no write and no decay)
      const size_t at = (size_t)min(tb + lane, t1 - 1) * H + h;
      bnext = tb + lane < t1 ? beta[at] : 0.f;
      gnext = tb + lane < t1 ? decay[at] : 1.f;
      kqnext = kq[(size_t)min(tb + lane, t1 - 1) * G + g];
    }
  };
  auto put = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int f = lane + 64 * j;
      if (f < TB * DKP / 4) {
        sk[f] = stk[j];
        sq[f] = stq[j];
      }
    }
    if (lane < TB) {
      ssc[lane] = f32x4{gnext, bnext, kqnext, 0.f};
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) vcur[tt] = vnext[tt];
  };
  ask(t0);
  put();
  __syncthreads();
  for (int tb = t0; tb < t1; tb += TB) {
    const bool more = tb + TB < t1;
    if (more) ask(tb + TB);
    float outs[TB];  // (the block's read-outs: stored together behind its last token)
    auto token = [&](int tt) __attribute__((always_inline)) {
      float kc[R], qc[R];
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const f32x4 a = sk[(tt * DKP + k0 + i) / 4], b = sq[(tt * DKP + k0 + i) / 4];
        kc[i] = a.x; kc[i + 1] = a.y; kc[i + 2] = a.z; kc[i + 3] = a.w;
        qc[i] = b.x; qc[i + 1] = b.y; qc[i + 2] = b.z; qc[i + 3] = b.w;
      }
      // With S the memory before the token: the write is u = beta (v - g S^T k), the read-out S'^T q of the memory
      // after it, S' = g S + k u^T, is g S^T q + (k . q) u: both products with S stand side by side, and from one
      // token to the next leads one multiply-add of the memory.
      const f32x4 sc = ssc[tt];
      const float gc = sc.x, bc = sc.y, kqc = sc.z;
      float d4[4] = {0.f, 0.f, 0.f, 0.f}, o4[4] = {0.f, 0.f, 0.f, 0.f};  // (four sums side by side, not a chain of R)
#pragma unroll
      for (int i = 0; i < R; ++i) {
        d4[i & 3] = __builtin_fmaf(S[i], kc[i], d4[i & 3]);
        o4[i & 3] = __builtin_fmaf(S[i], qc[i], o4[i & 3]);
      }
      const float dot = column_lanes_sum<KS>((d4[0] + d4[1]) + (d4[2] + d4[3]));
      const float oq = column_lanes_sum<KS>((o4[0] + o4[1]) + (o4[2] + o4[3]));
      const float u = bc * (vcur[tt] - gc * dot);
      const float out = __builtin_fmaf(kqc, u, gc * oq);
#pragma unroll
      for (int i = 0; i < R; ++i) S[i] = __builtin_fmaf(kc[i], u, gc * S[i]);
      outs[tt] = out;
    };
    if (tb + TB <= t1) {  // a whole block: no branch around a token, one stretch of code that the compiler may interleave
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) token(tt);
    } else {  // (the segment's last tokens, or all of a short one: no work for places behind its end)
#pragma unroll
      for (int tt = 0; tt < TB; ++tt)
        if (tb + tt < t1) token(tt);
    }
    if (live && ks == 0) {
      float* op = o_raw + ((size_t)tb * H + h) * dv + c;
#pragma unroll
      for (int tt = 0; tt < TB; ++tt)
        if (tb + tt < t1) op[(size_t)tt * H * dv] = outs[tt];
    }
    __syncthreads();
    if (more) put();
    __syncthreads();
  }
  if (live) {
    if (dk % 4 == 0) {
#pragma unroll
      for (int i = 0; i < R; i += 4)
        if (k0 + i < dk)
          *reinterpret_cast<float4*>(s_new + (size_t)c * dk + k0 + i) = float4{S[i], S[i + 1], S[i + 2], S[i + 3]};
    } else {
#pragma unroll
      for (int i = 0; i < R; ++i)
        if (k0 + i < dk) s_new[(size_t)c * dk + k0 + i] = S[i];
    }
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
               float* qn, float* kn, float* beta, float* decay, float* kq, float* o_raw, T* out, int N, int R_, int H,
               int G, int dk, int dv, int dkp, float eps, float floor, hipStream_t s) {
  // lanes a column: the fewest that leave a lane at most 16 rows of it (by the sizes alone)
  int KS = 1;
  while (KS < 64 && (dk + KS - 1) / KS > 16) KS <<= 1;
  const int per = (dk + KS - 1) / KS;
  const int RR = per <= 4 ? 4 : per <= 8 ? 8 : per <= 16 ? 16 : 32;
  if (dkp != KS * RR) return JLE_BAD_ARG;
  hipLaunchKernelGGL(gdr_prepare_kernel<T>, dim3(N, G + 1), dim3(64), 0, s, rows, gates, a_log, dt_bias, qn, kn, beta,
                     decay, kq, floor, H, G, dk, dv, dkp);
  JLE_LAUNCH_CHECK();
  // A step with few (segment, head) pairs leaves most of the machine idle, and what a token takes is the length of its
  // chain of dependent operations: then a column gets more lanes with fewer rows each (the row's width stays).
  int ks = KS, rr = RR;
  while (rr > 4 && ks < 16 && (long long)R_ * H * ((dv + 64 / ks - 1) / (64 / ks)) < 1024) {  // (up to a row of 16 lanes)
    ks <<= 1;
    rr >>= 1;
  }
  const int cols_ = 64 / ks;
  const dim3 grid(R_, H, (dv + cols_ - 1) / cols_);
#define JLE_SCAN(KS_, RR_)                                                                                          \
  hipLaunchKernelGGL((gdr_scan_kernel<T, KS_, RR_>), grid, dim3(64), 0, s, rows, qn, kn, beta, decay, kq, state, cu_seqlens, \
                     state_slots, state_phase, o_raw, H, G, dk, dv)
#define JLE_SCAN_R(KS_)              \
  do {                               \
    if (rr == 4) JLE_SCAN(KS_, 4);   \
    else if (rr == 8) JLE_SCAN(KS_, 8); \
    else if (rr == 16) JLE_SCAN(KS_, 16); \
    else JLE_SCAN(KS_, 32);          \
  } while (0)
  switch (ks) {
    case 1: JLE_SCAN_R(1); break;
    case 2: JLE_SCAN_R(2); break;
    case 4: JLE_SCAN_R(4); break;
    case 8: JLE_SCAN_R(8); break;
    case 16: JLE_SCAN_R(16); break;
    case 32: JLE_SCAN_R(32); break;
    default: JLE_SCAN_R(64); break;
  }
#undef JLE_SCAN_R
#undef JLE_SCAN
  JLE_LAUNCH_CHECK();
  hipLaunchKernelGGL(gdr_out_kernel<T>, dim3(N, H), dim3(64), 0, s, o_raw, gate, norm_w, out, eps, H, dv);
  JLE_LAUNCH_CHECK();
  return 0;
}

}  // namespace

// The width of a unit vector's row in the scratch arrays: dk rounded up to lanes a column x rows a lane.
JLE_API int jle_gated_delta_padded(int dk) {
  if (dk <= 0 || dk > 2048) return -1;
  int KS = 1;
  while (KS < 64 && (dk + KS - 1) / KS > 16) KS <<= 1;
  const int per = (dk + KS - 1) / KS;
  return KS * (per <= 4 ? 4 : per <= 8 ? 8 : per <= 16 ? 16 : 32);
}

// rows [N, 2 G dk + H dv] (q | k | v behind convolution and activation) and gate [N, H dv] in the run dtype; gates
// float32 [N, 2 H] (write strengths, then decays, before their biases and squashing); state float32 [slots, 2, H, dv,
// dk]; qn, kn [N, G, dkp] (dkp = jle_gated_delta_padded(dk), 16-byte aligned), beta, decay [N, H], o_raw [N, H, dv]:
// float32 scratch; out [N, H dv] in the run dtype.
JLE_API int jle_gated_delta(const void* rows, int is_bf16, const float* gates, const float* a_log, const float* dt_bias,
                            const float* norm_w, const void* gate, float* state, const int* cu_seqlens,
                            const int* state_slots, const int* state_phase, float* qn, float* kn, float* beta,
                            float* decay, float* kq, float* o_raw, void* out, int N, int R, int H, int G, int dk, int dv,
                            float eps, float floor, hipStream_t s) {
  if (N <= 0) return 0;
  const int dkp = jle_gated_delta_padded(dk);
  if (dkp <= 0 || ((uintptr_t)qn | (uintptr_t)kn) % 16) return JLE_BAD_ARG;
  if (R <= 0 || H <= 0 || G <= 0 || H % G || dk <= 0 || dk > 2048 || dv <= 0 || H > 65535 || G + 1 > 65535 ||
      rows == nullptr || gates == nullptr || state == nullptr || out == nullptr || gate == nullptr)
    return JLE_BAD_ARG;
  if (is_bf16)
    return launch_gdr<bf16_t>((const bf16_t*)rows, gates, a_log, dt_bias, norm_w, (const bf16_t*)gate, state, cu_seqlens,
                              state_slots, state_phase, qn, kn, beta, decay, kq, o_raw, (bf16_t*)out, N, R, H, G, dk, dv, dkp,
                              eps, floor, s);
  return launch_gdr<float>((const float*)rows, gates, a_log, dt_bias, norm_w, (const float*)gate, state, cu_seqlens,
                           state_slots, state_phase, qn, kn, beta, decay, kq, o_raw, (float*)out, N, R, H, G, dk, dv, dkp, eps,
                           floor, s);
}
