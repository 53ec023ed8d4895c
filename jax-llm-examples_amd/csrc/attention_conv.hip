// Behind a fused q|k|v projection whose rows pass a short causal convolution over time before anything else:
//     u[t]   = proj[t] + bias                                   (rounded to the run dtype: what the state keeps)
//     y[t,c] = sum_j w[j, c] * u[t - taps + 1 + j, c]           (zeros before the sequence's start)
// then, per head, the rotation of q and k (adjacent pairs of the leading rotary_dim elements, sines and cosines
// times a magnitude), their division by the root mean square over the head, and the write of k and v into their
// page.  Queries and keys have dk elements a head, values dv; the pages (and the queries handed on) hold heads of
// D >= max(dk, dv) elements, the rest zeros, so that the attention kernels see one head size.
//
// The rows before a segment's first token come from the request's state: state[slot][half][taps - 1][C], the
// oldest row first.  A step reads the half `phase` and writes the other, so a step that is run twice (once launch
// by launch, once as a recorded graph) reads the same rows both times.
//
// One wavefront per (token, head); a lane holds elements lane, lane + 64, ... of the head, so the two elements of
// a rotated pair lie in neighbouring lanes.  Everything in float32; the order of every sum depends on the sizes only.
#include "common.h"

using namespace jle;

namespace {

constexpr int kMaxPerLane = 8;  // heads of up to 512 elements

template <typename PT, typename T>
struct ConvArgs {
  const PT* proj;      // [N, C]
  const float* bias;   // [C] or null
  const float* w;      // [taps, C] (a tap's weights of all channels side by side) or null (taps == 0)
  T* state;            // [slots, 2, taps - 1, C] or null (taps <= 1)
  const int* token_segment;
  const int* cu_seqlens;
  const int* state_slots;
  const int* state_phase;
  const int* positions;
  const int* slot_mapping;
  const float* inv_freq;  // [rotary_dim / 2] or null
  T* q_out;               // [N, Hq, D]
  T* kv_cache;            // [pages, 2, Hkv, ps, D] (values [D][ps]) or null
  float magnitude, norm_eps;  // norm_eps < 0: no norm
  int taps, C, Hq, Hkv, dk, dv, D, ps, rotary_dim;
  int act;  // (the convolution alone) 1: y * sigmoid(y) before the rounding
};

__device__ __forceinline__ float conv_act(float y, int act) { return act == 1 ? y / (1.0f + expf(-y)) : y; }

// the projected value of channel c in row `row`, with its bias, as the run dtype holds it
template <typename PT, typename T>
__device__ __forceinline__ float projected(const ConvArgs<PT, T>& a, size_t row, int c) {
  float v = Num<PT>::load(a.proj + row * a.C + c);
  if (a.bias != nullptr) v += a.bias[c];
  return Num<T>::round(v);
}

template <typename PT, typename T>
__global__ __launch_bounds__(64) void conv_qk_prepare_kernel(ConvArgs<PT, T> a) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool is_q = h < a.Hq, is_v = h >= a.Hq + a.Hkv;
  if (!is_q && a.kv_cache == nullptr) return;
  const int dim = is_v ? a.dv : a.dk;
  const int c0 = is_q ? h * a.dk : is_v ? (a.Hq + a.Hkv) * a.dk + (h - a.Hq - a.Hkv) * a.dv : h * a.dk;
  const int seg = a.token_segment[n];
  const int row0 = a.cu_seqlens[seg];
  const int t = n - row0;  // the token's place in its segment
  const int K = a.taps;
  const T* old = nullptr;
  if (K > 1) old = a.state + ((size_t)a.state_slots[seg] * 2 + a.state_phase[seg]) * (K - 1) * a.C;
  float y[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int e = lane + 64 * i;
    y[i] = 0.f;
    if (e < dim) {
      const int c = c0 + e;
      if (K == 0) {
        y[i] = projected(a, (size_t)n, c);
      } else {
        float acc = 0.f;
        for (int j = 0; j < K; ++j) {
          const int back = K - 1 - j;
          const float u = t - back >= 0 ? projected(a, (size_t)(n - back), c)
                                        : Num<T>::load(old + (size_t)(K - 1 + t - back) * a.C + c);
          acc = __builtin_fmaf(a.w[(size_t)j * a.C + c], u, acc);
        }
        y[i] = Num<T>::round(acc);
      }
    }
  }
  if (!is_v) {
    const float pos = (float)a.positions[n];
    const int rd = a.inv_freq != nullptr ? a.rotary_dim : 0;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int e = lane + 64 * i;
      const float other = __shfl_xor(y[i], 1, 64);  // the pair's other element (every lane takes part)
      if (e < rd) {
        float sn, cs;
        sincosf(pos * a.inv_freq[e >> 1], &sn, &cs);
        sn *= a.magnitude;
        cs *= a.magnitude;
        y[i] = (e & 1) ? y[i] * cs + other * sn : y[i] * cs - other * sn;
      }
      ss = __builtin_fmaf(y[i], y[i], ss);
    }
    if (a.norm_eps >= 0.f) {
      const float mul = 1.0f / sqrtf(wave_sum(ss) / (float)a.dk + a.norm_eps);
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) y[i] *= mul;
    }
  }
  T* dst;
  size_t stride = 1;
  if (is_q) {
    dst = a.q_out + ((size_t)n * a.Hq + h) * a.D;
  } else {
    const int slot = a.slot_mapping[n];
    const int page = slot / a.ps, off = slot - page * a.ps;
    const int hk = is_v ? h - a.Hq - a.Hkv : h - a.Hq;
    T* plane = a.kv_cache + (((size_t)page * 2 + (is_v ? 1 : 0)) * a.Hkv + hk) * a.ps * a.D;
    if (is_v) {
      dst = plane + off;
      stride = a.ps;
    } else {
      dst = plane + (size_t)off * a.D;
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int e = lane + 64 * i;
    if (e < a.D) Num<T>::store(dst + (size_t)e * stride, e < dim ? y[i] : 0.f);
  }
}

// The state's other half: the last taps - 1 rows of u of every segment's request (older rows from the old half
// where the segment is shorter than that).
template <typename PT, typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(ConvArgs<PT, T> a) {
  const int seg = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.C) return;
  const int K = a.taps;
  const int row0 = a.cu_seqlens[seg], len = a.cu_seqlens[seg + 1] - row0;
  const size_t slot = (size_t)a.state_slots[seg];
  const int phase = a.state_phase[seg];
  const T* old = a.state + (slot * 2 + phase) * (K - 1) * a.C;
  T* fresh = a.state + (slot * 2 + (1 - phase)) * (K - 1) * a.C;
  for (int i = 0; i < K - 1; ++i) {
    const int rel = len - (K - 1) + i;  // the row's place counted from the segment's first token
    const float u = rel >= 0 ? projected(a, (size_t)(row0 + rel), c) : Num<T>::load(old + (size_t)(K - 1 + rel) * a.C + c);
    Num<T>::store(fresh + (size_t)i * a.C + c, u);
  }
}

// The convolution alone, for sizes that the plain preparation kernels take afterwards: y[N, C] in the run dtype
// (q heads, k heads, v heads as the projection laid them) and the state's other half, in one launch.  Blocks
// 0 .. N - 1 of the grid's first axis take a token each, the R behind them a segment's state; a thread a channel.
template <typename PT, typename T>
__global__ __launch_bounds__(256) void conv_rows_kernel(ConvArgs<PT, T> a, T* __restrict__ y_out, int N) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.C) return;
  const int K = a.taps;
  if ((int)blockIdx.x >= N) {  // a segment's state
    if (K <= 1) return;
    const int seg = blockIdx.x - N;
    const int row0 = a.cu_seqlens[seg], len = a.cu_seqlens[seg + 1] - row0;
    const size_t slot = (size_t)a.state_slots[seg];
    const int phase = a.state_phase[seg];
    const T* old = a.state + (slot * 2 + phase) * (K - 1) * a.C;
    T* fresh = a.state + (slot * 2 + (1 - phase)) * (K - 1) * a.C;
    for (int i = 0; i < K - 1; ++i) {
      const int rel = len - (K - 1) + i;
      const float u = rel >= 0 ? projected(a, (size_t)(row0 + rel), c) : Num<T>::load(old + (size_t)(K - 1 + rel) * a.C + c);
      Num<T>::store(fresh + (size_t)i * a.C + c, u);
    }
    return;
  }
  const int n = blockIdx.x;
  float y;
  if (K == 0) {
    y = projected(a, (size_t)n, c);
    if (a.act) y = Num<T>::round(conv_act(y, a.act));
  } else {
    const int seg = a.token_segment[n];
    const int t = n - a.cu_seqlens[seg];
    const T* old = nullptr;
    if (K > 1) old = a.state + ((size_t)a.state_slots[seg] * 2 + a.state_phase[seg]) * (K - 1) * a.C;
    float acc = 0.f;
    for (int j = 0; j < K; ++j) {  // (the same sum, in the same order, as conv_qk_prepare_kernel's)
      const int back = K - 1 - j;
      const float u = t - back >= 0 ? projected(a, (size_t)(n - back), c)
                                    : Num<T>::load(old + (size_t)(K - 1 + t - back) * a.C + c);
      acc = __builtin_fmaf(a.w[(size_t)j * a.C + c], u, acc);
    }
    y = Num<T>::round(conv_act(acc, a.act));
  }
  Num<T>::store(y_out + (size_t)n * a.C + c, y);
}

// Eight neighbouring channels a thread (C a multiple of 8, every array 16-byte aligned): the same sums in the same
// order as above, so which of the two kernels runs changes no bit.
template <typename T>
struct Row8;
template <>
struct Row8<float> {
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4*>(p + 4) = float4{v[4], v[5], v[6], v[7]};
  }
};
template <>
struct Row8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float* v) {
    *reinterpret_cast<uint4*>(p) = uint4{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]),
                                         pack_bf16(v[6], v[7])};
  }
};

template <typename PT, typename T>
__device__ __forceinline__ void projected8(const ConvArgs<PT, T>& a, size_t row, int c, const float* bias8, float* u) {
  Row8<PT>::load(a.proj + row * a.C + c, u);
#pragma unroll
  for (int i = 0; i < 8; ++i) u[i] = Num<T>::round(u[i] + bias8[i]);
}

constexpr int kRowsPerBlock = 8;  // tokens a block of the eight-channel kernel takes in a step of many tokens
constexpr int kTapsInRegisters = 8;

// A block takes rows_per_block consecutive tokens of the step for its channels (one in a step of few tokens, where
// the blocks are few as it is): the taps' weights and the bias are read once per block (up to kTapsInRegisters taps;
// more are read again for every token), and the rows that neighbouring tokens share come from the first-level
// cache.  A token's sums are the same whatever the number.
template <typename PT, typename T>
__global__ __launch_bounds__(256) void conv_rows_vec_kernel(ConvArgs<PT, T> a, T* __restrict__ y_out, int N,
                                                            int token_blocks, int rows_per_block) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= a.C) return;
  const int K = a.taps;
  float bias8[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) bias8[i] = 0.f;
  if (a.bias != nullptr) Row8<float>::load(a.bias + c, bias8);
  float u[8];
  if ((int)blockIdx.x >= token_blocks) {  // a segment's state
    if (K <= 1) return;
    const int seg = blockIdx.x - token_blocks;
    const int row0 = a.cu_seqlens[seg], len = a.cu_seqlens[seg + 1] - row0;
    const size_t slot = (size_t)a.state_slots[seg];
    const int phase = a.state_phase[seg];
    const T* old = a.state + (slot * 2 + phase) * (K - 1) * a.C;
    T* fresh = a.state + (slot * 2 + (1 - phase)) * (K - 1) * a.C;
    for (int i = 0; i < K - 1; ++i) {
      const int rel = len - (K - 1) + i;
      if (rel >= 0) projected8(a, (size_t)(row0 + rel), c, bias8, u);
      else Row8<T>::load(old + (size_t)(K - 1 + rel) * a.C + c, u);
      Row8<T>::store(fresh + (size_t)i * a.C + c, u);
    }
    return;
  }
  float wreg[kTapsInRegisters][8];
#pragma unroll
  for (int j = 0; j < kTapsInRegisters; ++j)
    if (j < K) Row8<float>::load(a.w + (size_t)j * a.C + c, wreg[j]);
  const int n_end = min(N, ((int)blockIdx.x + 1) * rows_per_block);
  for (int n = blockIdx.x * rows_per_block; n < n_end; ++n) {
    float y[8];
    if (K == 0) {
      projected8(a, (size_t)n, c, bias8, y);
      if (a.act) {
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = Num<T>::round(conv_act(y[i], a.act));
      }
    } else {
      const int seg = a.token_segment[n];
      const int t = n - a.cu_seqlens[seg];
      const T* old = nullptr;
      if (K > 1) old = a.state + ((size_t)a.state_slots[seg] * 2 + a.state_phase[seg]) * (K - 1) * a.C;
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = 0.f;
#pragma unroll
      for (int j = 0; j < kTapsInRegisters; ++j) {  // (the taps ascending, as in every kernel of this file)
        if (j < K) {
          const int back = K - 1 - j;
          if (t - back >= 0) projected8(a, (size_t)(n - back), c, bias8, u);
          else Row8<T>::load(old + (size_t)(K - 1 + t - back) * a.C + c, u);
#pragma unroll
          for (int i = 0; i < 8; ++i) y[i] = __builtin_fmaf(wreg[j][i], u[i], y[i]);
        }
      }
      for (int j = kTapsInRegisters; j < K; ++j) {
        const int back = K - 1 - j;
        if (t - back >= 0) projected8(a, (size_t)(n - back), c, bias8, u);
        else Row8<T>::load(old + (size_t)(K - 1 + t - back) * a.C + c, u);
        float w8[8];
        Row8<float>::load(a.w + (size_t)j * a.C + c, w8);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = __builtin_fmaf(w8[i], u[i], y[i]);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = Num<T>::round(conv_act(y[i], a.act));
    }
    Row8<T>::store(y_out + (size_t)n * a.C + c, y);
  }
}

template <typename PT, typename T>
int launch_conv_rows(const ConvArgs<PT, T>& a, void* y_out, int N, int R, hipStream_t s) {
  const uintptr_t all = (uintptr_t)a.proj | (uintptr_t)a.bias | (uintptr_t)a.w | (uintptr_t)a.state | (uintptr_t)y_out;
  if (a.C % 8 == 0 && all % 16 == 0)  // (by the sizes alone: the same kernel for every step of a model)
  {
    const int per = N >= 512 ? kRowsPerBlock : 1;
    const int token_blocks = (N + per - 1) / per;
    hipLaunchKernelGGL((conv_rows_vec_kernel<PT, T>), dim3(token_blocks + (a.taps > 1 ? R : 0), (a.C / 8 + 255) / 256),
                       dim3(256), 0, s, a, (T*)y_out, N, token_blocks, per);
  }
  else
    hipLaunchKernelGGL((conv_rows_kernel<PT, T>), dim3(N + (a.taps > 1 ? R : 0), (a.C + 255) / 256), dim3(256), 0, s, a,
                       (T*)y_out, N);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

template <typename PT, typename T>
int launch_conv(const ConvArgs<PT, T>& a, int N, int R, hipStream_t s) {
  hipLaunchKernelGGL((conv_qk_prepare_kernel<PT, T>), dim3(N, a.Hq + 2 * a.Hkv), dim3(64), 0, s, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  if (a.taps > 1) {
    hipLaunchKernelGGL((conv_state_kernel<PT, T>), dim3(R, (a.C + 255) / 256), dim3(256), 0, s, a);
    e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  return 0;
}

}  // namespace

// proj: [N, C] with C = (Hq + Hkv) * dk + Hkv * dv, float32 (proj_f32) or the run dtype (is_bf16).  N tokens in R
// segments.  kv_cache null: this run writes no pages (the queries are prepared all the same).
JLE_API int jle_conv_qk_prepare(const void* proj, int proj_f32, const float* bias, const float* conv_w, int taps,
                                void* state, const int* token_segment, const int* cu_seqlens, const int* state_slots,
                                const int* state_phase, const int* positions, const int* slot_mapping,
                                const float* inv_freq, int rotary_dim, float magnitude, float norm_eps, void* q_out,
                                void* kv_cache, int is_bf16, int N, int R, int Hq, int Hkv, int dk, int dv, int D,
                                int ps, hipStream_t s) {
  if (N <= 0) return 0;
  if (Hq <= 0 || Hkv <= 0 || dk <= 0 || dv <= 0 || D < dk || D < dv || D > 64 * kMaxPerLane || taps < 0 || R <= 0 ||
      Hq + 2 * Hkv > 65535 || R > 65535 * 16)
    return JLE_BAD_ARG;
  if ((taps > 0 && conv_w == nullptr) || (taps > 1 && (state == nullptr || state_slots == nullptr || state_phase == nullptr)))
    return JLE_BAD_ARG;
  if (inv_freq != nullptr && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > dk)) return JLE_BAD_ARG;
  if (kv_cache != nullptr && (slot_mapping == nullptr || ps <= 0)) return JLE_BAD_ARG;
  if (!is_bf16 && !proj_f32) return JLE_BAD_ARG;
  const int C = (Hq + Hkv) * dk + Hkv * dv;
  if ((C + 255) / 256 > 65535) return JLE_BAD_ARG;
#define JLE_CONV_ARGS(PT, T)                                                                                        \
  ConvArgs<PT, T> a{(const PT*)proj, bias, conv_w, (T*)state, token_segment, cu_seqlens, state_slots, state_phase, \
                    positions, slot_mapping, inv_freq, (T*)q_out, (T*)kv_cache, magnitude, norm_eps, taps, C, Hq,  \
                    Hkv, dk, dv, D, ps, rotary_dim}
  if (!is_bf16) {
    JLE_CONV_ARGS(float, float);
    return launch_conv(a, N, R, s);
  }
  if (proj_f32) {
    JLE_CONV_ARGS(float, bf16_t);
    return launch_conv(a, N, R, s);
  }
  JLE_CONV_ARGS(bf16_t, bf16_t);
  return launch_conv(a, N, R, s);
#undef JLE_CONV_ARGS
}

// The convolution alone: y [N, C] in the run dtype, C channels of any meaning; the state as above.
static int conv_rows_act(const void* proj, int proj_f32, const float* bias, const float* conv_w, int taps,
                         void* state, const int* token_segment, const int* cu_seqlens, const int* state_slots,
                         const int* state_phase, void* y_out, int is_bf16, int N, int R, int C, int act, hipStream_t s) {
  if (N <= 0) return 0;
  if (act < 0 || act > 1) return JLE_BAD_ARG;
  if (C <= 0 || taps < 0 || R <= 0 || (C + 255) / 256 > 65535 || y_out == nullptr) return JLE_BAD_ARG;
  if ((taps > 0 && conv_w == nullptr) || (taps > 1 && (state == nullptr || state_slots == nullptr || state_phase == nullptr)))
    return JLE_BAD_ARG;
  if (!is_bf16 && !proj_f32) return JLE_BAD_ARG;
#define JLE_ROWS_ARGS(PT, T)                                                                                        \
  ConvArgs<PT, T> a{(const PT*)proj, bias, conv_w, (T*)state, token_segment, cu_seqlens, state_slots, state_phase, \
                    nullptr, nullptr, nullptr, nullptr, nullptr, 1.f, -1.f, taps, C, 0, 0, 0, 0, 0, 0, 0, act}
  if (!is_bf16) {
    JLE_ROWS_ARGS(float, float);
    return launch_conv_rows(a, y_out, N, R, s);
  }
  if (proj_f32) {
    JLE_ROWS_ARGS(float, bf16_t);
    return launch_conv_rows(a, y_out, N, R, s);
  }
  JLE_ROWS_ARGS(bf16_t, bf16_t);
  return launch_conv_rows(a, y_out, N, R, s);
#undef JLE_ROWS_ARGS
}

JLE_API int jle_conv_rows(const void* proj, int proj_f32, const float* bias, const float* conv_w, int taps,
                          void* state, const int* token_segment, const int* cu_seqlens, const int* state_slots,
                          const int* state_phase, void* y_out, int is_bf16, int N, int R, int C, hipStream_t s) {
  return conv_rows_act(proj, proj_f32, bias, conv_w, taps, state, token_segment, cu_seqlens, state_slots, state_phase,
                       y_out, is_bf16, N, R, C, 0, s);
}

// The same with an activation on the convolution's result (act 1: y * sigmoid(y), float32, before the rounding).
JLE_API int jle_conv_rows_act(const void* proj, int proj_f32, const float* bias, const float* conv_w, int taps,
                              void* state, const int* token_segment, const int* cu_seqlens, const int* state_slots,
                              const int* state_phase, void* y_out, int is_bf16, int N, int R, int C, int act,
                              hipStream_t s) {
  return conv_rows_act(proj, proj_f32, bias, conv_w, taps, state, token_segment, cu_seqlens, state_slots, state_phase,
                       y_out, is_bf16, N, R, C, act, s);
}
