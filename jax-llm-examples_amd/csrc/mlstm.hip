// A matrix memory per head, carried from token to token (the mLSTM cell), float32 state and arithmetic.
//
//   m' = max(f + m, i);  C' = exp(f + m - m') C + exp(i - m') k v^T;  n' = exp(f + m - m') n + exp(i - m') k
//   o  = C'^T q / (max(|n' . q|, exp(-m')) + floor)
//
// Three launches.  (1) The gates: i = cap tanh((a + b_i) / cap), f = logsigmoid(cap tanh((b + b_f) / cap)), in place
// over the pre-activations, every (token, head) on its own.  (2) The recurrence: one wavefront per (segment, head,
// slice of 32 value columns) walks the segment's tokens in order.  Lane (p, j4), p = lane / 8, j4 = lane % 8, holds
// C[k][4 j4 .. 4 j4 + 3] of its slice for the rows k = p, p + 8, ...: a row of the slice is 128 contiguous bytes of
// the state, the products with q are summed over p by three lane exchanges, and nothing goes through shared
// memory.  The next token's q, k, v and gates are asked for before the present token is worked on.  A step reads
// the half `phase` of the request's state and writes the other.  (3) Every head's o divided by its root mean square,
// times the norm's weight, times the sigmoid of the output gate.
//
// rows: [N][2 H dk + 2 H dv] = q | k | v | output gate (T); gates: float32 [N][2 H]; state: float32
// [slots][2][H][dk dv + dk + 1] = C (dk rows of dv), n, m.  A token's result depends on its request's state and
// on the tokens before it in the segment only, each visited once and in order, whatever else the step holds.
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

__global__ void mlstm_gates_kernel(float* __restrict__ gates, const float* __restrict__ bias, float cap, int H,
                                   long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % (2 * H));
  const float z = cap * tanhf((gates[i] + bias[c]) / cap);
  gates[i] = c < H ? z : log_sigmoid(z);
}

template <typename T>
__device__ __forceinline__ f32x4 load_v4(const T* p);
template <>
__device__ __forceinline__ f32x4 load_v4<float>(const float* p) {
  return *reinterpret_cast<const f32x4*>(p);
}
template <>
__device__ __forceinline__ f32x4 load_v4<bf16_t>(const bf16_t* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return f32x4{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
               __uint_as_float(r.y & 0xffff0000u)};
}

// the sum over the eight lanes that share j4 (p = 0 .. 7), in all of them
__device__ __forceinline__ float sum_over_p(float v) {
  v += __shfl_xor(v, 8, 64);
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// VEC: dv is a multiple of 4 (a lane's four columns are there together, and rows of q | k | v | gate and of the state
// can be read four elements at a time); without it every column is guarded and read on its own.
template <typename T, int KP, bool VEC>
__global__ __launch_bounds__(64) void mlstm_scan_kernel(const T* __restrict__ rows, const float* __restrict__ gates,
                                                        float* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ slots, const int* __restrict__ phase,
                                                        float* __restrict__ o_raw, int H, int dk, int dv, float q_mul,
                                                        float floor_) {
  const int seg = blockIdx.x, h = blockIdx.y, slice = blockIdx.z;
  const int lane = threadIdx.x, p = lane >> 3, j4 = lane & 7;
  const int col = slice * 32 + 4 * j4;  // this lane's first value column
  const bool col_ok = col < dv;
  const int t0 = cu[seg], t1 = cu[seg + 1];
  const int width = 2 * H * dk + 2 * H * dv;
  const size_t per_head = (size_t)dk * dv + dk + 1;
  const size_t half = (size_t)H * per_head;
  const float* st_in = state + ((size_t)slots[seg] * 2 + phase[seg]) * half + h * per_head;
  float* st_out = state + ((size_t)slots[seg] * 2 + (1 - phase[seg])) * half + h * per_head;

  f32x4 C[KP];
  float nn[KP];
#pragma unroll
  for (int i = 0; i < KP; ++i) {
    const int k = p + 8 * i;
    C[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (k < dk && col_ok) {
      if (VEC) {
        C[i] = *reinterpret_cast<const f32x4*>(st_in + (size_t)k * dv + col);
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (col + c < dv) C[i][c] = st_in[(size_t)k * dv + col + c];
      }
    }
    nn[i] = k < dk ? st_in[(size_t)dk * dv + k] : 0.f;
  }
  float m = st_in[(size_t)dk * dv + dk];

  float qn[KP], kn[KP];
  f32x4 vn;
  float gi, gf;
  auto fetch = [&](int t) {
    const T* r = rows + (size_t)t * width;
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int k = p + 8 * i;
      qn[i] = k < dk ? Num<T>::load(r + h * dk + k) : 0.f;
      kn[i] = k < dk ? Num<T>::load(r + H * dk + h * dk + k) : 0.f;
    }
    vn = f32x4{0.f, 0.f, 0.f, 0.f};
    if (col_ok) {
      if (VEC) {
        vn = load_v4<T>(r + 2 * H * dk + h * dv + col);
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (col + c < dv) vn[c] = Num<T>::load(r + 2 * H * dk + h * dv + col + c);
      }
    }
    gi = gates[(size_t)t * 2 * H + h];
    gf = gates[(size_t)t * 2 * H + H + h];
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float q[KP], kk[KP];
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      q[i] = qn[i] * q_mul;
      kk[i] = kn[i];
    }
    const f32x4 v = vn;
    const float li = gi, lf = gf;
    if (t + 1 < t1) fetch(t + 1);
    const float m_new = fmaxf(lf + m, li);
    const float keep = expf(lf + m - m_new), take = expf(li - m_new);
    m = m_new;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    float nq = 0.f;
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const float tk = take * kk[i];
      C[i][0] = fmaf(keep, C[i][0], tk * v[0]);
      C[i][1] = fmaf(keep, C[i][1], tk * v[1]);
      C[i][2] = fmaf(keep, C[i][2], tk * v[2]);
      C[i][3] = fmaf(keep, C[i][3], tk * v[3]);
      nn[i] = fmaf(keep, nn[i], tk);
      o[0] = fmaf(C[i][0], q[i], o[0]);
      o[1] = fmaf(C[i][1], q[i], o[1]);
      o[2] = fmaf(C[i][2], q[i], o[2]);
      o[3] = fmaf(C[i][3], q[i], o[3]);
      nq = fmaf(nn[i], q[i], nq);
    }
    o[0] = sum_over_p(o[0]);
    o[1] = sum_over_p(o[1]);
    o[2] = sum_over_p(o[2]);
    o[3] = sum_over_p(o[3]);
    nq = sum_over_p(nq);
    const float den = fmaxf(fabsf(nq), expf(-m)) + floor_;
    if (p == 0 && col_ok) {
      const f32x4 r = {o[0] / den, o[1] / den, o[2] / den, o[3] / den};
      float* dst = o_raw + (size_t)t * H * dv + h * dv + col;
      if (VEC) {
        *reinterpret_cast<f32x4*>(dst) = r;
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (col + c < dv) dst[c] = r[c];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < KP; ++i) {
    const int k = p + 8 * i;
    if (k < dk && col_ok) {
      if (VEC) {
        *reinterpret_cast<f32x4*>(st_out + (size_t)k * dv + col) = C[i];
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (col + c < dv) st_out[(size_t)k * dv + col + c] = C[i][c];
      }
    }
    if (k < dk && slice == 0 && j4 == 0) st_out[(size_t)dk * dv + k] = nn[i];
  }
  if (slice == 0 && lane == 0) st_out[(size_t)dk * dv + dk] = m;
}

// out[t][h][:] = o / sqrt(mean(o^2) + eps) * w[h][:] * sigmoid(gate[t][h][:]); one wavefront per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void mlstm_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ rows,
                                                        const float* __restrict__ w, T* __restrict__ out, int N, int H,
                                                        int dk, int dv, float eps) {
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= N * H) return;
  const int lane = threadIdx.x & 63;
  const int t = item / H, h = item - t * H;
  const float* o = o_raw + (size_t)t * H * dv + h * dv;
  const T* g = rows + (size_t)t * (2 * H * dk + 2 * H * dv) + 2 * H * dk + H * dv + h * dv;
  float ss = 0.f;
  for (int d = lane; d < dv; d += 64) ss = fmaf(o[d], o[d], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int d = lane; d < dv; d += 64) {
    const float gate = 1.0f / (1.0f + expf(-Num<T>::load(g + d)));
    Num<T>::store(out + (size_t)t * H * dv + h * dv + d, o[d] * inv * w[h * dv + d] * gate);
  }
}

// gates is changed in place (pre-activations in, logarithms of the two gates out); o_raw: float32 [N][H dv] scratch.
JLE_API int jle_mlstm(const void* rows, int is_bf16, float* gates, const float* b_gates, const float* norm_w,
                      float* state, const int* cu, const int* slots, const int* phase, float* o_raw, void* out, int N,
                      int R, int H, int dk, int dv, float cap, float eps, float floor_, hipStream_t s) {
  if (N <= 0 || R <= 0) return 0;
  if (H < 1 || dk < 1 || dk > 256 || dv < 1 || !(cap > 0.f)) return JLE_BAD_ARG;
  const long long total = (long long)N * 2 * H;
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gates, b_gates, cap, H,
                     total);
  JLE_LAUNCH_CHECK();
  const dim3 grid(R, H, (dv + 31) / 32);
  const float q_mul = 1.0f / sqrtf((float)dk);
  const int need = (dk + 7) / 8;
  const bool vec = dv % 4 == 0;
#define SCAN(T, KP)                                                                                                   \
  do {                                                                                                                \
    if (vec)                                                                                                          \
      hipLaunchKernelGGL((mlstm_scan_kernel<T, KP, true>), grid, dim3(64), 0, s, (const T*)rows, gates, state, cu,    \
                         slots, phase, o_raw, H, dk, dv, q_mul, floor_);                                              \
    else                                                                                                              \
      hipLaunchKernelGGL((mlstm_scan_kernel<T, KP, false>), grid, dim3(64), 0, s, (const T*)rows, gates, state, cu,   \
                         slots, phase, o_raw, H, dk, dv, q_mul, floor_);                                              \
  } while (0)
#define PICK(T)                   \
  do {                            \
    if (need <= 2) SCAN(T, 2);    \
    else if (need <= 4) SCAN(T, 4);   \
    else if (need <= 6) SCAN(T, 6);   \
    else if (need <= 8) SCAN(T, 8);   \
    else if (need <= 12) SCAN(T, 12); \
    else if (need <= 16) SCAN(T, 16); \
    else if (need <= 24) SCAN(T, 24); \
    else SCAN(T, 32);             \
  } while (0)
  if (is_bf16) PICK(bf16_t);
  else PICK(float);
#undef PICK
#undef SCAN
  JLE_LAUNCH_CHECK();
  const dim3 og((unsigned)(((long long)N * H + 3) / 4));
  if (is_bf16)
    hipLaunchKernelGGL(mlstm_out_kernel<bf16_t>, og, dim3(256), 0, s, o_raw, (const bf16_t*)rows, norm_w, (bf16_t*)out,
                       N, H, dk, dv, eps);
  else
    hipLaunchKernelGGL(mlstm_out_kernel<float>, og, dim3(256), 0, s, o_raw, (const float*)rows, norm_w, (float*)out, N,
                       H, dk, dv, eps);
  JLE_LAUNCH_CHECK();
  return 0;
}
