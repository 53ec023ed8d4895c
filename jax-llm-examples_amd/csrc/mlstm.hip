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

// ------------------------------------------------------------------------------------------------------------------
// Segments of many tokens: chunks of 64 tokens, worked on side by side.  With b_s the sum of the chunk's f up to
// and including token s, a_s = i_s - b_s, and (C0, n0, m0) the state in front of the chunk, the recurrence above
// unrolls to (every exponent below is <= 0, and b_t has left the exponents):
//   g_t = max(m0, max_{s <= t} a_s);   m_t = b_t + g_t
//   C_t^T q_t = exp(m0 - g_t) C0^T q_t + sum_{s <= t} exp(a_s - g_t) (k_s . q_t) v_s      (n_t . q_t likewise)
//   at the chunk's end, with A = max_s a_s:  m' = max(b_L + m0, b_L + A)
//   C' = exp(b_L + m0 - m') C0 + exp(b_L + A - m') sum_s exp(a_s - A) k_s v_s^T
// Three launches over a table of chunks (segment, first row, rows <= 64):
//   state:  per (chunk, head, slice of 64 value columns) the chunk's own sum_s exp(a_s - A) k_s v_s^T, the same with
//           k_s alone, b_L + A and b_L;
//   carry:  per (segment, head), every element of C and n on its own: walks the segment's chunks in order, leaves
//           in each chunk's place the state in front of it, and writes the request's new state;
//   out:    per (chunk, head, slice): Q K^T, the weights exp(a_s - g_t) below the diagonal, times V, plus the
//           part of the state in front; the division.
// All products run on the float32 matrix instruction (16 x 16 x 4: float32 operands, products and sums), from
// shared memory; q, k and v are the projection's rows widened to float32.  Key sizes up to 128.
constexpr int kChunk = 64;
constexpr int kSlice = 64;
constexpr int kPad = 4;  // floats behind a row in shared memory

__device__ __forceinline__ f32x4 mma(float a, float b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// The first wavefront: b_s (the chunk's running sum of f, in lane order) and a_s = i_s - b_s; lanes behind the
// chunk's last token keep b and get an a that no maximum picks and whose exponential is zero.  The sums, a, g and
// their differences are formed in float64 and rounded to float32 where they enter an exponential: under strong
// forgetting b reaches hundreds, and a float32 difference of two such numbers would cost the weights of the
// chunk's last tokens four digits.
__device__ __forceinline__ void chunk_gates(const float* __restrict__ gates, int t0, int n, int H, int h, double* s_a,
                                            double* s_b) {
  const int lane = threadIdx.x;
  const bool ok = lane < n;
  const float f = ok ? gates[(size_t)(t0 + lane) * 2 * H + H + h] : 0.f;
  const float i = ok ? gates[(size_t)(t0 + lane) * 2 * H + h] : 0.f;
  double b = (double)f;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const double u = __shfl_up(b, o, 64);
    if (lane >= o) b += u;
  }
  s_b[lane] = b;
  s_a[lane] = ok ? (double)i - b : -1e30;
}

// rows of the step's q | k | v | gate rows into shared memory as float32: `cols` columns from column `first` of
// the chunk's tokens, `padded` columns a row (zeros behind the real ones and behind the chunk's last token)
template <typename T>
__device__ __forceinline__ void stage_rows(const T* __restrict__ rows, int width, int t0, int n, int first, int cols,
                                           int padded, int stride, float mul, float* dst) {
  constexpr int V = sizeof(T) == 2 ? 8 : 4;  // elements of a 16-byte load
  if (cols % V == 0 && first % V == 0 && width % V == 0) {
    const int per_row = padded / V;  // (padded is a multiple of 16, stride of 4)
    for (int idx = threadIdx.x; idx < kChunk * per_row; idx += blockDim.x) {
      const int s = idx / per_row, c = (idx - s * per_row) * V;
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
      if (s < n && c < cols) {
        const T* src = rows + (size_t)(t0 + s) * width + first + c;
        lo = load_v4<T>(src);
        if (V == 8) hi = load_v4<T>(src + 4);
      }
      *reinterpret_cast<f32x4*>(dst + s * stride + c) = f32x4{lo[0] * mul, lo[1] * mul, lo[2] * mul, lo[3] * mul};
      if (V == 8)
        *reinterpret_cast<f32x4*>(dst + s * stride + c + 4) = f32x4{hi[0] * mul, hi[1] * mul, hi[2] * mul, hi[3] * mul};
    }
    return;
  }
  for (int idx = threadIdx.x; idx < kChunk * padded; idx += blockDim.x) {
    const int s = idx / padded, c = idx - s * padded;
    float v = 0.f;
    if (s < n && c < cols) v = Num<T>::load(rows + (size_t)(t0 + s) * width + first + c) * mul;
    dst[s * stride + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void mlstm_chunk_state_kernel(const T* __restrict__ rows,
                                                                const float* __restrict__ gates,
                                                                const int* __restrict__ chunks, float* __restrict__ ws_C,
                                                                float* __restrict__ ws_n, float* __restrict__ ws_m,
                                                                int H, int dk, int dv) {
  extern __shared__ float lds[];
  const int chunk = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * kSlice;
  const int t0 = chunks[3 * chunk + 1], n = chunks[3 * chunk + 2];
  const int dkp = (dk + 15) & ~15, KS = dkp + kPad, VS = kSlice + kPad;
  const int width = 2 * H * dk + 2 * H * dv;
  double* s_a = reinterpret_cast<double*>(lds);  // [64] each
  double* s_b = s_a + kChunk;
  float* sK = lds + 4 * kChunk;     // [64][KS]
  float* sV = sK + kChunk * KS;     // [64][VS]
  float* s_w = sV + kChunk * VS;    // [64]
  if (threadIdx.x < 64) chunk_gates(gates, t0, n, H, h, s_a, s_b);
  stage_rows<T>(rows, width, t0, n, H * dk + h * dk, dk, dkp, KS, 1.0f, sK);
  stage_rows<T>(rows, width, t0, n, 2 * H * dk + h * dv + c0, min(kSlice, dv - c0), kSlice, VS, 1.0f, sV);
  __syncthreads();
  if (threadIdx.x < 64) {
    double top = s_a[threadIdx.x];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) top = fmax(top, __shfl_xor(top, o, 64));
    s_w[threadIdx.x] = threadIdx.x < n ? expf((float)(s_a[threadIdx.x] - top)) : 0.f;
    if (threadIdx.x == 0 && blockIdx.z == 0) {
      ws_m[((size_t)chunk * H + h) * 2] = (float)(s_b[kChunk - 1] + top);
      ws_m[((size_t)chunk * H + h) * 2 + 1] = (float)s_b[kChunk - 1];
    }
  }
  __syncthreads();
  const int w = wave_index(), lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  const int RT = dkp / 16;
  f32x4 acc[8];
#pragma unroll
  for (int rt = 0; rt < 8; ++rt) acc[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int n4 = (n + 3) & ~3;
  for (int s0 = 0; s0 < n4; s0 += 4) {
    const int s = s0 + g;
    const float b = sV[s * VS + 16 * w + c16];
    const float ww = s_w[s];
#pragma unroll
    for (int rt = 0; rt < 8; ++rt)
      if (rt < RT) acc[rt] = mma(sK[s * KS + 16 * rt + c16] * ww, b, acc[rt]);
  }
  float* dC = ws_C + ((size_t)chunk * H + h) * dk * dv;
  const int c = c0 + 16 * w + c16;
#pragma unroll
  for (int rt = 0; rt < 8; ++rt)
    if (rt < RT) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k = 16 * rt + 4 * g + r;
        if (k < dk && c < dv) dC[(size_t)k * dv + c] = acc[rt][r];
      }
    }
  if (blockIdx.z == 0 && threadIdx.x < dk) {
    float a = 0.f;
    for (int s = 0; s < n; ++s) a = fmaf(s_w[s], sK[s * KS + threadIdx.x], a);
    ws_n[((size_t)chunk * H + h) * dk + threadIdx.x] = a;
  }
}

__global__ __launch_bounds__(256) void mlstm_chunk_carry_kernel(float* __restrict__ state, const int* __restrict__ slots,
                                                                const int* __restrict__ phase,
                                                                const int* __restrict__ seg_chunk0,
                                                                float* __restrict__ ws_C, float* __restrict__ ws_n,
                                                                const float* __restrict__ ws_m,
                                                                float* __restrict__ ws_m0, int H, int dk, int dv) {
  const int seg = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int CE = dk * dv, E = CE + dk;
  const size_t per_head = (size_t)E + 1, half = (size_t)H * per_head;
  const float* st_in = state + ((size_t)slots[seg] * 2 + phase[seg]) * half + h * per_head;
  float* st_out = state + ((size_t)slots[seg] * 2 + (1 - phase[seg])) * half + h * per_head;
  const int c_first = seg_chunk0[seg], c_end = seg_chunk0[seg + 1];
  const bool live = e < E;
  float m = st_in[E];
  float cur = live ? st_in[e] : 0.f;
  auto place = [&](int c) -> float* {
    return e < CE ? ws_C + ((size_t)c * H + h) * CE + e : ws_n + ((size_t)c * H + h) * dk + (e - CE);
  };
  float delta = (live && c_first < c_end) ? *place(c_first) : 0.f;
  for (int c = c_first; c < c_end; ++c) {
    const float here = delta;
    if (live && c + 1 < c_end) delta = *place(c + 1);  // (asked for before this chunk's place is written)
    const float top = ws_m[((size_t)c * H + h) * 2], bl = ws_m[((size_t)c * H + h) * 2 + 1];
    if (live) *place(c) = cur;
    if (e == 0) ws_m0[(size_t)c * H + h] = m;
    const float m_new = fmaxf(bl + m, top);
    cur = fmaf(expf(bl + m - m_new), cur, expf(top - m_new) * here);
    m = m_new;
  }
  if (live) st_out[e] = cur;
  if (e == 0) st_out[E] = m;
}

template <typename T>
__global__ __launch_bounds__(256) void mlstm_chunk_out_kernel(const T* __restrict__ rows, const float* __restrict__ gates,
                                                              const int* __restrict__ chunks,
                                                              const float* __restrict__ ws_C,
                                                              const float* __restrict__ ws_n,
                                                              const float* __restrict__ ws_m0, float* __restrict__ o_raw,
                                                              int H, int dk, int dv, float q_mul, float floor_) {
  extern __shared__ float lds[];
  const int chunk = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * kSlice;
  const int t0 = chunks[3 * chunk + 1], n = chunks[3 * chunk + 2];
  const int dkp = (dk + 15) & ~15, KS = dkp + kPad, VS = kSlice + kPad;
  const int width = 2 * H * dk + 2 * H * dv;
  double* s_a = reinterpret_cast<double*>(lds);  // [64] each
  double* s_b = s_a + kChunk;
  double* s_g = s_b + kChunk;
  float* sQ = lds + 6 * kChunk;      // [64][KS], times q_mul
  float* sK = sQ + kChunk * KS;      // [64][KS]
  float* sV = sK + kChunk * KS;      // [64][VS]
  float* sP = sV + kChunk * VS;      // [64][VS]: the weighted scores, query by key
  float* sC = sP + kChunk * VS;      // [dkp][VS]: the state in front of the chunk, this slice's columns
  float* s_n = sC + dkp * VS;        // [dkp]
  float* s_coef = s_n + dkp;         // [64] each
  float* s_rs = s_coef + kChunk;
  float* s_qn = s_rs + kChunk;
  const float m0 = ws_m0[(size_t)chunk * H + h];
  if (threadIdx.x < 64) {
    chunk_gates(gates, t0, n, H, h, s_a, s_b);
    const int lane = threadIdx.x;
    double top = s_a[lane];  // (the lane's own value, written by itself)
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const double u = __shfl_up(top, o, 64);
      if (lane >= o) top = fmax(top, u);
    }
    top = fmax(top, (double)m0);
    s_g[lane] = top;
    s_coef[lane] = expf((float)((double)m0 - top));
  }
  stage_rows<T>(rows, width, t0, n, h * dk, dk, dkp, KS, q_mul, sQ);
  stage_rows<T>(rows, width, t0, n, H * dk + h * dk, dk, dkp, KS, 1.0f, sK);
  stage_rows<T>(rows, width, t0, n, 2 * H * dk + h * dv + c0, min(kSlice, dv - c0), kSlice, VS, 1.0f, sV);
  const float* C0 = ws_C + ((size_t)chunk * H + h) * dk * dv;
  if (dv % 4 == 0) {  // (four columns a load: they are there together or not at all)
    for (int idx = threadIdx.x; idx < dkp * (kSlice / 4); idx += 256) {
      const int k = idx / (kSlice / 4), c = (idx - k * (kSlice / 4)) * 4;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (k < dk && c0 + c < dv) v = *reinterpret_cast<const f32x4*>(C0 + (size_t)k * dv + c0 + c);
      *reinterpret_cast<f32x4*>(sC + k * VS + c) = v;
    }
  } else {
    for (int idx = threadIdx.x; idx < dkp * kSlice; idx += 256) {
      const int k = idx / kSlice, c = idx - k * kSlice;
      sC[k * VS + c] = (k < dk && c0 + c < dv) ? C0[(size_t)k * dv + c0 + c] : 0.f;
    }
  }
  for (int k = threadIdx.x; k < dkp; k += 256) s_n[k] = k < dk ? ws_n[((size_t)chunk * H + h) * dk + k] : 0.f;
  __syncthreads();
  const int w = wave_index(), lane = threadIdx.x & 63, c16 = lane & 15, g = lane >> 4;
  if (16 * w >= n) return;  // (no token of the chunk in this wavefront's rows; no barrier follows that all must reach)
  // the weighted scores of this wavefront's 16 queries, key block by key block up to the diagonal
  float rowsum[4] = {0.f, 0.f, 0.f, 0.f};
  for (int kb = 0; kb <= w; ++kb) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int kk = 0; kk < dkp; kk += 4)
      acc = mma(sQ[(16 * w + c16) * KS + kk + g], sK[(16 * kb + c16) * KS + kk + g], acc);
    const int s = 16 * kb + c16;
    const double as = s_a[s];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int t = 16 * w + 4 * g + r;
      const float p = s <= t ? acc[r] * expf((float)(as - s_g[t])) : 0.f;
      sP[t * VS + s] = p;
      rowsum[r] += p;
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) rowsum[r] += __shfl_xor(rowsum[r], o, 64);
    if (c16 == 0) s_rs[16 * w + 4 * g + r] = rowsum[r];
  }
  {  // q . n of the state in front, for the query 16 w + c16
    float a = 0.f;
    for (int k = g; k < dkp; k += 4) a = fmaf(sQ[(16 * w + c16) * KS + k], s_n[k], a);
    a += __shfl_xor(a, 16, 64);
    a += __shfl_xor(a, 32, 64);
    if (g == 0) s_qn[16 * w + c16] = a;
  }
  // (sP's rows, s_rs and s_qn of this wavefront are written and read by itself: its own writes are waited for)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  f32x4 out[4];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct) out[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < 16 * (w + 1); s0 += 4) {
    const float a = sP[(16 * w + c16) * VS + s0 + g];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) out[ct] = mma(a, sV[(s0 + g) * VS + 16 * ct + c16], out[ct]);
  }
  const float cf = s_coef[16 * w + c16];
  for (int kk = 0; kk < dkp; kk += 4) {
    const float a = sQ[(16 * w + c16) * KS + kk + g] * cf;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) out[ct] = mma(a, sC[(kk + g) * VS + 16 * ct + c16], out[ct]);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = 16 * w + 4 * g + r;
    if (t >= n) continue;
    const float nq = fmaf(s_coef[t], s_qn[t], s_rs[t]);
    const float den = fmaxf(fabsf(nq), expf((float)(-(s_b[t] + s_g[t])))) + floor_;
    float* dst = o_raw + (size_t)(t0 + t) * H * dv + h * dv + c0;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
      const int c = 16 * ct + c16;
      if (c0 + c < dv) dst[c] = out[ct][r] / den;
    }
  }
}

namespace {
template <typename K>
int allow_lds(K kernel, size_t smem, size_t& allowed) {
  if (smem > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return (int)e;
    allowed = smem;
  }
  return 0;
}
}  // namespace

JLE_API int jle_mlstm_chunk_tokens() { return kChunk; }
JLE_API int jle_mlstm_chunked_supported(int dk, int dv) { return dk >= 1 && dk <= 128 && dv >= 1; }

// chunks: [num_chunks][3] = (segment, first row, rows <= 64), the chunks of a segment one after the other;
// seg_chunk0: [R + 1], where each segment's chunks begin.  ws_C: num_chunks * H * dk * dv floats, ws_n:
// num_chunks * H * dk, ws_m: num_chunks * H * 2, ws_m0: num_chunks * H.  Everything else as jle_mlstm.
JLE_API int jle_mlstm_chunked(const void* rows, int is_bf16, float* gates, const float* b_gates, const float* norm_w,
                              float* state, const int* slots, const int* phase, const int* chunks, int num_chunks,
                              const int* seg_chunk0, float* ws_C, float* ws_n, float* ws_m, float* ws_m0, float* o_raw,
                              void* out, int N, int R, int H, int dk, int dv, float cap, float eps, float floor_,
                              hipStream_t s) {
  if (N <= 0 || R <= 0) return 0;
  if (H < 1 || !jle_mlstm_chunked_supported(dk, dv) || !(cap > 0.f) || num_chunks < 0) return JLE_BAD_ARG;
  const long long total = (long long)N * 2 * H;
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gates, b_gates, cap, H,
                     total);
  JLE_LAUNCH_CHECK();
  const int dkp = (dk + 15) & ~15, KS = dkp + kPad, VS = kSlice + kPad;
  const int slices = (dv + kSlice - 1) / kSlice;
  const size_t smem_state = sizeof(float) * ((size_t)kChunk * KS + kChunk * VS + 5 * kChunk);
  const size_t smem_out = sizeof(float) * ((size_t)2 * kChunk * KS + 2 * kChunk * VS + (size_t)dkp * VS + dkp + 9 * kChunk);
  const float q_mul = 1.0f / sqrtf((float)dk);
  static size_t allowed[4] = {0, 0, 0, 0};
  if (num_chunks > 0) {
    const dim3 grid(num_chunks, H, slices);
    int rc;
    if (is_bf16) {
      if ((rc = allow_lds(&mlstm_chunk_state_kernel<bf16_t>, smem_state, allowed[0]))) return rc;
      hipLaunchKernelGGL(mlstm_chunk_state_kernel<bf16_t>, grid, dim3(256), smem_state, s, (const bf16_t*)rows, gates,
                         chunks, ws_C, ws_n, ws_m, H, dk, dv);
    } else {
      if ((rc = allow_lds(&mlstm_chunk_state_kernel<float>, smem_state, allowed[1]))) return rc;
      hipLaunchKernelGGL(mlstm_chunk_state_kernel<float>, grid, dim3(256), smem_state, s, (const float*)rows, gates,
                         chunks, ws_C, ws_n, ws_m, H, dk, dv);
    }
    JLE_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(mlstm_chunk_carry_kernel, dim3(R, H, (dk * dv + dk + 255) / 256), dim3(256), 0, s, state, slots,
                     phase, seg_chunk0, ws_C, ws_n, ws_m, ws_m0, H, dk, dv);
  JLE_LAUNCH_CHECK();
  if (num_chunks > 0) {
    const dim3 grid(num_chunks, H, slices);
    int rc;
    if (is_bf16) {
      if ((rc = allow_lds(&mlstm_chunk_out_kernel<bf16_t>, smem_out, allowed[2]))) return rc;
      hipLaunchKernelGGL(mlstm_chunk_out_kernel<bf16_t>, grid, dim3(256), smem_out, s, (const bf16_t*)rows, gates, chunks,
                         ws_C, ws_n, ws_m0, o_raw, H, dk, dv, q_mul, floor_);
    } else {
      if ((rc = allow_lds(&mlstm_chunk_out_kernel<float>, smem_out, allowed[3]))) return rc;
      hipLaunchKernelGGL(mlstm_chunk_out_kernel<float>, grid, dim3(256), smem_out, s, (const float*)rows, gates, chunks,
                         ws_C, ws_n, ws_m0, o_raw, H, dk, dv, q_mul, floor_);
    }
    JLE_LAUNCH_CHECK();
  }
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
