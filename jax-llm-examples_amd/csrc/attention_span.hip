// Queries and keys normed over the whole projection, then queries to their rows and keys and values to their pages.
//
// rows: [N][Hq dk] (queries only) or [N][Hq dk + Hk dk + Hk dv].  One RMS norm over all Hq dk queries of a token
// (weights wq of that size) and one over all its Hk dk keys (wk); the queries times 1 + attn_scale * ln(1 +
// floor((pos + 1) / floor_scale)) (floor_scale <= 0: no factor).  Heads are stored PD elements wide (PD >= dk, dv),
// zeros behind the real ones: q_out [N][Hq][PD]; pages [page][2][Hk][..]: keys [ps][PD], values [PD][ps].
// One block per token; statistics, weights and the factor in float32; sums of squares in an order that depends on the
// sizes only.
#include "common.h"

using namespace jle;

template <typename T>
__global__ __launch_bounds__(256) void span_prepare_kernel(const T* __restrict__ rows, T* __restrict__ q_out,
                                                           T* __restrict__ kv, const int* __restrict__ positions,
                                                           const int* __restrict__ slot_mapping,
                                                           const float* __restrict__ wq, const float* __restrict__ wk,
                                                           float eps, float floor_scale, float attn_scale, int Hq,
                                                           int Hk, int dk, int dv, int PD, int ps, int own_kv) {
  __shared__ float red[4];
  const size_t n = blockIdx.x;
  const int nq = Hq * dk, nk = Hk * dk, nv = Hk * dv;
  const int width = own_kv ? nq + nk + nv : nq;
  const T* r = rows + n * width;
  float ssq = 0.f, ssk = 0.f;
  for (int c = threadIdx.x; c < nq; c += 256) {
    const float v = Num<T>::load(r + c);
    ssq = fmaf(v, v, ssq);
  }
  const bool write = own_kv && kv != nullptr;
  if (write)
    for (int c = threadIdx.x; c < nk; c += 256) {
      const float v = Num<T>::load(r + nq + c);
      ssk = fmaf(v, v, ssk);
    }
  const float tq = block_sum<256>(ssq, red);
  float inv_q = 1.0f / sqrtf(tq / (float)nq + eps);
  if (floor_scale > 0.f)
    inv_q *= 1.0f + attn_scale * log1pf(floorf(((float)positions[n] + 1.0f) / floor_scale));
  T* qo = q_out + n * (size_t)Hq * PD;
  for (int c = threadIdx.x; c < Hq * PD; c += 256) {
    const int h = c / PD, d = c - h * PD;
    float v = 0.f;
    if (d < dk) v = Num<T>::load(r + h * dk + d) * wq[h * dk + d] * inv_q;
    Num<T>::store(qo + c, v);
  }
  if (!write) return;
  const float tk = block_sum<256>(ssk, red);
  const float inv_k = 1.0f / sqrtf(tk / (float)nk + eps);
  const int slot = slot_mapping[n];
  const int page = slot / ps, off = slot - page * ps;
  const size_t plane = (size_t)ps * PD;
  T* kpage = kv + (size_t)page * 2 * Hk * plane;
  T* vpage = kpage + (size_t)Hk * plane;
  for (int c = threadIdx.x; c < Hk * PD; c += 256) {
    const int h = c / PD, d = c - h * PD;
    float kx = 0.f, vx = 0.f;
    if (d < dk) kx = Num<T>::load(r + nq + h * dk + d) * wk[h * dk + d] * inv_k;
    if (d < dv) vx = Num<T>::load(r + nq + nk + h * dv + d);
    Num<T>::store(kpage + h * plane + (size_t)off * PD + d, kx);
    Num<T>::store(vpage + h * plane + (size_t)d * ps + off, vx);
  }
}

JLE_API int jle_span_prepare(const void* rows, void* q_out, void* kv, const int* positions, const int* slot_mapping,
                             const float* wq, const float* wk, float eps, float floor_scale, float attn_scale,
                             int is_bf16, int N, int Hq, int Hk, int dk, int dv, int PD, int ps, int own_kv,
                             hipStream_t s) {
  if (N <= 0) return 0;
  if (Hq < 1 || Hk < 1 || dk < 1 || dv < 1 || PD < dk || PD < dv || ps < 1 || wq == nullptr) return JLE_BAD_ARG;
  if (kv != nullptr && (!own_kv || wk == nullptr || slot_mapping == nullptr)) return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(span_prepare_kernel<bf16_t>, dim3(N), dim3(256), 0, s, (const bf16_t*)rows, (bf16_t*)q_out,
                       (bf16_t*)kv, positions, slot_mapping, wq, wk, eps, floor_scale, attn_scale, Hq, Hk, dk, dv, PD,
                       ps, own_kv);
  else
    hipLaunchKernelGGL(span_prepare_kernel<float>, dim3(N), dim3(256), 0, s, (const float*)rows, (float*)q_out,
                       (float*)kv, positions, slot_mapping, wq, wk, eps, floor_scale, attn_scale, Hq, Hk, dk, dv, PD, ps,
                       own_kv);
  JLE_LAUNCH_CHECK();
  return 0;
}

// rows[n][:] *= sigmoid(h32[n] . w): one number a token, the product and the sigmoid in float32.  One block per row.
template <typename T>
__global__ __launch_bounds__(256) void row_gate_kernel(T* __restrict__ rows, const float* __restrict__ h32,
                                                       const float* __restrict__ w, int K, int D) {
  __shared__ float red[4];
  const size_t n = blockIdx.x;
  float dot = 0.f;
  for (int c = threadIdx.x; c < K; c += 256) dot = fmaf(h32[n * K + c], w[c], dot);
  const float z = block_sum<256>(dot, red);
  const float gate = 1.0f / (1.0f + expf(-z));
  for (int d = threadIdx.x; d < D; d += 256) Num<T>::store(rows + n * D + d, Num<T>::load(rows + n * D + d) * gate);
}

JLE_API int jle_row_gate(void* rows, int is_bf16, const float* h32, const float* w, int N, int K, int D,
                         hipStream_t s) {
  if (N <= 0) return 0;
  if (K < 1 || D < 1) return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(row_gate_kernel<bf16_t>, dim3(N), dim3(256), 0, s, (bf16_t*)rows, h32, w, K, D);
  else
    hipLaunchKernelGGL(row_gate_kernel<float>, dim3(N), dim3(256), 0, s, (float*)rows, h32, w, K, D);
  JLE_LAUNCH_CHECK();
  return 0;
}
